"""Clebsch-Gordan coefficients <l1 m1 l2 m2 | l m> on the CPU (oracle; test infrastructure).

Follows the Racah closed form that the reference evaluates with log-factorials in
CGNet/ClebschGordan/ClebschGordan.cpp:360-394 (device twin
CGNet/cudaCG/cudaCG_sparse.cu:33-57).  There the two sign factors
(-1)^(l1-l2-m3) and (-1)^(l1-l2+m) multiply to +1 (m3 = -m) and sqrt(2l+1) is folded
into the prefactor, so the value is the standard Condon-Shortley coefficient

    C = delta(m, m1+m2)
        * sqrt( (2l+1) (l+l1-l2)! (l-l1+l2)! (l1+l2-l)! / (l1+l2+l+1)! )
        * sqrt( (l+m)! (l-m)! (l1-m1)! (l1+m1)! (l2-m2)! (l2+m2)! )
        * sum_k (-1)^k / ( k! (l1+l2-l-k)! (l1-m1-k)! (l2+m2-k)! (l-l2+m1+k)! (l-l1-m2+k)! )

Two evaluations are kept on purpose: ``cg_exact`` (big-integer rational arithmetic,
one entry at a time, no rounding until the final square root) and ``cg_block`` /
``cg_matrix`` / ``flat_cg_table`` (vectorised float64 log-factorials, the algorithm
of the reference).  Tests pin the first to sympy and the second to the first.
"""
from fractions import Fraction
from math import factorial, isqrt

import numpy as np


def cg_exact(l1, m1, l2, m2, l, m):
    """Exact-rational Racah sum, rounded once to float64."""
    if m != m1 + m2 or abs(m1) > l1 or abs(m2) > l2 or abs(m) > l:
        return 0.0
    if l < abs(l1 - l2) or l > l1 + l2:
        return 0.0
    f = factorial
    k_lo = max(0, l2 - m1 - l, l1 + m2 - l)
    k_hi = min(l1 + l2 - l, l1 - m1, l2 + m2)
    s = Fraction(0)
    for k in range(k_lo, k_hi + 1):
        den = (f(k) * f(l1 + l2 - l - k) * f(l1 - m1 - k) * f(l2 + m2 - k)
               * f(l - l2 + m1 + k) * f(l - l1 - m2 + k))
        s += Fraction(-1 if k & 1 else 1, den)
    if s == 0:
        return 0.0
    pref = Fraction((2 * l + 1) * f(l + l1 - l2) * f(l - l1 + l2) * f(l1 + l2 - l), f(l1 + l2 + l + 1))
    pref *= f(l + m) * f(l - m) * f(l1 - m1) * f(l1 + m1) * f(l2 - m2) * f(l2 + m2)
    sq = pref * s * s                      # C^2 as an exact rational
    # sqrt(num/den) with 80 extra bits so the single final rounding is the only one
    shift = 160
    num = sq.numerator << shift
    root = isqrt(num // sq.denominator)
    val = float(Fraction(root, 1 << (shift // 2)))
    return val if s > 0 else -val


def _logfact(nmax):
    t = np.zeros(nmax + 2, dtype=np.float64)
    t[2:] = np.cumsum(np.log(np.arange(2, nmax + 2, dtype=np.float64)))
    return t  # t[n] = log(n!)


def cg_block(l1, l2, l):
    """Dense float64 array C[m1+l1, m2+l2, m+l] for one (l1, l2, l) by log-factorials."""
    out = np.zeros((2 * l1 + 1, 2 * l2 + 1, 2 * l + 1), dtype=np.float64)
    if l < abs(l1 - l2) or l > l1 + l2:
        return out
    lf = _logfact(2 * (l1 + l2 + l) + 4)
    m1 = np.arange(-l1, l1 + 1)[:, None]
    m2 = np.arange(-l2, l2 + 1)[None, :]
    m = m1 + m2
    ok = np.abs(m) <= l
    mc = np.where(ok, m, 0)
    log_a = 0.5 * (np.log(2.0 * l + 1.0) + lf[l + l1 - l2] + lf[l - l1 + l2] + lf[l1 + l2 - l] - lf[l1 + l2 + l + 1])
    log_a = log_a + 0.5 * (lf[l + mc] + lf[l - mc] + lf[l1 - m1] + lf[l1 + m1] + lf[l2 - m2] + lf[l2 + m2])
    acc = np.zeros(m.shape, dtype=np.float64)
    for k in range(0, l1 + l2 - l + 1):
        a = [k + 0 * mc, l1 + l2 - l - k + 0 * mc, l1 - m1 - k + 0 * mc, l2 + m2 - k + 0 * mc,
             l - l2 + m1 + k + 0 * mc, l - l1 - m2 + k + 0 * mc]
        valid = ok.copy()
        for x in a:
            valid &= (x >= 0)
        log_b = sum(lf[np.where(valid, x, 0)] for x in a)
        term = np.exp(log_a - log_b)
        acc += np.where(valid, -term if k & 1 else term, 0.0)
    i1, i2 = np.nonzero(ok)
    out[i1, i2, (m[i1, i2] + l)] = acc[i1, i2]
    return out


def cg_matrix(l1, l2, l, dtype=np.float64):
    """Matrix of shape (2l+1, (2l1+1)(2l2+1)), entry [m+l, (m1+l1)(2l2+1)+(m2+l2)].

    This is the layout of the dictionary values built at
    CGNet/ClebschGordan/CGmodule.cpp:70-119 (consumed at CGNet/CGutils.py:57-70).
    """
    blk = cg_block(l1, l2, l)                         # [m1, m2, m]
    mat = blk.reshape((2 * l1 + 1) * (2 * l2 + 1), 2 * l + 1).T
    return np.ascontiguousarray(mat).astype(dtype)


def flat_cg_table(triples, dtype=np.float32):
    """Flat per-triple table; triple i owns (2l+1)(2l2+1) entries [m+l][m2+l2] = C(l1,m-m2;l2,m2|l,m).

    Entries whose m1 = m - m2 falls outside [-l1, l1] are zero.  Layout of
    CGNet/cudaCG/cudaCG_sparse.cu:68-92 and CGNet/CGutils.py:160-177.
    Returns (table, offsets) with len(offsets) = len(triples) + 1.
    """
    offs = [0]
    chunks = []
    for (l, l1, l2) in triples:
        blk = cg_block(l1, l2, l)                     # [m1, m2, m]
        mm = np.arange(2 * l + 1)[:, None]
        mm2 = np.arange(2 * l2 + 1)[None, :]
        i1 = (mm - l) - (mm2 - l2) + l1               # index of m1 = m - m2
        inside = (i1 >= 0) & (i1 <= 2 * l1)
        t = np.where(inside, blk[np.clip(i1, 0, 2 * l1), mm2, mm], 0.0)
        chunks.append(t.reshape(-1))
        offs.append(offs[-1] + t.size)
    table = np.concatenate(chunks) if chunks else np.zeros(0)
    return table.astype(dtype), np.asarray(offs, dtype=np.int64)
