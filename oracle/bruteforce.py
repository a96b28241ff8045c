"""Dense, loop-level definitions used only to pin the oracle on tiny inputs (test infrastructure).

Nothing here shares code with ``cg_layer``: coefficients come from ``cg_coeff.cg_exact`` one
entry at a time and the contractions are explicit Python loops over complex numbers.
"""
import numpy as np

from . import cg_coeff


def dense_cg(l1, l2, l):
    c = np.zeros((2 * l1 + 1, 2 * l2 + 1, 2 * l + 1))
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            m = m1 + m2
            if abs(m) <= l:
                c[m1 + l1, m2 + l2, m + l] = cg_coeff.cg_exact(l1, m1, l2, m2, l, m)
    return c


def cg_product_loops(fs_complex, triples_list, taus):
    """fs_complex[l]: complex ndarray (B, tau, 2l+1).  Returns list over l of complex
    (B, t_FF[l], 2l+1) with channels ordered by triple, then t1*tau2+t2."""
    lmax = len(fs_complex) - 1
    bsz = fs_complex[0].shape[0]
    out = [[] for _ in range(lmax + 1)]
    for (l, l1, l2) in triples_list:
        c = dense_cg(l1, l2, l)
        blk = np.zeros((bsz, taus[l1] * taus[l2], 2 * l + 1), dtype=np.complex128)
        for b in range(bsz):
            for t1 in range(taus[l1]):
                for t2 in range(taus[l2]):
                    for m1 in range(2 * l1 + 1):
                        for m2 in range(2 * l2 + 1):
                            mm = (m1 - l1) + (m2 - l2) + l
                            if 0 <= mm <= 2 * l:
                                blk[b, t1 * taus[l2] + t2, mm] += (c[m1, m2, mm] * fs_complex[l1][b, t1, m1]
                                                                   * fs_complex[l2][b, t2, m2])
        out[l].append(blk)
    return [np.concatenate(o, axis=1) if o else np.zeros((bsz, 0, 2 * l + 1), complex) for l, o in enumerate(out)]


def wigner_small_d(l, beta):
    """d^l_{m' m}(beta) by Wigner's explicit sum (z-y-z convention), index [m'+l, m+l]."""
    from math import factorial as f, cos, sin, sqrt
    d = np.zeros((2 * l + 1, 2 * l + 1))
    cb, sb = cos(beta / 2), sin(beta / 2)
    for mp in range(-l, l + 1):
        for m in range(-l, l + 1):
            pre = sqrt(f(l + mp) * f(l - mp) * f(l + m) * f(l - m))
            s = 0.0
            for k in range(max(0, m - mp), min(l + m, l - mp) + 1):
                den = f(l + m - k) * f(k) * f(mp - m + k) * f(l - mp - k)
                s += (-1) ** (mp - m + k) * cb ** (2 * l + m - mp - 2 * k) * sb ** (mp - m + 2 * k) / den
            d[mp + l, m + l] = pre * s
    return d


def wigner_D(l, alpha, beta, gamma):
    """D^l_{m' m}(alpha, beta, gamma) = exp(-i m' alpha) d^l_{m' m}(beta) exp(-i m gamma)."""
    m = np.arange(-l, l + 1)
    return np.exp(-1j * m[:, None] * alpha) * wigner_small_d(l, beta) * np.exp(-1j * m[None, :] * gamma)
