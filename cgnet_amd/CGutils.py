"""Host-side metadata of the Clebsch-Gordan layer: which (l1, l2) -> l triples are kept,
their flat encodings and offsets, Clebsch-Gordan tables, and fragment reshaping helpers.

Public names, argument meaning and return layouts follow the reference's
``CGNet/CGutils.py`` (``compute_MST`` :73-98, ``SparseLtuples`` :101-187,
``reshape_out`` :190-197, ``Complex_bmm`` :15-21, ``calc_prod_taus`` :33-41,
``ClebschGordanDict`` :49-70) so that code written against the reference keeps working.
Everything here is integer / float64 bookkeeping done once per layer on the host.
"""
import math

import numpy as np
import torch

REAL_PART, IMAG_PART = 0, 1


# --------------------------------------------------------------------------- complex helpers
def Complex_bmm(w, f):
    """Batched complex matrix product of (B, M, K, 2) with (B, K, N, 2)."""
    a = torch.view_as_complex(w.contiguous())
    b = torch.view_as_complex(f.contiguous())
    return torch.view_as_real(torch.bmm(a, b))


def Complex_mm(w, f):
    """Batched complex matrix product of (B, M, K) x (B, K, N) tensors with a trailing (re, im) axis."""
    return torch.view_as_real(torch.bmm(torch.view_as_complex(w.contiguous()),
                                        torch.view_as_complex(f.contiguous())))


def calc_prod_taus(lmax, taus, taus2=None):
    """Number of degree-l channels produced by the full half-pair CG product of taus x taus2."""
    taus2 = taus if taus2 is None else taus2
    if not (len(taus) == len(taus2) == lmax + 1):
        raise AssertionError("taus must have lmax+1 entries")
    n = [0] * (lmax + 1)
    for l1 in range(lmax + 1):
        for l2 in range(l1 + 1):
            for l in range(l1 - l2, min(l1 + l2, lmax) + 1):
                n[l] += int(taus[l1]) * int(taus2[l2])
    return n


def reshape_out(output, taus):
    """Straight tensor (B, sum tau[l](2l+1), 2) -> list of views (B, tau[l], 2l+1, 2)."""
    total = sum((2 * l + 1) * int(t) for l, t in enumerate(taus))
    if total != output.shape[1]:
        raise AssertionError("taus do not match the tensor: %d != %d" % (total, output.shape[1]))
    pieces, start = [], 0
    for l, t in enumerate(taus):
        width = (2 * l + 1) * int(t)
        pieces.append(output[:, start:start + width, :].view(output.shape[0], int(t), 2 * l + 1, 2))
        start += width
    return pieces


# --------------------------------------------------------------------------- CG coefficients (host, float64)
_LOGFACT = np.zeros(2, dtype=np.float64)


def _logfact_table(nmax):
    global _LOGFACT
    if _LOGFACT.shape[0] <= nmax:
        t = np.zeros(nmax + 64, dtype=np.float64)
        t[2:] = np.cumsum(np.log(np.arange(2, nmax + 64, dtype=np.float64)))
        _LOGFACT = t
    return _LOGFACT


def clebsch_gordan(l1, m1, l2, m2, l, m):
    """Condon-Shortley <l1 m1 l2 m2 | l m> by the Racah sum with float64 log-factorials
    (the quantity of the reference's ClebschGordan.cpp:360-394 / cudaCG_sparse.cu:33-57)."""
    if m1 + m2 != m or abs(m1) > l1 or abs(m2) > l2 or abs(m) > l or not (abs(l1 - l2) <= l <= l1 + l2):
        return 0.0
    lf = _logfact_table(l1 + l2 + l + 2)
    head = 0.5 * (math.log(2 * l + 1.0) + lf[l + l1 - l2] + lf[l - l1 + l2] + lf[l1 + l2 - l] - lf[l1 + l2 + l + 1]
                  + lf[l + m] + lf[l - m] + lf[l1 - m1] + lf[l1 + m1] + lf[l2 - m2] + lf[l2 + m2])
    lo = max(0, l2 - m1 - l, l1 + m2 - l)
    hi = min(l1 + l2 - l, l1 - m1, l2 + m2)
    total = 0.0
    for k in range(lo, hi + 1):
        tail = (lf[k] + lf[l1 + l2 - l - k] + lf[l1 - m1 - k] + lf[l2 + m2 - k]
                + lf[l - l2 + m1 + k] + lf[l - l1 - m2 + k])
        term = math.exp(head - tail)
        total += -term if (k & 1) else term
    return total


def _cg_matrix_f64(l1, l2, l):
    """(2l+1, (2l1+1)(2l2+1)) float64, entry [m+l, (m1+l1)(2l2+1)+(m2+l2)]."""
    out = np.zeros((2 * l + 1, (2 * l1 + 1) * (2 * l2 + 1)), dtype=np.float64)
    for m1 in range(-l1, l1 + 1):
        for m2 in range(-l2, l2 + 1):
            m = m1 + m2
            if -l <= m <= l:
                out[m + l, (m1 + l1) * (2 * l2 + 1) + (m2 + l2)] = clebsch_gordan(l1, m1, l2, m2, l, m)
    return out


class ClebschGordanDict:
    """Dictionary of float32 CG matrices keyed ``l + (lmax+1)*(l2 + (lmax+1)*l1)``,
    built lazily (the reference precomputes every admissible (l1, l2, l))."""

    def __init__(self, lmax, cudaFlag=False):
        self.lmax = lmax
        self.Dict = {}

    def _key(self, l1, l2, l):
        return l + (self.lmax + 1) * (l2 + (self.lmax + 1) * l1)

    def getCGmat(self, l1, l2, l):
        if max(l1, l2, l) > self.lmax or not (abs(l1 - l2) <= l <= l1 + l2):
            return None
        k = self._key(l1, l2, l)
        if k not in self.Dict:
            self.Dict[k] = torch.from_numpy(_cg_matrix_f64(l1, l2, l)).float()
        return self.Dict[k]

    def getEntry(self, l1, l2, l, m1, m2, m):
        mat = self.getCGmat(l1, l2, l)
        if mat is None:
            return None
        return mat[m + l, (m1 + l1) * (2 * l2 + 1) + (m2 + l2)]


# --------------------------------------------------------------------------- MST pair selection
def compute_MST(l, lmax, diag=False):
    """Minimum spanning tree of the degree graph of output degree l (Cobb et al. reduction).

    Nodes 0..lmax; an edge joins a < b iff b - a <= l <= a + b, with weight
    (2l+1)(2a+1)(2b+1).  Returns (l1s, l2s) with l1 > l2 for tree edges; ``diag`` appends
    (a, a) for every a with l <= 2a.  The tree is found by Kruskal's algorithm over edges
    ordered by (weight, bigger, smaller) and reported in (bigger, smaller) lexicographic
    order, which reproduces what scipy's ``minimum_spanning_tree`` (used by the reference)
    returns for these graphs, ties included.
    """
    edges = [((2 * l + 1) * (2 * a + 1) * (2 * b + 1), b, a)
             for a in range(lmax + 1) for b in range(a + 1, lmax + 1) if b - a <= l <= a + b]
    edges.sort()
    root = list(range(lmax + 1))

    def find(x):
        while root[x] != x:
            root[x] = root[root[x]]
            x = root[x]
        return x

    tree = []
    for _, b, a in edges:
        ra, rb = find(a), find(b)
        if ra != rb:
            root[ra] = rb
            tree.append((b, a))
    tree.sort()
    l1s = [p[0] for p in tree]
    l2s = [p[1] for p in tree]
    if diag:
        same = [a for a in range(lmax + 1) if l <= 2 * a]
        l1s += same
        l2s += same
    return l1s, l2s


# --------------------------------------------------------------------------- triple lists
class SparseLtuples:
    """Builders for ``ltuples`` (``ltuples[l]`` = list of (l1, l2), l1 >= l2) and their flat forms."""

    @classmethod
    def compute_default_ltuples(cls, lmax):
        """Every l2 <= l1 with |l1 - l2| <= l <= min(l1 + l2, lmax); per l in (l1, l2) ascending order."""
        return [[(l1, l2) for l1 in range(lmax + 1) for l2 in range(l1 + 1)
                 if l1 - l2 <= l <= l1 + l2] for l in range(lmax + 1)]

    @classmethod
    def compute_debug_ltuples(cls, lmax):
        """The first two pairs of every degree of the default list."""
        return [pairs[:2] for pairs in cls.compute_default_ltuples(lmax)]

    @classmethod
    def compute_mst_ltuples(cls, lmax):
        out = []
        for l in range(lmax + 1):
            l1s, l2s = compute_MST(l, lmax, diag=True)
            out.append(list(zip(l1s, l2s)))
        return out

    @classmethod
    def sparse_rep_ltuples_sorted(cls, ltuples):
        """-> (llls, l_l1_to_lllidx_offsets).

        ``llls`` holds ``(l*(lmax+1)+l1)*(lmax+1)+l2`` per kept triple, ordered by l and,
        inside one l, stably by l1.  The second value is a flat (lmax+1) x (lmax+2) int
        table whose entry [l, a] is the index in ``llls`` of the first triple of degree l
        with l1 >= a (entry [l, lmax+1] = one past the last triple of l).
        """
        n1 = len(ltuples)
        llls = []
        table = np.zeros((n1, n1 + 1), dtype=np.int64)
        for l, pairs in enumerate(ltuples):
            pairs = [(int(a), int(b)) for a, b in pairs]
            if any(a < b for a, b in pairs):
                raise AssertionError("every pair must satisfy l1 >= l2")
            order = sorted(range(len(pairs)), key=lambda i: pairs[i][0])
            start = len(llls)
            per_l1 = np.zeros(n1, dtype=np.int64)
            for i in order:
                a, b = pairs[i]
                llls.append((l * n1 + a) * n1 + b)
                per_l1[a] += 1
            table[l, 0] = start
            table[l, 1:] = start + np.cumsum(per_l1)
        return llls, table.reshape(-1)

    @classmethod
    def get_iter(cls, lmax, llls):
        """Decoded [(l, l1, l2), ...]."""
        n1 = lmax + 1
        return [(int(c) // (n1 * n1), (int(c) // n1) % n1, int(c) % n1) for c in llls]

    @classmethod
    def get_CG_length(cls, lmax, llls):
        return int(sum((2 * l + 1) * (2 * l2 + 1) for l, _, l2 in cls.get_iter(lmax, llls)))

    @classmethod
    def cal_CG_offsets(cls, lmax, llls):
        """Start of every triple's (2l+1) x (2l2+1) table, plus the total length as last entry."""
        sizes = [(2 * l + 1) * (2 * l2 + 1) for l, _, l2 in cls.get_iter(lmax, llls)]
        return [0] + np.cumsum(np.asarray(sizes, dtype=np.int64)).tolist() if sizes else [0]

    @classmethod
    def precompute_CG_from_llls(cls, lmax, llls):
        """Host (CPU tensor) version of the flat table: entry [m+l][m2+l2] of triple i is
        C(l1, m-m2; l2, m2 | l, m), zero when |m - m2| > l1."""
        chunks = []
        for l, l1, l2 in cls.get_iter(lmax, llls):
            t = np.zeros((2 * l + 1, 2 * l2 + 1), dtype=np.float64)
            for m in range(-l, l + 1):
                for m2 in range(-l2, l2 + 1):
                    if abs(m - m2) <= l1:
                        t[m + l, m2 + l2] = clebsch_gordan(l1, m - m2, l2, m2, l, m)
            chunks.append(t.reshape(-1))
        flat = np.concatenate(chunks) if chunks else np.zeros(0)
        return torch.from_numpy(flat).float()
