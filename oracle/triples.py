"""Kept (l1, l2) -> l triples and their flat encodings (oracle; test infrastructure).

Restates CGNet/CGutils.py:73-187 and CGNet/CG_layers.py:253-262 of the reference.
A "pair list" is ``pairs[l] = [(l1, l2), ...]`` with l1 >= l2.
"""
import numpy as np


def default_pairs(lmax):
    """All 0 <= l2 <= l1 <= lmax with |l1-l2| <= l <= min(l1+l2, lmax)   (CGutils.py:112-119)."""
    pairs = [[] for _ in range(lmax + 1)]
    for l1 in range(lmax + 1):
        for l2 in range(l1 + 1):
            for l in range(l1 - l2, min(l1 + l2, lmax) + 1):
                pairs[l].append((l1, l2))
    return pairs


def debug_pairs(lmax):
    """First two pairs of every l in the default enumeration order   (CGutils.py:102-110)."""
    return [p[:2] for p in default_pairs(lmax)]


def mst_edges(l, lmax):
    """Edges {a<b} of the degree graph for output l with their weights   (CGutils.py:78-84)."""
    e = []
    for a in range(lmax + 1):
        for b in range(a + 1, lmax + 1):
            if b - a <= l <= a + b:
                e.append(((2 * l + 1) * (2 * a + 1) * (2 * b + 1), b, a))
    return e


def mst_pairs_scipy(l, lmax, diag=True):
    """The reference's own route: scipy's minimum_spanning_tree   (CGutils.py:73-98).

    scipy is a third-party dependency of the reference (no version pinned in
    its README); rows of the sparse matrix are the bigger degree, columns the smaller.
    """
    from scipy.sparse import csr_matrix
    from scipy.sparse.csgraph import minimum_spanning_tree
    e = mst_edges(l, lmax)
    w = [x[0] for x in e]
    big = [x[1] for x in e]
    small = [x[2] for x in e]
    g = csr_matrix((w, (big, small)), shape=(lmax + 1, lmax + 1))
    t = minimum_spanning_tree(g).tocoo()
    out = list(zip(t.row.tolist(), t.col.tolist()))
    if diag:
        out += [(a, a) for a in range(lmax + 1) if l <= 2 * a]
    return out


def mst_pairs_kruskal(l, lmax, diag=True):
    """Stable Kruskal with edges ordered by (weight, bigger, smaller); output in row-major
    (bigger, smaller) order like a COO view of a CSR matrix, then the diagonal pairs."""
    parent = list(range(lmax + 1))

    def find(x):
        while parent[x] != x:
            parent[x] = parent[parent[x]]
            x = parent[x]
        return x

    kept = []
    for (w, b, a) in sorted(mst_edges(l, lmax)):
        ra, rb = find(a), find(b)
        if ra != rb:
            parent[ra] = rb
            kept.append((b, a))
    kept.sort()
    if diag:
        kept += [(a, a) for a in range(lmax + 1) if l <= 2 * a]
    return kept


def mst_pairs(lmax, use_scipy=True):
    f = mst_pairs_scipy if use_scipy else mst_pairs_kruskal
    return [f(l, lmax, True) for l in range(lmax + 1)]


def encode_sorted(pairs):
    """llls codes ((l*(L+1)+l1)*(L+1)+l2), per l stably sorted by l1, and the flat
    (L+1)x(L+2) table "index of the first triple of l whose l1 >= column"   (CGutils.py:121-140)."""
    lmax = len(pairs) - 1
    n1 = lmax + 1
    codes = []
    first = np.zeros((n1, n1 + 1), dtype=np.int64)
    for l in range(n1):
        ordered = sorted(pairs[l], key=lambda p: p[0])
        for (l1, l2) in ordered:
            if l1 < l2:
                raise AssertionError("pairs must have l1 >= l2")
        base = len(codes)
        cnt = np.zeros(n1, dtype=np.int64)
        for (l1, l2) in ordered:
            codes.append((l * n1 + l1) * n1 + l2)
            cnt[l1] += 1
        first[l, 0] = base
        first[l, 1:] = base + np.cumsum(cnt)
    return codes, first.reshape(-1)


def decode(lmax, codes):
    """[(l, l1, l2), ...]   (CGutils.py:142-151)."""
    n1 = lmax + 1
    return [(c // (n1 * n1), (c // n1) % n1, c % n1) for c in codes]


def cg_table_offsets(lmax, codes):
    """Cumulative (2l+1)(2l2+1), length len(codes)+1   (CGutils.py:153-158,179-187)."""
    offs = [0]
    for (l, l1, l2) in decode(lmax, codes):
        offs.append(offs[-1] + (2 * l + 1) * (2 * l2 + 1))
    return offs


def product_taus(lmax, codes, taus):
    """t_FF[l] and the per-triple channel offset inside degree l   (CG_layers.py:253-262)."""
    t_ff = [0] * (lmax + 1)
    t_off = []
    for (l, l1, l2) in decode(lmax, codes):
        t_off.append(t_ff[l])
        t_ff[l] += int(taus[l1]) * int(taus[l2])
    return t_ff, t_off


def cumulative_tm(taus):
    """[0, cumsum(tau[l]*(2l+1))]   (CG_layers.py:86,96,219,242)."""
    out = [0]
    for l, t in enumerate(taus):
        out.append(out[-1] + int(t) * (2 * l + 1))
    return out


def cumulative_w(t_ff, t_out):
    """[0, cumsum(t_FF[l]*t_O[l])]   (CG_layers.py:98)."""
    out = [0]
    for a, b in zip(t_ff, t_out):
        out.append(out[-1] + int(a) * int(b))
    return out
