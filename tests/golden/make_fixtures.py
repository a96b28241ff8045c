"""Writes the committed fixtures in this directory.  Run from the repository root:

    python tests/golden/make_fixtures.py

* cg_sympy.json   Clebsch-Gordan coefficients from sympy (sympy.physics.quantum.cg.CG,
                  exact symbolic evaluation, then evalf to 30 digits): every non-zero entry
                  with l1, l2, l <= 4 and a seeded random sample of entries at higher degrees
                  (up to 20).  sympy is independent of both the reference and this build.
* mst_scipy.json  For L in {3, 4, 8, 11, 15, 20}: per output degree l, the (l1, l2) pairs that
                  scipy.sparse.csgraph.minimum_spanning_tree keeps on the reference's degree
                  graph (edge {a<b} iff b-a <= l <= a+b, weight (2l+1)(2a+1)(2b+1), matrix rows =
                  bigger degree), in COO order, followed by the diagonal pairs (a, a), l <= 2a.
                  scipy is a third-party dependency of the reference; the fixture records its
                  version.  No reference code is imported or executed.
"""
import json
import os
import random

HERE = os.path.dirname(os.path.abspath(__file__))


def sympy_cg(l1, m1, l2, m2, l, m):
    from sympy import S
    from sympy.physics.quantum.cg import CG
    return float(CG(S(l1), S(m1), S(l2), S(m2), S(l), S(m)).doit().evalf(30))


def make_cg():
    rows = []
    for l1 in range(5):
        for l2 in range(5):
            for l in range(abs(l1 - l2), min(l1 + l2, 4) + 1):
                for m1 in range(-l1, l1 + 1):
                    for m2 in range(-l2, l2 + 1):
                        m = m1 + m2
                        if abs(m) <= l:
                            rows.append([l1, m1, l2, m2, l, m, sympy_cg(l1, m1, l2, m2, l, m)])
    rng = random.Random(20181203)
    for lmax in (6, 11, 15, 20):
        for _ in range(40):
            l1 = rng.randint(0, lmax)
            l2 = rng.randint(0, l1)
            l = rng.randint(l1 - l2, min(l1 + l2, lmax))
            m1 = rng.randint(-l1, l1)
            lo, hi = max(-l2, -l - m1), min(l2, l - m1)
            if lo > hi:
                continue
            m2 = rng.randint(lo, hi)
            rows.append([l1, m1, l2, m2, l, m1 + m2, sympy_cg(l1, m1, l2, m2, l, m1 + m2)])
    import sympy
    with open(os.path.join(HERE, "cg_sympy.json"), "w") as fh:
        json.dump({"source": "sympy.physics.quantum.cg.CG", "sympy": sympy.__version__,
                   "columns": ["l1", "m1", "l2", "m2", "l", "m", "value"], "rows": rows}, fh)
    print("cg_sympy.json:", len(rows), "entries")


def make_mst():
    import scipy
    from scipy.sparse import csr_matrix
    from scipy.sparse.csgraph import minimum_spanning_tree
    out = {"source": "scipy.sparse.csgraph.minimum_spanning_tree", "scipy": scipy.__version__, "lmax": {}}
    for lmax in (3, 4, 8, 11, 15, 20):
        per_l = []
        for l in range(lmax + 1):
            big, small, w = [], [], []
            for a in range(lmax + 1):
                for b in range(a + 1, lmax + 1):
                    if b - a <= l <= a + b:
                        small.append(a)
                        big.append(b)
                        w.append((2 * l + 1) * (2 * a + 1) * (2 * b + 1))
            tree = minimum_spanning_tree(csr_matrix((w, (big, small)), shape=(lmax + 1, lmax + 1))).tocoo()
            pairs = [[int(r), int(c)] for r, c in zip(tree.row, tree.col)]
            pairs += [[a, a] for a in range(lmax + 1) if l <= 2 * a]
            per_l.append(pairs)
        out["lmax"][str(lmax)] = per_l
        print("mst L=%d: %d triples" % (lmax, sum(len(p) for p in per_l)))
    with open(os.path.join(HERE, "mst_scipy.json"), "w") as fh:
        json.dump(out, fh)


if __name__ == "__main__":
    make_mst()
    make_cg()
