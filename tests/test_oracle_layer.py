"""Pins the oracle's layer arithmetic (oracle/cg_layer.py): CG product against a dense loop
definition, closed-form special cases and rotation equivariance; fragment norm against the
numpy closed form; weight mixing against a complex einsum; gradients by gradcheck."""
import math

import numpy as np
import pytest
import torch

from oracle import bruteforce as BF
from oracle import cg_coeff as C
from oracle import cg_layer as O
from oracle import triples as T


def rand_fragments(taus, bsz, seed, dtype=torch.float64, scale=False):
    g = torch.Generator().manual_seed(seed)
    out = []
    for l, t in enumerate(taus):
        x = torch.randn(bsz, t, 2 * l + 1, 2, generator=g, dtype=torch.float64)
        if scale:
            x = x / math.sqrt(2 * l + 1)
        out.append(x.to(dtype))
    return out


def to_complex(fs):
    return [f[..., 0].numpy().astype(np.complex128) + 1j * f[..., 1].numpy() for f in fs]


@pytest.mark.parametrize("mode", ["default", "mst", "debug"])
def test_cg_product_matches_dense_loops(mode):
    lmax, taus, bsz = 3, [2, 1, 2, 3], 2
    pairs = {"default": T.default_pairs, "mst": lambda L: T.mst_pairs(L, False), "debug": T.debug_pairs}[mode](lmax)
    codes, _ = T.encode_sorted(pairs)
    fs = rand_fragments(taus, bsz, 1)
    got = O.cg_product(fs, lmax, codes, taus)
    # exact (non-rounded) coefficients in the loop definition -> allow the float32 rounding of the table
    want = BF.cg_product_loops(to_complex(fs), T.decode(lmax, codes), taus)
    t_ff, _ = T.product_taus(lmax, codes, taus)
    for l in range(lmax + 1):
        assert got[l].shape == (bsz, t_ff[l], 2 * l + 1, 2)
        g = got[l][..., 0].numpy() + 1j * got[l][..., 1].numpy()
        assert np.max(np.abs(g - want[l])) < 5e-7 * max(1.0, np.max(np.abs(want[l])))


def test_cg_product_scalar_partner_and_invariant():
    lmax, taus, bsz = 4, [3, 2, 2, 1, 2], 3
    codes, _ = T.encode_sorted(T.default_pairs(lmax))
    trip = T.decode(lmax, codes)
    _, t_off = T.product_taus(lmax, codes, taus)
    fs = rand_fragments(taus, bsz, 2)
    fc = to_complex(fs)
    got = O.cg_product(fs, lmax, codes, taus)
    for (l, l1, l2), off in zip(trip, t_off):
        blk = got[l][:, off:off + taus[l1] * taus[l2]]
        blk = (blk[..., 0].numpy() + 1j * blk[..., 1].numpy()).reshape(bsz, taus[l1], taus[l2], 2 * l + 1)
        if l2 == 0:
            # coupling with a scalar: C = 1, FF[t1, t2, m] = F_l1[t1, m] * F_0[t2, 0]
            want = fc[l1][:, :, None, :] * fc[0][:, None, :, 0:1]
            assert np.allclose(blk, want, atol=1e-6)
        if l == 0:
            # invariant: sum_m (-1)^(l1-m) / sqrt(2 l1 + 1) F[m] F'[-m]
            m = np.arange(-l1, l1 + 1)
            sign = ((-1.0) ** (l1 - m)) / math.sqrt(2 * l1 + 1)
            want = np.einsum("m,btm,bsm->bts", sign, fc[l1], fc[l2][:, :, ::-1])[..., None]
            assert np.allclose(blk, want, atol=1e-6)


def test_wigner_d_known_values_and_unitarity():
    b = 0.7
    d1 = BF.wigner_small_d(1, b)
    assert d1[1, 1] == pytest.approx(math.cos(b))
    assert d1[2, 1] == pytest.approx(-math.sin(b) / math.sqrt(2))
    assert d1[2, 2] == pytest.approx((1 + math.cos(b)) / 2)
    for l in (2, 5):
        D = BF.wigner_D(l, 0.3, 1.1, -2.0)
        assert np.allclose(D @ D.conj().T, np.eye(2 * l + 1), atol=1e-12)
        # composition of rotations about z
        assert np.allclose(BF.wigner_D(l, 0.3, 0, 0) @ BF.wigner_D(l, 0.5, 0, 0), BF.wigner_D(l, 0.8, 0, 0))


@pytest.mark.parametrize("mode", ["default", "mst"])
def test_cg_product_rotation_equivariance(mode):
    # the identity the reference's write-up lists (ClebschGordan/description.tex:60-80):
    # rotating every input fragment by D^l rotates every output fragment by D^l
    lmax, taus, bsz = 5, [2, 2, 1, 2, 1, 2], 2
    pairs = T.default_pairs(lmax) if mode == "default" else T.mst_pairs(lmax, False)
    codes, _ = T.encode_sorted(pairs)
    fs = rand_fragments(taus, bsz, 3)
    ang = (0.4, 1.3, -0.9)
    Ds = [BF.wigner_D(l, *ang) for l in range(lmax + 1)]

    def rotate(parts):
        out = []
        for l, f in enumerate(parts):
            z = f[..., 0].numpy() + 1j * f[..., 1].numpy()
            z = np.einsum("pm,btm->btp", Ds[l], z)
            out.append(torch.from_numpy(np.stack([z.real, z.imag], -1)))
        return out

    a = rotate(O.cg_product(fs, lmax, codes, taus))
    b = O.cg_product(rotate(fs), lmax, codes, taus)
    for l in range(lmax + 1):
        assert torch.allclose(a[l], b[l], atol=2e-6), l


def test_straight_and_list_inputs_agree():
    lmax, taus = 3, [2, 2, 2, 2]
    codes, _ = T.encode_sorted(T.default_pairs(lmax))
    fs = rand_fragments(taus, 4, 0)
    a = O.cg_product(fs, lmax, codes, taus)
    b = O.cg_product(O.join_straight(fs), lmax, codes, taus)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    assert O.join_straight(a).shape == (4, 396, 2)


def test_fragment_norm_closed_form_and_invariants():
    rng = np.random.default_rng(0)
    f = torch.from_numpy(rng.normal(size=(6, 5, 7, 2)))
    s = O.fragment_std(f)
    mod = np.sqrt(f.numpy()[..., 0] ** 2 + f.numpy()[..., 1] ** 2)
    n = 6 * 7
    want = np.sqrt(np.maximum(0, (mod ** 2).sum((0, 2)) / n - (mod.sum((0, 2)) / n) ** 2))
    assert np.allclose(s, want, rtol=1e-12)
    assert np.allclose(O.fragment_std(3.5 * f), 3.5 * s, rtol=1e-12)            # scaling law
    # moving average: updated BEFORE use, with count starting at 1
    stds = [np.full(5, 0.25)]
    O.fragment_norm_update([f], stds, 1.0, True)
    assert np.allclose(stds[0], 0.25 * 0.5 + s * 0.5)
    O.fragment_norm_update([f], stds, 2.0, True)
    assert np.allclose(stds[0], (0.25 * 0.5 + s * 0.5) * (2 / 3) + s / 3)
    keep = [stds[0].copy()]
    O.fragment_norm_update([f], keep, 3.0, False)                                 # eval: untouched
    assert np.array_equal(keep[0], stds[0])
    # eps floor
    out = O.fragment_normalise([f], [np.array([1e-9, 0.5, 2.0, 1e-9, 1.0])], 1e-5)[0]
    assert torch.allclose(out[:, 0], f[:, 0] / 1e-5) and torch.allclose(out[:, 1], f[:, 1] / 0.5)


def test_weight_mix_matches_complex_einsum():
    g = torch.Generator().manual_seed(4)
    t_ff, t_out = [5, 3, 4], [2, 0, 3]
    ffs = [torch.randn(3, t_ff[l], 2 * l + 1, 2, generator=g, dtype=torch.float64) for l in range(3)]
    w = torch.randn(sum(a * b for a, b in zip(t_ff, t_out)), 2, generator=g, dtype=torch.float64)
    got = O.weight_mix(ffs, w, t_ff, t_out)
    o = 0
    for l in range(3):
        n = t_ff[l] * t_out[l]
        wl = torch.view_as_complex(w[o:o + n].reshape(t_out[l], t_ff[l], 2).contiguous())
        o += n
        want = torch.einsum("oc,bcm->bom", wl, torch.view_as_complex(ffs[l].contiguous()))
        assert got[l].shape == (3, t_out[l], 2 * l + 1, 2)
        assert torch.allclose(torch.view_as_complex(got[l].contiguous()), want, atol=1e-12)


def _tiny_layer(batchnorm):
    lmax, tin, tout = 2, [2, 1, 2], [1, 2, 1]
    codes, _ = T.encode_sorted(T.default_pairs(lmax))
    layer = O.LayerOracle(lmax, tin, tout, codes, batchnorm=batchnorm)
    layer.set_stds_flat(np.linspace(0.3, 1.2, sum(layer.t_ff)))
    layer.training = False
    return layer, tin, tout


@pytest.mark.parametrize("batchnorm", [False, True])
def test_layer_gradcheck_float64(batchnorm):
    layer, tin, tout = _tiny_layer(batchnorm)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, sum(t * (2 * l + 1) for l, t in enumerate(tin)), 2, generator=g, dtype=torch.float64,
                    requires_grad=True)
    w = torch.randn(T.cumulative_w(layer.t_ff, tout)[-1], 2, generator=g, dtype=torch.float64, requires_grad=True)

    def fn(xx, ww):
        return O.join_straight(layer.forward(xx, ww))
    assert torch.autograd.gradcheck(fn, (x, w), eps=1e-6, atol=1e-6)


def test_layer_adjoint_identity():
    # <gO, J dF> = <J^T gO, dF> for the CG product alone (bilinear map linearised at F)
    lmax, taus = 3, [2, 2, 1, 2]
    codes, _ = T.encode_sorted(T.default_pairs(lmax))
    g = torch.Generator().manual_seed(9)
    n = sum(t * (2 * l + 1) for l, t in enumerate(taus))
    x = torch.randn(2, n, 2, generator=g, dtype=torch.float64, requires_grad=True)
    dx = torch.randn(2, n, 2, generator=g, dtype=torch.float64)
    y = O.join_straight(O.cg_product(x, lmax, codes, taus))
    gy = torch.randn(y.shape, generator=g, dtype=torch.float64)
    (gx,) = torch.autograd.grad(y, x, gy)
    h = 1e-6
    yp = O.join_straight(O.cg_product(x.detach() + h * dx, lmax, codes, taus))
    ym = O.join_straight(O.cg_product(x.detach() - h * dx, lmax, codes, taus))
    lhs = float((gy * (yp - ym) / (2 * h)).sum())
    rhs = float((gx * dx).sum())
    assert lhs == pytest.approx(rhs, rel=1e-7)
    # bilinearity: doubling the input quadruples the output
    y2 = O.join_straight(O.cg_product(2 * x.detach(), lmax, codes, taus))
    assert torch.allclose(y2, 4 * y.detach(), rtol=1e-12)


def test_training_forward_updates_then_normalises():
    layer, tin, tout = _tiny_layer(True)
    layer.training = True
    g = torch.Generator().manual_seed(11)
    x = torch.randn(5, sum(t * (2 * l + 1) for l, t in enumerate(tin)), 2, generator=g, dtype=torch.float64)
    w = torch.randn(T.cumulative_w(layer.t_ff, tout)[-1], 2, generator=g, dtype=torch.float64)
    before = layer.stds_flat().copy()
    ff = O.cg_product(x, layer.lmax, layer.codes, tin)
    batch = np.concatenate([O.fragment_std(f) for f in ff])
    out = layer.forward(x, w)
    after = layer.stds_flat()
    assert np.allclose(after, 0.5 * before + 0.5 * batch)
    assert layer.cnt == 2.0
    # the output used the UPDATED stds
    layer2, _, _ = _tiny_layer(True)
    layer2.set_stds_flat(after)
    out2 = layer2.forward(x, w)
    assert all(torch.allclose(a, b, atol=1e-12) for a, b in zip(out, out2))


def test_stack_embedding_shape():
    lmax = 2
    taus = [[1, 1, 1], [2, 2, 2], [3, 1, 2]]
    codes, _ = T.encode_sorted(T.default_pairs(lmax))
    layers, ws = [], []
    g = torch.Generator().manual_seed(1)
    for i in range(2):
        ly = O.LayerOracle(lmax, taus[i], taus[i + 1], codes, batchnorm=True)
        ly.set_stds_flat(np.ones(sum(ly.t_ff)))
        layers.append(ly)
        ws.append(torch.randn(T.cumulative_w(ly.t_ff, taus[i + 1])[-1], 2, generator=g, dtype=torch.float64))
    x = torch.randn(3, 9, 2, generator=g, dtype=torch.float64)
    emb = O.stack_forward(layers, ws, x, taus[0], skipconn=True)
    assert emb.shape == (3, 2 * (1 + 2 + 3))
    assert torch.equal(emb[:, :2], x[:, 0:1, :].reshape(3, 2))
