"""CPU restatement of the reference's python CG layer (oracle; test infrastructure).

Fragments are a list over l of real tensors (B, tau[l], 2l+1, 2), last dim (re, im),
or the "straight" concatenation (B, sum_l tau[l](2l+1), 2)   (CG_layers_python.py:113-122).
Every function takes the dtype of its inputs, so the same code is the float64 arbiter
and the float32 twin of the reference's python path.
"""
import numpy as np
import torch

from . import cg_coeff, triples as T


def split_straight(x, taus):
    """Straight tensor -> list of (B, tau, 2l+1, 2) views   (CGutils.py:190-197)."""
    out, o = [], 0
    for l, t in enumerate(taus):
        n = int(t) * (2 * l + 1)
        out.append(x[:, o:o + n, :].reshape(x.shape[0], int(t), 2 * l + 1, 2))
        o += n
    assert o == x.shape[1]
    return out


def join_straight(fs):
    b = fs[0].shape[0]
    return torch.cat([f.reshape(b, -1, 2) for f in fs], dim=1)


def _kron_cols(a, b):
    """Batched Kronecker product of (B, n1, d1) with (B, n2, d2) -> (B, n1*n2, d1*d2),
    row = i1*n2 + i2, column = j1*d2 + j2   (Complex_math.py:12-35)."""
    bsz, n1, d1 = a.shape
    _, n2, d2 = b.shape
    return (a[:, :, None, :, None] * b[:, None, :, None, :]).reshape(bsz, n1 * n2, d1 * d2)


def cg_product(fs, lmax, codes, taus, cg_mats=None):
    """CG product over the kept triples   (CG_layers_python.py:113-133).

    Per triple (l, l1, l2): Kronecker product of the transposed fragments, complex
    parts expanded as in Complex_math.py:46-67, then the real CG matrix applied from
    the left by a batched matmul (Complex_math.py:73-74); blocks of one l are
    concatenated along channels in triple order.  Returns the list form.
    """
    if not isinstance(fs, (list, tuple)):
        fs = split_straight(fs, taus)
    dt = fs[0].dtype
    tr = [f.permute(0, 2, 1, 3) for f in fs]               # (B, 2l+1, tau, 2)
    blocks = [[] for _ in range(lmax + 1)]
    cache = {} if cg_mats is None else cg_mats
    for (l, l1, l2) in T.decode(lmax, codes):
        key = (l1, l2, l)
        if key not in cache:
            cache[key] = torch.from_numpy(cg_coeff.cg_matrix(l1, l2, l, np.float64))
        # the reference keeps the dictionary in float32 (CGutils.py:57); the float64 arbiter
        # uses the same rounded coefficients so that it measures arithmetic error only
        cmat = cache[key].to(torch.float32).to(dt)
        ar, ai = tr[l1][..., 0], tr[l1][..., 1]
        br, bi = tr[l2][..., 0], tr[l2][..., 1]
        kr = _kron_cols(ar, br) - _kron_cols(ai, bi)
        ki = _kron_cols(ar, bi) + _kron_cols(ai, br)
        outr = torch.matmul(cmat, kr)                        # (B, 2l+1, tau1*tau2)
        outi = torch.matmul(cmat, ki)
        blocks[l].append(torch.stack([outr, outi], dim=3).permute(0, 2, 1, 3))
    return [torch.cat(b, dim=1) for b in blocks]


def fragment_std(ff_l):
    """Population std over (batch, m) of |z| for each channel of one degree
    (CG_layers_python.py:175-177: numpy norm over the complex axis, numpy std over axes 0,2)."""
    v = ff_l.detach().cpu().numpy()
    nrm = np.linalg.norm(v, ord=2, axis=3)
    return np.std(nrm, axis=(0, 2))


def fragment_norm_update(ffs, stds, cnt, training):
    """Moving-average update of the per-channel stds (in place on the numpy list ``stds``)
    (CG_layers_python.py:173-183; CUDA twin cudaCG_FNWMM.cu:29-79).

    The running value is updated with the current batch BEFORE it is used to
    normalise that batch; cnt starts at 1 and is incremented by the caller.
    """
    if not training:
        return stds
    for l, f in enumerate(ffs):
        s = fragment_std(f).astype(stds[l].dtype)
        stds[l] *= stds[l].dtype.type(cnt / (cnt + 1.0))
        stds[l] += s / stds[l].dtype.type(cnt + 1.0)
    return stds


def fragment_normalise(ffs, stds, eps):
    """fl / max(eps, std) per channel; the stds are constants for autograd
    (CG_layers_python.py:181)."""
    out = []
    for l, f in enumerate(ffs):
        d = torch.from_numpy(np.maximum(stds[l], stds[l].dtype.type(eps))).to(f.dtype)
        out.append(f / d.reshape(1, -1, 1, 1))
    return out


def complex_bmm(w, f):
    """(B, M, K, 2) x (B, K, N, 2) -> (B, M, N, 2) by four real bmm   (CGutils.py:15-21)."""
    wr, wi = w[..., 0], w[..., 1]
    fr, fi = f[..., 0], f[..., 1]
    re = torch.bmm(wr, fr) - torch.bmm(wi, fi)
    im = torch.bmm(wr, fi) + torch.bmm(wi, fr)
    return torch.stack([re, im], dim=3)


def weight_mix(ffs, w_flat, t_ff, t_out):
    """Per-l complex channel mixing O_l = W_l . FF_l with W_l = (t_O[l], t_FF[l]) row-major
    slices of the flat (nW, 2) parameter   (CG_layers_python.py:259-266)."""
    out, o = [], 0
    b = ffs[0].shape[0]
    for l, f in enumerate(ffs):
        n = int(t_ff[l]) * int(t_out[l])
        wl = w_flat[o:o + n, :].reshape(int(t_out[l]), int(t_ff[l]), 2)
        o += n
        out.append(complex_bmm(wl.unsqueeze(0).expand(b, -1, -1, -1).contiguous(), f))
    assert o == w_flat.shape[0]
    return out


class LayerOracle:
    """One CG -> fragment norm -> weight mixing layer   (CG_layers_python.py:188-269).

    ``stds`` (list of numpy arrays per l) and ``w`` are injected by the caller: the
    reference draws its initial weights on the CUDA RNG (CG_layers_python.py:242), which
    cannot be reproduced elsewhere.
    """

    def __init__(self, lmax, taus_in, taus_out, codes, batchnorm=True, eps=1e-5):
        self.lmax, self.taus_in, self.taus_out, self.codes = lmax, list(taus_in), list(taus_out), list(codes)
        self.t_ff, self.t_off = T.product_taus(lmax, codes, taus_in)
        self.batchnorm, self.eps = batchnorm, eps
        self.cnt = 1.0
        self.training = True
        self.stds = None
        self._mats = {}

    def set_stds_flat(self, flat):
        o, self.stds = 0, []
        for t in self.t_ff:
            self.stds.append(np.array(flat[o:o + t], copy=True))
            o += t

    def stds_flat(self):
        return np.concatenate(self.stds)

    def forward(self, fs, w_flat):
        ffs = cg_product(fs, self.lmax, self.codes, self.taus_in, self._mats)
        if self.batchnorm:
            fragment_norm_update(ffs, self.stds, self.cnt, self.training)
            ffs = fragment_normalise(ffs, self.stds, self.eps)
            if self.training:
                self.cnt += 1.0
        return weight_mix(ffs, w_flat, self.t_ff, self.taus_out)


def stack_forward(layers, ws, f_input, taus0, skipconn=True):
    """l=0 skip-connection embedding of a stack of layers   (CGNet.py:52-69)."""
    fs = f_input if isinstance(f_input, (list, tuple)) else split_straight(f_input, taus0)
    b = fs[0].shape[0]
    emb = [fs[0].reshape(b, -1)] if skipconn else []
    for layer, w in zip(layers, ws):
        fs = layer.forward(fs, w)
        if skipconn:
            emb.append(fs[0].reshape(b, -1))
    return torch.cat(emb, dim=1) if skipconn else fs[0].reshape(b, -1)
