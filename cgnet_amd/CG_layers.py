"""Clebsch-Gordan layer modules and autograd Functions with the reference's API
(CGNet/CG_layers.py): ``_CG_sparse_cuda`` (:168-203), ``_MyBatchNormWeightMM_cuda`` (:14-72),
``CG_woFilter_cuda`` (:205-286), ``MyBatchNormWeightMM_cuda`` (:74-132), ``CGBN_cuda``
(:289-318), ``precomputeCG`` (:134-165).  Constructor keywords, ``forward`` arguments, the
parameter names in ``state_dict`` (``bnWMM.W``, ``bnWMM.bn_stds``, ``bnWMM.bn_eps``) and the
Functions' positional signatures / ``None`` padding are the reference's.

All arithmetic runs in libcgnet_hip (HIP kernels for gfx950) through ``CG_cuda_ops``; there
is no CPU implementation behind these classes.  Modules can be constructed without a GPU
(parameters and metadata only); the native plans are created on first use.
"""
import functools
import os

import numpy as np
import torch
from torch import nn

from . import CG_cuda_ops, CGutils, _lib
from . import _plans
from ._plans import CGPlan, WMMPlan

BN_FLAG = _lib.FN_BATCHNORM
UPDATESTD_FLAG = _lib.FN_UPDATE_STD


def _as_float(x):
    return float(x.item()) if isinstance(x, torch.Tensor) else float(x)


def _cumulative_tm(taus):
    taus = np.asarray(taus, dtype=np.int64)
    return np.concatenate([[0], np.cumsum(taus * (2 * np.arange(len(taus)) + 1))])


# --------------------------------------------------------------------------- fragment norm + mixing
class _MyBatchNormWeightMM_cuda(torch.autograd.Function):
    @staticmethod
    def forward(ctx, FF, W, t_FF, cumu_tm_FF, t_O, cumu_tm_O, cumu_tt_W, bn_stds, bn_cnt, bn_eps, bn_updateflag):
        lmax = t_FF.shape[0] - 1
        B = FF.shape[0]
        plan = CG_cuda_ops._wmm_plan(lmax, t_FF, cumu_tm_O)
        flags = (BN_FLAG if bn_stds is not None else 0) | (UPDATESTD_FLAG if bn_updateflag else 0)
        eps = _as_float(bn_eps)
        FF = FF.contiguous()
        W = W.contiguous()
        output = torch.empty(B, plan.nO, 2, device=FF.device, dtype=torch.float)
        plan.forward(FF, output, W, B, bn_stds, float(bn_cnt), eps, flags)
        # bn_stds was updated in place; backward must see the value used for this batch
        saved_stds = bn_stds.detach().clone() if bn_stds is not None else None
        ctx.plan, ctx.B, ctx.eps, ctx.flags = plan, B, eps, flags
        ctx.save_for_backward(FF, W, saved_stds)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        FF, W, stds = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_FF = torch.empty_like(FF) if ctx.needs_input_grad[0] else None
        grad_W = torch.empty_like(W) if ctx.needs_input_grad[1] else None
        if grad_FF is not None or grad_W is not None:
            ctx.plan.backward(grad_output, grad_FF, grad_W, FF, W, ctx.B, stds, ctx.eps, ctx.flags)
        return grad_FF, grad_W, None, None, None, None, None, None, None, None, None


class MyBatchNormWeightMM_cuda(nn.Module):
    def __init__(self, lmax, t_FF, tau_out, batchnorm=True, weight_scale=0.05, init='random', eps=1e-5,
                 device='cuda'):
        super().__init__()
        self.lmax = lmax
        self._init_method = init
        self.weight_scale = weight_scale
        self.t_FF = np.asarray(t_FF, dtype=np.int64)
        if len(self.t_FF) - 1 != lmax:
            raise AssertionError("t_FF must have lmax+1 entries")
        self.t_O = np.asarray(tau_out, dtype=np.int64)
        if len(self.t_O) - 1 != lmax:
            raise AssertionError("tau_out must have lmax+1 entries")
        self.cumu_tm_FF = _cumulative_tm(self.t_FF)
        self.cumu_tm_O = _cumulative_tm(self.t_O)
        self.cumu_tm_W = np.concatenate([[0], np.cumsum(self.t_FF * self.t_O)])

        self.batchnorm = batchnorm
        self.bn_stds = None
        self.bn_eps = nn.Parameter(eps * torch.ones(1), requires_grad=False)
        self._eps_host = float(eps)
        self.bn_cnt = 1.
        self.W = None
        self._device = torch.device(device)
        self.reset_parameters()

        i32 = dict(dtype=torch.int32, device=self._device)
        self.d_t_FF = torch.tensor(self.t_FF, **i32)
        self.d_cumu_tm_FF = torch.tensor(self.cumu_tm_FF, **i32)
        self.d_t_O = torch.tensor(self.t_O, **i32)
        self.d_cumu_tm_O = torch.tensor(self.cumu_tm_O, **i32)
        self.d_cumu_tt_W = torch.tensor(self.cumu_tm_W, **i32)
        self._plan = None
        self.to(self._device)

    def reset_parameters(self):
        if self._init_method not in {'debug', 'random'}:
            raise NotImplementedError()
        if self._init_method == 'debug':
            torch.manual_seed(0)
            np.random.seed(0)
        if self.batchnorm:
            stds = np.random.rand(int(self.t_FF.sum()))
            self.bn_stds = nn.Parameter(torch.tensor(stds, dtype=torch.float), requires_grad=False)
        n_w = int((self.t_FF * self.t_O).sum())
        w = self.weight_scale * torch.rand(n_w, 2, device=self._device, dtype=torch.float)
        self.W = nn.Parameter(w, requires_grad=True)

    def native_plan(self):
        """The native plan, created on first use and registered for ``CG_cuda_ops`` lookups."""
        if self._plan is None:
            self._plan = WMMPlan(self.lmax, self.t_FF.tolist(), self.t_O.tolist())
            CG_cuda_ops.register_wmm_plan(self._plan, self.d_t_FF, self.d_cumu_tm_O)
        return self._plan

    def _apply(self, fn, *args, **kwargs):
        # keep the metadata tensors (plain attributes, as in the reference) on the module's device
        out = super()._apply(fn, *args, **kwargs)
        moved = False
        for name in ("d_t_FF", "d_cumu_tm_FF", "d_t_O", "d_cumu_tm_O", "d_cumu_tt_W"):
            t = getattr(self, name, None)
            if t is not None:
                nt = fn(t)
                moved |= nt is not t
                setattr(self, name, nt)
        if moved and self._plan is not None:
            CG_cuda_ops.register_wmm_plan(self._plan, self.d_t_FF, self.d_cumu_tm_O)
        return out

    def forward(self, FF):
        self.native_plan()
        output = _MyBatchNormWeightMM_cuda.apply(FF, self.W, self.d_t_FF, self.d_cumu_tm_FF, self.d_t_O,
                                                 self.d_cumu_tm_O, self.d_cumu_tt_W, self.bn_stds, self.bn_cnt,
                                                 self._eps_host, self.training)
        if self.batchnorm and self.training:
            self.bn_cnt += 1
        return output

    # ``bn_cnt`` is the plain float attribute of the reference (CG_layers.py:92,130: read on every forward, so it
    # must not live on the device) and, as there, is NOT part of ``state_dict`` by default: the key set is exactly the
    # reference's (``W``, ``bn_stds``, ``bn_eps``), so checkpoints load with ``strict=True`` in both directions.  The
    # reference loses the count on a resume; ``persist_bn_cnt = True`` (on the class or on an instance) adds the entry
    # ``bn_cnt`` to ``state_dict`` so that a resumed run continues the moving average where it stopped -- such a
    # checkpoint is rejected by the reference's strict loader.  A ``bn_cnt`` entry is accepted on load either way.
    persist_bn_cnt = False

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        if self.persist_bn_cnt:
            destination[prefix + "bn_cnt"] = torch.tensor(float(self.bn_cnt), dtype=torch.float64)

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                              error_msgs):
        key = prefix + "bn_cnt"
        cnt = state_dict.pop(key, None) if key in state_dict else None
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys,
                                      error_msgs)
        if cnt is not None:
            self.bn_cnt = float(cnt)
            state_dict[key] = cnt          # the caller's dictionary is left as it was
        self._eps_host = float(self.bn_eps.detach().cpu().item())


# --------------------------------------------------------------------------- CG tables
def _precomputeCG_cuda(lmax, llls, device='cuda'):
    CG_len = CGutils.SparseLtuples.get_CG_length(lmax, llls)
    CG_offsets = CGutils.SparseLtuples.cal_CG_offsets(lmax, llls)
    CG_coefs = torch.zeros(CG_len, dtype=torch.float, device=device, requires_grad=False)
    d_offsets = torch.tensor(CG_offsets, dtype=torch.int, device=device, requires_grad=False)
    d_llls = torch.tensor(llls, dtype=torch.int, device=device, requires_grad=False)
    CG_cuda_ops.sparse_precomputeCG(CG_coefs, lmax, d_llls, d_offsets)
    return CG_coefs, d_offsets


def _precomputeCG_MST(lmax, method='mst', device='cuda'):
    assert method == 'mst', '%s is not implemented' % method
    mst_llls = CGutils.SparseLtuples.sparse_rep_ltuples_sorted(CGutils.SparseLtuples.compute_mst_ltuples(lmax))[0]
    return _precomputeCG_cuda(lmax, mst_llls, device=device)


@functools.lru_cache(10)
def precomputeCG(lmax, method='mst', device='cuda'):
    """Cached (CG table, CG offsets) on ``device`` for the default (method=None) or 'mst' triple list."""
    if method is None:
        ltuples = CGutils.SparseLtuples.compute_default_ltuples(lmax)
        llls = CGutils.SparseLtuples.sparse_rep_ltuples_sorted(ltuples)[0]
        return _precomputeCG_cuda(lmax, llls, device=device)
    if method == 'mst':
        return _precomputeCG_MST(lmax, 'mst', device=device)
    raise NotImplementedError()


def _straight(fragments):
    """List over l of (B, tau[l], 2l+1, 2) GPU tensors -> the straight tensor (B, sum tau[l](2l+1), 2).  When the
    fragments are the consecutive views ``CGutils.reshape_out`` makes of one straight tensor (what a stack of these
    layers hands from one to the next), that tensor is returned as it is; otherwise the fragments are concatenated
    (reference: CGNet/CG_layers.py:275)."""
    first = fragments[0]
    assert first.is_cuda
    B = first.shape[0]
    base = first._base
    if base is not None and base.dim() == 3 and base.shape[0] == B and base.shape[2] == 2 and base.is_contiguous():
        off, ok = base.storage_offset(), True
        row = base.shape[1] * 2
        for v in fragments:
            n = v.numel() // B if B else 0
            if (v._base is not base or v.dim() != 4 or v.shape[0] != B or v.shape[3] != 2
                    or v.storage_offset() != off or v.stride() != (row, v.shape[2] * 2, 2, 1)):
                ok = False
                break
            off += n
        if ok and off - base.storage_offset() == row:
            return base
    return torch.cat([v.reshape(B, -1, 2) for v in fragments], dim=1)


# --------------------------------------------------------------------------- CG product
class _CG_sparse_cuda(torch.autograd.Function):
    @staticmethod
    def forward(ctx, Fs, output_length, t_F, cumu_tm_F, t_FF, cumu_tm_FF, llls, l_l1_to_lllidx_offsets, t_offsets,
                CG, CG_offsets):
        lmax = len(t_F) - 1
        assert lmax <= CG_cuda_ops.sparse_maxL(), f"Does not support lmax={lmax}"
        plan = CG_cuda_ops._cg_plan(lmax, t_F, llls, t_offsets, CG_offsets)
        if int(output_length) != plan.nFF:
            raise RuntimeError("output_length=%d does not match the triple list (%d)" % (output_length, plan.nFF))
        Fs = Fs.contiguous()
        B = Fs.shape[0]
        output = torch.empty(B, plan.nFF, 2, device=Fs.device, dtype=torch.float)
        plan.forward(Fs, output, CG, B)
        ctx.plan = plan
        ctx.save_for_backward(Fs, CG)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        Fs, CG = ctx.saved_tensors
        grad_input = None
        if ctx.needs_input_grad[0]:
            grad_input = torch.empty_like(Fs)
            ctx.plan.backward(Fs, grad_input, grad_output.contiguous(), CG, Fs.shape[0])
        return grad_input, None, None, None, None, None, None, None, None, None, None


class CG_woFilter_cuda(nn.Module):
    def __init__(self, lmax, taus, lll_mode=None, device='cuda'):
        """
        :param lmax: degrees l = 0..lmax
        :param taus: channels of the input per degree; fragment l has shape (B, taus[l], 2l+1, 2)
        :param lll_mode: None (every l2 <= l1 pair), 'mst' (minimum-spanning-tree subset),
            'debug' (first two pairs per degree) or a list whose item l is a list of (l1, l2)
        """
        super().__init__()
        self.lmax = lmax
        self.t_F = np.asarray(taus, dtype=np.int64)
        if len(self.t_F) != lmax + 1:
            raise AssertionError("taus must have lmax+1 entries")
        self.cum_taus = _cumulative_tm(self.t_F)
        self._device = torch.device(device)
        self._lll_mode = lll_mode if (lll_mode is None or isinstance(lll_mode, str)) else 'custom'

        if lll_mode is None:
            ltuples = CGutils.SparseLtuples.compute_default_ltuples(lmax)
        elif isinstance(lll_mode, str) and lll_mode == 'mst':
            ltuples = CGutils.SparseLtuples.compute_mst_ltuples(lmax)
        elif isinstance(lll_mode, str) and lll_mode == 'debug':
            ltuples = CGutils.SparseLtuples.compute_debug_ltuples(lmax)
        else:
            ltuples = lll_mode
            if len(ltuples) != lmax + 1:
                raise AssertionError("a custom triple list needs one entry per degree")
            for l, pairs in enumerate(ltuples):
                for l1, l2 in pairs:
                    if not (0 <= l2 <= l1 <= lmax and l1 - l2 <= l <= l1 + l2):
                        raise AssertionError("(l1=%d, l2=%d) -> l=%d is not an admissible triple" % (l1, l2, l))
        self.lll_list, self.l_l1_to_lllidx_offsets = CGutils.SparseLtuples.sparse_rep_ltuples_sorted(ltuples)
        self.t_FF, t_offsets = self.cal_new_tau_and_offsets(self.t_F)
        self.cumu_tm_FF = _cumulative_tm(self.t_FF)
        self._t_offsets_host = t_offsets
        self._cg_offsets_host = CGutils.SparseLtuples.cal_CG_offsets(lmax, self.lll_list)

        i32 = dict(dtype=torch.int32, device=self._device)
        self.d_t_F = torch.tensor(self.t_F, **i32)
        self.d_cumu_tm_F = torch.tensor(self.cum_taus, **i32)
        self.d_t_FF = torch.tensor(self.t_FF, **i32)
        self.d_cumu_tm_FF = torch.tensor(self.cumu_tm_FF, **i32)
        self.d_l_l1_to_lllidx_offsets = torch.tensor(self.l_l1_to_lllidx_offsets, **i32)
        self.d_llls = torch.tensor(self.lll_list, **i32)
        self.t_offsets = torch.tensor(t_offsets, **i32)
        self.CGspace, self.CG_offsets = None, None
        self._plan = None
        if self._device.type == 'cuda':
            self._materialise()

    def _materialise(self):
        """CG table on the GPU (shared through the ``precomputeCG`` cache for the two stock
        modes) and the native plan, registered under this module's metadata tensors."""
        dev = str(self._device)
        if self._lll_mode in (None, 'mst'):
            self.CGspace, self.CG_offsets = precomputeCG(self.lmax, self._lll_mode, dev)
        else:
            self.CGspace, self.CG_offsets = _precomputeCG_cuda(self.lmax, self.lll_list, device=dev)
        self._plan = CGPlan(self.lmax, self.t_F.tolist(), self.lll_list, self._t_offsets_host, self._cg_offsets_host)
        CG_cuda_ops.register_cg_plan(self._plan, self.d_t_F, self.d_llls, self.t_offsets)

    def native_plan(self):
        if self._plan is None:
            self._materialise()
        return self._plan

    def _apply(self, fn, *args, **kwargs):
        out = super()._apply(fn, *args, **kwargs)
        names = ("d_t_F", "d_cumu_tm_F", "d_t_FF", "d_cumu_tm_FF", "d_l_l1_to_lllidx_offsets", "d_llls", "t_offsets")
        moved = False
        for name in names:
            t = getattr(self, name, None)
            if t is not None:
                nt = fn(t)
                moved |= nt is not t
                setattr(self, name, nt)
        if moved:
            self._device = self.d_t_F.device
            self._plan = None
            self.CGspace, self.CG_offsets = None, None
            if self._device.type == 'cuda':
                self._materialise()
        return out

    def cal_new_tau_and_offsets(self, taus):
        t_offsets = []
        t_FF = np.zeros(self.lmax + 1, dtype=np.int64)
        for l, l1, l2 in CGutils.SparseLtuples.get_iter(self.lmax, self.lll_list):
            t_offsets.append(int(t_FF[l]))
            t_FF[l] += int(taus[l1]) * int(taus[l2])
        return t_FF, t_offsets

    def forward(self, activations, straight_output=True):
        """``activations``: list over l of (B, tau[l], 2l+1, 2) GPU tensors, or the straight
        tensor (B, sum tau[l](2l+1), 2).  Returns the straight product, or its list form."""
        if isinstance(activations, (list, tuple)):
            new_activations = _straight(activations)
        else:
            new_activations = activations
        assert new_activations.is_cuda
        self.native_plan()
        output = _CG_sparse_cuda.apply(new_activations, int(self.cumu_tm_FF[-1]), self.d_t_F, self.d_cumu_tm_F,
                                       self.d_t_FF, self.d_cumu_tm_FF, self.d_llls,
                                       self.d_l_l1_to_lllidx_offsets, self.t_offsets, self.CGspace, self.CG_offsets)
        if not straight_output:
            output = CGutils.reshape_out(output, self.t_FF)
        return output


# --------------------------------------------------------------------------- the whole layer
# CGNET_FUSED_BACKWARD=0: new layers take the two-kernel backward (grad_FF in memory) even where the one-kernel
# backward is available
_FUSED_BACKWARD = bool(int(os.environ.get("CGNET_FUSED_BACKWARD", "1")))
# CGNET_FUSED_INFERENCE=0: new layers materialise FF in evaluation mode too
_FUSED_INFERENCE = bool(int(os.environ.get("CGNET_FUSED_INFERENCE", "1")))
# CGNET_COMPACT_FF=0: the product tensor inside a layer keeps the reference's layout (both orderings of every channel
# pair of a diagonal triple) also where nothing outside the layer's own kernels reads it
_COMPACT_FF = bool(int(os.environ.get("CGNET_COMPACT_FF", "1")))


class _CGBN_fused(torch.autograd.Function):
    """CG product -> fragment norm -> weight mixing in one autograd node (``cgnet_CGBN_forward``).  Same
    arithmetic and results as ``_CG_sparse_cuda`` followed by ``_MyBatchNormWeightMM_cuda``; the per-channel
    statistics come out of the product kernel instead of a second pass over FF, and neither FF nor grad_FF is
    visible outside the node, so the backward may skip grad_FF altogether (``fused_backward``)."""

    @staticmethod
    def forward(ctx, Fs, W, layer_plan, CG, bn_stds, bn_cnt, bn_eps, training, fused_backward=True):
        cg_plan, wmm_plan = layer_plan.cg_plan, layer_plan.wmm_plan
        Fs = Fs.contiguous()
        W = W.contiguous()
        B = Fs.shape[0]
        dev = Fs.device
        flags = (BN_FLAG if bn_stds is not None else 0) | (UPDATESTD_FLAG if training else 0)
        need_grad = ctx.needs_input_grad[0] or ctx.needs_input_grad[1]
        ctx.fused_backward = bool(fused_backward) and layer_plan.fused_backward_supported
        # With the one-kernel backward nothing reads FF but the mixing and the weight gradient, and the layer keeps
        # it in its compact layout (one channel per pair of a diagonal triple) where it has one.
        if ctx.fused_backward and layer_plan.compact_supported and _COMPACT_FF:
            flags |= _lib.LAYER_COMPACT_FF
        FF = torch.empty(B, layer_plan.internal_nFF(flags), 2, device=dev, dtype=torch.float)
        out = torch.empty(B, wmm_plan.nO, 2, device=dev, dtype=torch.float)
        # the operands of the one-kernel backward are prepared beside those of the mixing forward, in the same launch
        saved_ops = layer_plan.forward(Fs, FF, out, W, CG, B, bn_stds, float(bn_cnt), float(bn_eps), flags,
                                       save=ctx.fused_backward and ctx.needs_input_grad[0])
        # bn_stds was updated in place; backward must see the value used for this batch: the copy the forward left
        # among the saved operands, else a clone
        saved_stds = None
        if bn_stds is not None and need_grad:
            saved_stds = layer_plan.saved_stds(saved_ops, B)
            if saved_stds is None:
                saved_stds = bn_stds.detach().clone()
        ctx.layer_plan, ctx.B, ctx.eps, ctx.flags = layer_plan, B, float(bn_eps), flags
        ctx.save_for_backward(Fs, W, FF, CG, saved_stds, saved_ops)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        Fs, W, FF, CG, stds, saved_ops = ctx.saved_tensors
        cg_plan, wmm_plan = ctx.layer_plan.cg_plan, ctx.layer_plan.wmm_plan
        grad_output = grad_output.contiguous()
        need_F, need_W = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        grad_W = torch.empty_like(W) if need_W else None
        grad_F = torch.empty_like(Fs) if need_F else None
        if ctx.fused_backward:
            # The gradient with respect to FF never exists in memory: the product's backward forms every tile of
            # it in LDS from grad_output and the weights.  The weight gradient needs FF, not grad_FF.
            if need_W:
                ctx.layer_plan.backward_gradw(grad_output, FF, grad_W, ctx.B, stds, ctx.eps, ctx.flags)
            if need_F:
                ctx.layer_plan.backward_fused(Fs, grad_F, grad_output, W, CG, ctx.B, stds, ctx.eps,
                                              ctx.flags & (BN_FLAG | UPDATESTD_FLAG), saved_ops)
            return grad_F, grad_W, None, None, None, None, None, None, None
        grad_FF = torch.empty_like(FF) if need_F else None
        if need_F or need_W:
            wmm_plan.backward(grad_output, grad_FF, grad_W, FF, W, ctx.B, stds, ctx.eps, ctx.flags)
        if need_F:
            cg_plan.backward(Fs, grad_F, grad_FF, CG, ctx.B)
        return grad_F, grad_W, None, None, None, None, None, None, None


class CGBN_cuda(nn.Module):
    def __init__(self, lmax, taus_fs, tau_out, batchnorm=True, sparse_flag=False, device='cuda',
                 weight_scale=0.05, init='random', eps=1e-5):
        super().__init__()
        self.lmax = lmax
        self._init_method = init
        # sparse_flag=True selects the MST subset; False the full half-pair list
        self.sparse_flag = sparse_flag
        self.cg = CG_woFilter_cuda(lmax, taus_fs, lll_mode='mst' if sparse_flag else None, device=device)
        self.t_F = self.cg.t_F
        self.t_FF = self.cg.t_FF
        self.tau_out = tau_out
        self.bnWMM = MyBatchNormWeightMM_cuda(lmax, self.t_FF, tau_out, batchnorm, weight_scale, init, eps, device)
        self.fused = True      # False: chain the two reference Functions (separate statistics pass)
        # With ``fused``: True takes the backward from grad_output to the input gradient in one kernel, without a
        # grad_FF tensor (B x nFF complex) in memory, where the shapes allow it
        # (cgnet_CGBN_backward_fused_supported); False keeps the two-kernel backward.  Same gradients either way.
        self.fused_backward = _FUSED_BACKWARD
        # With ``fused``: when no gradient is wanted and the statistics are not updated (evaluation mode, or no fragment
        # norm), True takes the forward without the product tensor FF (B x nFF complex) in memory, every tile of it mixed
        # in LDS, where the shapes allow it (cgnet_CGBN_forward_inference_supported); same output up to rounding.
        self.fused_inference = _FUSED_INFERENCE
        self._layer_plan = None
        self.to(device)

    def native_layer_plan(self):
        """The native layer plan (product plan linked with the mixing plan), created on first use and again
        whenever one of the two plans has been rebuilt (a move to another device)."""
        cg_plan, wmm_plan = self.cg.native_plan(), self.bnWMM.native_plan()
        lp = self._layer_plan
        if lp is None or lp.cg_plan is not cg_plan or lp.wmm_plan is not wmm_plan:
            lp = self._layer_plan = _plans.LayerPlan(cg_plan, wmm_plan)
        return lp

    def forward(self, fs, straight_output=False):
        if self.fused:
            if isinstance(fs, (list, tuple)):
                fs = _straight(fs)
            assert fs.is_cuda
            bn = self.bnWMM
            lp = self.native_layer_plan()
            wants_grad = torch.is_grad_enabled() and (fs.requires_grad or bn.W.requires_grad)
            updates = bn.batchnorm and bn.training
            if self.fused_inference and not wants_grad and not updates and lp.inference_forward_supported:
                B = fs.shape[0]
                new_fs = torch.empty(B, lp.wmm_plan.nO, 2, device=fs.device, dtype=torch.float)
                lp.forward_inference(fs.detach().contiguous(), new_fs, bn.W.detach().contiguous(), self.cg.CGspace, B,
                                     bn.bn_stds, bn._eps_host, BN_FLAG if bn.bn_stds is not None else 0)
            else:
                new_fs = _CGBN_fused.apply(fs, bn.W, lp, self.cg.CGspace, bn.bn_stds, bn.bn_cnt, bn._eps_host, bn.training,
                                           self.fused_backward)
            if updates:
                bn.bn_cnt += 1
        else:
            new_fs = self.cg(fs, straight_output=True)
            new_fs = self.bnWMM(new_fs)
        if not straight_output:
            new_fs = CGutils.reshape_out(new_fs, self.tau_out)
        return new_fs
