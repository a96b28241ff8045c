"""Python owners of the native plan objects and thin torch-tensor front ends for the C ABI.

torch is used here only for device memory (the tensors whose ``data_ptr()`` is handed over),
for the caller's current HIP stream and for workspace allocation through its caching allocator.
"""
import ctypes

import torch

from . import _lib


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _require_gpu(name, t, dtype=torch.float32):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError("%s must be a tensor in GPU memory (got %s); this package has no CPU path"
                           % (name, "a %s tensor" % t.device if isinstance(t, torch.Tensor) else type(t).__name__))
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError("%s must have dtype %s (got %s)" % (name, dtype, t.dtype))


def _aligned16(t):
    """The streaming kernels use 16-byte loads; a view that starts mid-allocation is copied."""
    return t if t is None or t.data_ptr() % 16 == 0 else t.clone()


def _workspace(nbytes, device):
    return torch.empty(max(int(nbytes), 1), dtype=torch.uint8, device=device)


def fill_cg_table(cg, lmax, llls, cg_offsets):
    """Write the flat Clebsch-Gordan table into the GPU tensor ``cg`` (float32)."""
    _require_gpu("CG", cg)
    llls = [int(v) for v in llls]
    cg_offsets = [int(v) for v in cg_offsets]
    if len(cg_offsets) != len(llls) + 1:
        raise RuntimeError("CG_offsets must have len(llls)+1 entries")
    if cg.numel() < cg_offsets[-1]:
        raise RuntimeError("CG tensor has %d entries, %d needed" % (cg.numel(), cg_offsets[-1]))
    lib = _lib.load()
    with torch.cuda.device(cg.device):
        _lib.check(lib.cgnet_sparse_precomputeCG(_ptr(cg), int(lmax), _lib.int_array(llls), len(llls),
                                                 _lib.int_array(cg_offsets), _stream(cg.device)))


class CGPlan:
    """Plan of one CG product (``cgnet_cg_plan``): input channels per degree + kept triples."""

    def __init__(self, lmax, t_F, llls, t_offsets=None, cg_offsets=None):
        self.lmax = int(lmax)
        self.t_F = [int(v) for v in t_F]
        self.llls = [int(v) for v in llls]
        if len(self.t_F) != self.lmax + 1:
            raise RuntimeError("t_F must have lmax+1 = %d entries (got %d)" % (self.lmax + 1, len(self.t_F)))
        lib = _lib.load()
        h = ctypes.c_void_p()
        toff = None if t_offsets is None else _lib.int_array(t_offsets)
        cgo = None if cg_offsets is None else _lib.int_array(cg_offsets)
        if t_offsets is not None and len(t_offsets) != len(self.llls):
            raise RuntimeError("t_offsets must have one entry per triple")
        if cg_offsets is not None and len(cg_offsets) != len(self.llls) + 1:
            raise RuntimeError("CG_offsets must have len(llls)+1 entries")
        _lib.check(lib.cgnet_cg_plan_create(ctypes.byref(h), self.lmax, _lib.int_array(self.t_F),
                                            _lib.int_array(self.llls), len(self.llls), toff, cgo))
        self._h = h
        sizes = (ctypes.c_int * 5)()
        _lib.check(lib.cgnet_cg_plan_sizes(self._h, sizes))
        self.nF, self.nFF, self.sum_tFF, self.cg_len, _ = [int(v) for v in sizes]
        tff = (ctypes.c_int * (self.lmax + 1))()
        toffs = (ctypes.c_int * max(1, len(self.llls)))()
        _lib.check(lib.cgnet_cg_plan_channels(self._h, tff, toffs))
        self.t_FF = [int(v) for v in tff]
        self.t_offsets = [int(v) for v in toffs][:len(self.llls)]
        self.backward_lds = int(lib.cgnet_cg_plan_backward_lds(self._h))   # bytes per work-group of the backward
        self.forward_lds = int(lib.cgnet_cg_plan_forward_lds(self._h))     # ... of the forward (largest launch class)
        self.backward_groups = int(lib.cgnet_cg_plan_backward_groups(self._h))   # backward work-groups per compute unit

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h is not None and _lib._lib is not None:
            _lib._lib.cgnet_cg_plan_destroy(h)

    def _check_io(self, F, B):
        _require_gpu("input", F)
        if F.numel() != B * self.nF * 2:
            raise RuntimeError("input has %d floats, expected B*nF*2 = %d*%d*2" % (F.numel(), B, self.nF))

    def forward(self, F, FF, CG, B):
        self._check_io(F, B)
        _require_gpu("output", FF)
        _require_gpu("CG", CG)
        if FF.numel() != B * self.nFF * 2:
            raise RuntimeError("output has %d floats, expected B*nFF*2 = %d*%d*2" % (FF.numel(), B, self.nFF))
        if CG.numel() < self.cg_len:
            raise RuntimeError("CG table has %d entries, %d needed" % (CG.numel(), self.cg_len))
        with torch.cuda.device(F.device):
            _lib.check(_lib.load().cgnet_sparse_forward(self._h, _ptr(F), _ptr(FF), _ptr(CG), int(B), _stream(F.device)))

    def forward_stats(self, F, FF, CG, B, sums):
        """Product plus per-channel (sum |z|, sum |z|^2) in the float64 tensor ``sums`` (sum_tFF, 2)."""
        self._check_io(F, B)
        _require_gpu("output", FF)
        _require_gpu("CG", CG)
        _require_gpu("sums", sums, torch.float64)
        if FF.numel() != B * self.nFF * 2 or sums.numel() != 2 * self.sum_tFF or CG.numel() < self.cg_len:
            raise RuntimeError("forward_stats: tensor sizes do not match the plan")
        lib = _lib.load()
        with torch.cuda.device(F.device):
            ws = _workspace(lib.cgnet_sparse_forward_stats_workspace(self._h, int(B)), F.device)
            _lib.check(lib.cgnet_sparse_forward_stats(self._h, _ptr(F), _ptr(FF), _ptr(CG), int(B), _ptr(sums),
                                                      _ptr(ws), ws.numel(), _stream(F.device)))

    def forward_stats_static(self, F, FF, CG, B, sums):
        """``forward_stats`` through the entry point that allocates nothing (partial sums in the
        library's fixed area; raises when they do not fit)."""
        self._check_io(F, B)
        _require_gpu("output", FF)
        _require_gpu("CG", CG)
        _require_gpu("sums", sums, torch.float64)
        if FF.numel() != B * self.nFF * 2 or sums.numel() != 2 * self.sum_tFF or CG.numel() < self.cg_len:
            raise RuntimeError("forward_stats_static: tensor sizes do not match the plan")
        with torch.cuda.device(F.device):
            _lib.check(_lib.load().cgnet_sparse_forward_stats_static(self._h, _ptr(F), _ptr(FF), _ptr(CG), int(B),
                                                                     _ptr(sums), _stream(F.device)))

    def backward(self, F, gF, gFF, CG, B):
        self._check_io(F, B)
        _require_gpu("grad_in", gF)
        _require_gpu("grad_out", gFF)
        _require_gpu("CG", CG)
        if gF.numel() != F.numel() or gFF.numel() != B * self.nFF * 2 or CG.numel() < self.cg_len:
            raise RuntimeError("backward: tensor sizes do not match the plan")
        lib = _lib.load()
        with torch.cuda.device(F.device):
            ws = _workspace(lib.cgnet_sparse_backward_workspace(self._h, int(B)), F.device)
            _lib.check(lib.cgnet_sparse_backward(self._h, _ptr(F), _ptr(gF), _ptr(gFF), _ptr(CG), int(B),
                                                 _ptr(ws), ws.numel(), _stream(F.device)))


class WMMPlan:
    """Plan of the fragment norm + weight mixing of one layer (``cgnet_wmm_plan``)."""

    def __init__(self, lmax, t_FF, t_O):
        self.lmax = int(lmax)
        self.t_FF = [int(v) for v in t_FF]
        self.t_O = [int(v) for v in t_O]
        if len(self.t_FF) != self.lmax + 1 or len(self.t_O) != self.lmax + 1:
            raise RuntimeError("t_FF and t_O must have lmax+1 entries")
        lib = _lib.load()
        h = ctypes.c_void_p()
        _lib.check(lib.cgnet_wmm_plan_create(ctypes.byref(h), self.lmax, _lib.int_array(self.t_FF),
                                             _lib.int_array(self.t_O)))
        self._h = h
        sizes = (ctypes.c_int * 4)()
        _lib.check(lib.cgnet_wmm_plan_sizes(self._h, sizes))
        self.nFF, self.nO, self.nW, self.sum_tFF = [int(v) for v in sizes]
        self.gradw_lds = int(lib.cgnet_wmm_plan_gradw_lds(self._h))        # bytes per work-group of the weight gradient

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h is not None and _lib._lib is not None:
            _lib._lib.cgnet_wmm_plan_destroy(h)

    def forward(self, FF, O, W, B, stds, cnt, eps, flags, sums=None):
        _require_gpu("FF", FF)
        _require_gpu("output", O)
        _require_gpu("W", W)
        if flags & _lib.FN_BATCHNORM:
            _require_gpu("FN_stds", stds)
            if stds.numel() != self.sum_tFF:
                raise RuntimeError("FN_stds has %d entries, expected %d" % (stds.numel(), self.sum_tFF))
        else:
            stds = None
        if sums is not None:
            _require_gpu("sums", sums, torch.float64)
        if FF.numel() != B * self.nFF * 2 or O.numel() != B * self.nO * 2 or W.numel() != self.nW * 2:
            raise RuntimeError("FN_WMM_forward: tensor sizes do not match the plan "
                               "(FF %d vs %d, out %d vs %d, W %d vs %d)"
                               % (FF.numel(), B * self.nFF * 2, O.numel(), B * self.nO * 2, W.numel(), self.nW * 2))
        lib = _lib.load()
        with torch.cuda.device(FF.device):
            ws = _workspace(lib.cgnet_FN_WMM_forward_workspace(self._h, int(B)), FF.device)
            _lib.check(lib.cgnet_FN_WMM_forward(self._h, _ptr(FF), _ptr(O), _ptr(W), int(B), _ptr(stds), float(cnt),
                                                float(eps), int(flags), _ptr(sums), _ptr(ws), ws.numel(),
                                                _stream(FF.device)))

    def backward(self, gO, gFF, gW, FF, W, B, stds, eps, flags):
        _require_gpu("grad_out", gO)
        _require_gpu("FF", FF)
        _require_gpu("W", W)
        if gFF is not None:
            _require_gpu("grad_FF", gFF)
        if gW is not None:
            _require_gpu("grad_W", gW)
        if flags & _lib.FN_BATCHNORM:
            _require_gpu("FN_stds", stds)
        else:
            stds = None
        if (gO.numel() != B * self.nO * 2 or FF.numel() != B * self.nFF * 2 or W.numel() != self.nW * 2
                or (gFF is not None and gFF.numel() != FF.numel()) or (gW is not None and gW.numel() != W.numel())):
            raise RuntimeError("FN_WMM_backward: tensor sizes do not match the plan")
        lib = _lib.load()
        gO, FF = _aligned16(gO), _aligned16(FF)
        if gFF is not None and gFF.data_ptr() % 16:
            raise RuntimeError("grad_FF must be 16-byte aligned")
        with torch.cuda.device(FF.device):
            ws = _workspace(lib.cgnet_FN_WMM_backward_workspace(self._h, int(B)), FF.device)
            _lib.check(lib.cgnet_FN_WMM_backward(self._h, _ptr(gO), _ptr(gFF), _ptr(gW), _ptr(FF), _ptr(W), int(B),
                                                 _ptr(stds), float(eps), int(flags), _ptr(ws), ws.numel(),
                                                 _stream(FF.device)))


class LayerPlan:
    """One CGBN layer (``cgnet_layer_plan``): a product plan linked with the mixing plan that consumes its
    output.  Keeps both alive.  ``fused_backward_supported`` says whether ``backward_fused`` takes the layer."""

    def __init__(self, cg_plan, wmm_plan):
        self.cg_plan, self.wmm_plan = cg_plan, wmm_plan
        lib = _lib.load()
        h = ctypes.c_void_p()
        _lib.check(lib.cgnet_layer_plan_create(ctypes.byref(h), cg_plan._h, wmm_plan._h))
        self._h = h
        self.fused_backward_supported = bool(lib.cgnet_CGBN_backward_fused_supported(self._h))
        self.fused_backward_reason = lib.cgnet_CGBN_backward_fused_reason(self._h).decode("utf-8", "replace")
        self.inference_forward_supported = bool(lib.cgnet_CGBN_forward_inference_supported(self._h))
        self.inference_forward_reason = lib.cgnet_CGBN_forward_inference_reason(self._h).decode("utf-8", "replace")
        # the layer may keep its product tensor in a compact layout (one channel per pair of a diagonal triple)
        self.compact_supported = bool(lib.cgnet_CGBN_compact_supported(self._h))

    def internal_nFF(self, flags):
        """Complex entries per sample of the product tensor ``forward`` writes with these flags."""
        return int(_lib.load().cgnet_CGBN_internal_nFF(self._h, int(flags)))

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h is not None and _lib._lib is not None:
            _lib._lib.cgnet_layer_plan_destroy(h)

    def forward(self, F, FF, O, W, CG, B, stds, cnt, eps, flags, save=True):
        """O = layer(F); FF is written too.  Returns the saved-operand tensor for ``backward_fused`` (None when
        ``save`` is false or the fused backward is not supported); ``saved_stds`` is the view of it that holds the
        stds this batch was normalised with."""
        cg, wmm = self.cg_plan, self.wmm_plan
        cg._check_io(F, B)
        _require_gpu("FF", FF)
        _require_gpu("output", O)
        _require_gpu("W", W)
        _require_gpu("CG", CG)
        if flags & _lib.FN_BATCHNORM:
            _require_gpu("FN_stds", stds)
            if stds.numel() != wmm.sum_tFF:
                raise RuntimeError("FN_stds has %d entries, expected %d" % (stds.numel(), wmm.sum_tFF))
        else:
            stds = None
        if (FF.numel() != B * self.internal_nFF(flags) * 2 or O.numel() != B * wmm.nO * 2 or W.numel() != wmm.nW * 2
                or CG.numel() < cg.cg_len):
            raise RuntimeError("CGBN forward: tensor sizes do not match the plans")
        lib = _lib.load()
        with torch.cuda.device(F.device):
            saved = None
            if save and self.fused_backward_supported:
                saved = _workspace(lib.cgnet_CGBN_saved_bytes(self._h, int(B)), F.device)
            ws = _workspace(lib.cgnet_CGBN_forward_workspace(self._h, int(B)), F.device)
            _lib.check(lib.cgnet_CGBN_forward(self._h, _ptr(F), _ptr(FF), _ptr(O), _ptr(W), _ptr(CG), int(B), _ptr(stds),
                                              float(cnt), float(eps), int(flags), _ptr(saved),
                                              0 if saved is None else saved.numel(), _ptr(ws), ws.numel(),
                                              _stream(F.device)))
        return saved

    def forward_inference(self, F, O, W, CG, B, stds, eps, flags):
        """O = layer(F) without FF in memory (cgnet_CGBN_forward_inference): evaluation mode, no gradient."""
        cg, wmm = self.cg_plan, self.wmm_plan
        cg._check_io(F, B)
        _require_gpu("output", O)
        _require_gpu("W", W)
        _require_gpu("CG", CG)
        if flags & _lib.FN_BATCHNORM:
            _require_gpu("FN_stds", stds)
            if stds.numel() != wmm.sum_tFF:
                raise RuntimeError("FN_stds has %d entries, expected %d" % (stds.numel(), wmm.sum_tFF))
        else:
            stds = None
        if O.numel() != B * wmm.nO * 2 or W.numel() != wmm.nW * 2 or CG.numel() < cg.cg_len:
            raise RuntimeError("CGBN inference forward: tensor sizes do not match the plans")
        lib = _lib.load()
        with torch.cuda.device(F.device):
            ws = _workspace(lib.cgnet_CGBN_forward_inference_workspace(self._h, int(B)), F.device)
            _lib.check(lib.cgnet_CGBN_forward_inference(self._h, _ptr(F), _ptr(O), _ptr(W), _ptr(CG), int(B), _ptr(stds),
                                                        float(eps), int(flags), _ptr(ws), ws.numel(), _stream(F.device)))

    def saved_stds(self, saved, B):
        """The float32 view of the stds copy inside a saved-operand tensor (None if it holds none)."""
        if saved is None:
            return None
        n = int(_lib.load().cgnet_CGBN_saved_stds_bytes(self._h, int(B)))
        return saved[:n].view(torch.float32) if n else None

    def backward_fused(self, F, gF, gO, W, CG, B, stds, eps, flags, saved=None):
        """gF of the whole layer straight from gO (no gFF in memory): cgnet_CGBN_backward_fused."""
        cg, wmm = self.cg_plan, self.wmm_plan
        _require_gpu("input", F)
        _require_gpu("grad_in", gF)
        _require_gpu("grad_out", gO)
        _require_gpu("W", W)
        _require_gpu("CG", CG)
        if flags & _lib.FN_BATCHNORM:
            _require_gpu("FN_stds", stds)
        else:
            stds = None
        if (F.numel() != B * cg.nF * 2 or gF.numel() != F.numel() or gO.numel() != B * wmm.nO * 2
                or W.numel() != wmm.nW * 2 or CG.numel() < cg.cg_len):
            raise RuntimeError("fused backward: tensor sizes do not match the plans")
        lib = _lib.load()
        with torch.cuda.device(F.device):
            ws = _workspace(lib.cgnet_CGBN_backward_fused_workspace(self._h, int(B)), F.device)
            _lib.check(lib.cgnet_CGBN_backward_fused(self._h, _ptr(F), _ptr(gF), _ptr(gO), _ptr(W), _ptr(CG), int(B),
                                                     _ptr(stds), float(eps), int(flags), _ptr(saved),
                                                     0 if saved is None else saved.numel(), _ptr(ws), ws.numel(),
                                                     _stream(F.device)))

    def backward_gradw(self, gO, FF, gW, B, stds, eps, flags):
        """gW of the layer from gO and the product tensor ``forward`` wrote with the same flags
        (cgnet_CGBN_backward_gradw)."""
        wmm = self.wmm_plan
        _require_gpu("grad_out", gO)
        _require_gpu("FF", FF)
        _require_gpu("grad_W", gW)
        if flags & _lib.FN_BATCHNORM:
            _require_gpu("FN_stds", stds)
        else:
            stds = None
        if (gO.numel() != B * wmm.nO * 2 or FF.numel() != B * self.internal_nFF(flags) * 2 or gW.numel() != wmm.nW * 2):
            raise RuntimeError("layer weight gradient: tensor sizes do not match the plans")
        gO, FF = _aligned16(gO), _aligned16(FF)
        lib = _lib.load()
        with torch.cuda.device(gO.device):
            ws = _workspace(lib.cgnet_CGBN_backward_gradw_workspace(self._h, int(B), int(flags)), gO.device)
            _lib.check(lib.cgnet_CGBN_backward_gradw(self._h, _ptr(gO), _ptr(FF), _ptr(gW), int(B), _ptr(stds), float(eps),
                                                     int(flags), _ptr(ws), ws.numel(), _stream(gO.device)))
