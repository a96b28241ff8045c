"""Drop-in for the reference's native operator module ``CG_cuda_ops``
(pybind11 module of CGNet/cudaCG/cudaCG_all.cpp:207-215): the same six functions with the
same positional arguments, implemented on libcgnet_hip through its C ABI.

The reference passes the per-degree metadata as int32 GPU tensors on every call.  Here they
identify a cached native plan: the first call with a given set of metadata tensors copies them
to the host once and builds the plan; later calls find it by tensor identity and never
synchronise.  ``register_cg_plan`` / ``register_wmm_plan`` let a module that already knows the
host values seed the cache so that no copy happens at all.
"""
import collections

import torch

from . import _lib
from ._plans import CGPlan, WMMPlan, fill_cg_table

_CACHE_SIZE = 256
_cg_cache = collections.OrderedDict()     # key -> (tensors kept alive, versions, plan)
_wmm_cache = collections.OrderedDict()


def _key(tensors):
    return tuple((t.data_ptr(), t.numel()) for t in tensors)


def _lookup(cache, tensors):
    ent = cache.get(_key(tensors))
    if ent is None:
        return None
    kept, versions, plan = ent
    if any(a is not b for a, b in zip(kept, tensors)) or versions != tuple(t._version for t in tensors):
        return None
    cache.move_to_end(_key(tensors))
    return plan


def _store(cache, tensors, plan):
    cache[_key(tensors)] = (tuple(tensors), tuple(t._version for t in tensors), plan)
    while len(cache) > _CACHE_SIZE:
        cache.popitem(last=False)


def _host(t):
    return t.detach().to("cpu").reshape(-1).tolist()


def _check_input(name, t):
    # same contract as CHECK_INPUT at cudaCG_all.cpp:34-36
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)


def register_cg_plan(plan, t_F, llls, t_offsets):
    """Associate an existing plan with the metadata tensors a caller will pass."""
    _store(_cg_cache, (t_F, llls, t_offsets), plan)


def register_wmm_plan(plan, t_FF, cumu_tm_O):
    _store(_wmm_cache, (t_FF, cumu_tm_O), plan)


def _cg_plan(L, t_F, llls, t_offsets, CG_offsets):
    plan = _lookup(_cg_cache, (t_F, llls, t_offsets))
    if plan is None:
        plan = CGPlan(L, _host(t_F), _host(llls), _host(t_offsets), _host(CG_offsets))
        _store(_cg_cache, (t_F, llls, t_offsets), plan)
    return plan


def _wmm_plan(L, t_FF, cumu_tm_O):
    plan = _lookup(_wmm_cache, (t_FF, cumu_tm_O))
    if plan is None:
        cum = _host(cumu_tm_O)
        t_O = []
        for l in range(L + 1):
            width = cum[l + 1] - cum[l]
            if width % (2 * l + 1):
                raise RuntimeError("cumu_tm_O is not a cumulative sum of t_O[l]*(2l+1)")
            t_O.append(width // (2 * l + 1))
        plan = WMMPlan(L, _host(t_FF), t_O)
        _store(_wmm_cache, (t_FF, cumu_tm_O), plan)
    return plan


# ------------------------------------------------------------------ the six reference functions
def sparse_maxL():
    return int(_lib.load().cgnet_sparse_maxL())


def sparse_precomputeCG(CG_tensor, L, llls, CG_offsets):
    _check_input("CG_tensor", CG_tensor)
    fill_cg_table(CG_tensor, L, _host(llls), _host(CG_offsets))
    return 0


def sparse_forward(input, output, L, B, t_F, cumu_tm_F, t_FF, cumu_tm_FF, llls, ll1_to_lllidx, t_offsets,
                   CG, CG_offsets):
    for n, t in (("input", input), ("output", output), ("t_F", t_F), ("cumu_tm_F", cumu_tm_F), ("t_FF", t_FF),
                 ("cumu_tm_FF", cumu_tm_FF), ("llls", llls), ("ll1_to_lllidx", ll1_to_lllidx),
                 ("t_offsets", t_offsets), ("CG", CG), ("CG_offsets", CG_offsets)):
        _check_input(n, t)
    _cg_plan(int(L), t_F, llls, t_offsets, CG_offsets).forward(input, output, CG, int(B))
    return 0


def sparse_backward(input, grad_in, grad_out, L, B, t_F, cumu_tm_F, t_FF, cumu_tm_FF, llls, t_offsets, CG,
                    CG_offsets):
    for n, t in (("input", input), ("grad_in", grad_in), ("grad_out", grad_out), ("t_F", t_F),
                 ("cumu_tm_F", cumu_tm_F), ("t_FF", t_FF), ("cumu_tm_FF", cumu_tm_FF), ("llls", llls),
                 ("t_offsets", t_offsets), ("CG", CG), ("CG_offsets", CG_offsets)):
        _check_input(n, t)
    _cg_plan(int(L), t_F, llls, t_offsets, CG_offsets).backward(input, grad_in, grad_out, CG, int(B))
    return 0


def FN_WMM_forward(FF_tensor, output_tensor, W_tensor, L, B, size_FN, size_WMM, t_FF, cumu_tm_FF, cumu_tm_O,
                   cumu_tt_W, FN_stds_tensor, FN_cnt, FN_eps, FN_flags):
    for n, t in (("FF_tensor", FF_tensor), ("output_tensor", output_tensor), ("W_tensor", W_tensor),
                 ("t_FF", t_FF), ("cumu_tm_FF", cumu_tm_FF), ("cumu_tm_O", cumu_tm_O), ("cumu_tt_W", cumu_tt_W)):
        _check_input(n, t)
    flags = int(FN_flags)
    stds = None
    if flags & _lib.FN_BATCHNORM:
        _check_input("FN_stds_tensor", FN_stds_tensor)
        stds = FN_stds_tensor
    plan = _wmm_plan(int(L), t_FF, cumu_tm_O)
    if int(size_FN) != plan.sum_tFF or int(size_WMM) != plan.nO:
        raise RuntimeError("size_FN / size_WMM (%d, %d) do not match the metadata (%d, %d)"
                           % (size_FN, size_WMM, plan.sum_tFF, plan.nO))
    plan.forward(FF_tensor, output_tensor, W_tensor, int(B), stds, float(FN_cnt), float(FN_eps), flags)
    return 0


def FN_WMM_backward(grad_out_tensor, grad_FF_tensor, grad_W_tensor, FF_tensor, W_tensor, L, B, size_FF, size_W,
                    t_FF, cumu_tm_FF, t_O, cumu_tm_O, cumu_tt_W, FN_stds_tensor, FN_cnt, FN_eps, FN_flags):
    for n, t in (("grad_out_tensor", grad_out_tensor), ("grad_FF_tensor", grad_FF_tensor),
                 ("grad_W_tensor", grad_W_tensor), ("FF_tensor", FF_tensor), ("W_tensor", W_tensor),
                 ("t_FF", t_FF), ("cumu_tm_FF", cumu_tm_FF), ("t_O", t_O), ("cumu_tm_O", cumu_tm_O),
                 ("cumu_tt_W", cumu_tt_W)):
        _check_input(n, t)
    flags = int(FN_flags)
    stds = None
    if flags & _lib.FN_BATCHNORM:
        _check_input("FN_stds_tensor", FN_stds_tensor)
        stds = FN_stds_tensor
    plan = _wmm_plan(int(L), t_FF, cumu_tm_O)
    if int(size_FF) != plan.nFF or int(size_W) != plan.nW:
        raise RuntimeError("size_FF / size_W (%d, %d) do not match the metadata (%d, %d)"
                           % (size_FF, size_W, plan.nFF, plan.nW))
    plan.backward(grad_out_tensor, grad_FF_tensor, grad_W_tensor, FF_tensor, W_tensor, int(B), stds,
                  float(FN_eps), flags)
    return 0
