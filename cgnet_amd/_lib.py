"""ctypes binding of libcgnet_hip.so (C ABI declared in include/cgnet_hip.h).

The library is built in-tree by ``make -C cgnet_amd/csrc`` (``__graft_entry__.build()``).
There is no fallback: if the shared object is missing every operation raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# CGNET_HIP_LIBRARY names another build of the same library (kernel experiments); the default is the in-tree one
LIB_PATH = os.environ.get("CGNET_HIP_LIBRARY") or os.path.join(_HERE, "csrc", "libcgnet_hip.so")

OK, ERR_ARG, ERR_HIP, ERR_WORKSPACE, ERR_UNSUPPORTED = 0, -1, -2, -3, -4
FN_BATCHNORM, FN_UPDATE_STD = 0x1, 0x2
LAYER_COMPACT_FF = 0x4     # cgnet_CGBN_forward / _backward_gradw: product tensor in the layer's compact layout

_c_int_p = ctypes.POINTER(ctypes.c_int)
_vp = ctypes.c_void_p

# name -> (restype, argtypes); the single source for the binding and for the symbol test
SIGNATURES = {
    "cgnet_last_error": (ctypes.c_char_p, []),
    "cgnet_abi_version": (ctypes.c_int, []),
    "cgnet_sparse_maxL": (ctypes.c_int, []),
    "cgnet_sparse_precomputeCG": (ctypes.c_int, [_vp, ctypes.c_int, _c_int_p, ctypes.c_int, _c_int_p, _vp]),
    "cgnet_cg_plan_create": (ctypes.c_int, [ctypes.POINTER(_vp), ctypes.c_int, _c_int_p, _c_int_p, ctypes.c_int,
                                            _c_int_p, _c_int_p]),
    "cgnet_cg_plan_destroy": (ctypes.c_int, [_vp]),
    "cgnet_cg_plan_sizes": (ctypes.c_int, [_vp, _c_int_p]),
    "cgnet_cg_plan_channels": (ctypes.c_int, [_vp, _c_int_p, _c_int_p]),
    "cgnet_sparse_forward": (ctypes.c_int, [_vp, _vp, _vp, _vp, ctypes.c_int, _vp]),
    "cgnet_sparse_forward_stats_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_sparse_forward_stats": (ctypes.c_int, [_vp, _vp, _vp, _vp, ctypes.c_int, _vp, _vp, ctypes.c_size_t, _vp]),
    "cgnet_sparse_forward_stats_static_limit": (ctypes.c_size_t, []),
    "cgnet_sparse_forward_stats_static": (ctypes.c_int, [_vp, _vp, _vp, _vp, ctypes.c_int, _vp, _vp]),
    "cgnet_sparse_backward_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_sparse_backward": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_size_t, _vp]),
    "cgnet_wmm_plan_create": (ctypes.c_int, [ctypes.POINTER(_vp), ctypes.c_int, _c_int_p, _c_int_p]),
    "cgnet_wmm_plan_destroy": (ctypes.c_int, [_vp]),
    "cgnet_wmm_plan_sizes": (ctypes.c_int, [_vp, _c_int_p]),
    "cgnet_FN_WMM_forward_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_FN_WMM_forward": (ctypes.c_int, [_vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_float, ctypes.c_float,
                                            ctypes.c_int, _vp, _vp, ctypes.c_size_t, _vp]),
    "cgnet_FN_WMM_backward_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_FN_WMM_backward": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_float,
                                             ctypes.c_int, _vp, ctypes.c_size_t, _vp]),
    "cgnet_layer_plan_create": (ctypes.c_int, [ctypes.POINTER(_vp), _vp, _vp]),
    "cgnet_layer_plan_destroy": (ctypes.c_int, [_vp]),
    "cgnet_CGBN_backward_fused_supported": (ctypes.c_int, [_vp]),
    "cgnet_CGBN_backward_fused_reason": (ctypes.c_char_p, [_vp]),
    "cgnet_CGBN_saved_bytes": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_CGBN_saved_stds_bytes": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_CGBN_forward_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_CGBN_forward": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_float,
                                          ctypes.c_float, ctypes.c_int, _vp, ctypes.c_size_t, _vp, ctypes.c_size_t, _vp]),
    "cgnet_CGBN_backward_fused_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_CGBN_backward_fused": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_float,
                                                 ctypes.c_int, _vp, ctypes.c_size_t, _vp, ctypes.c_size_t, _vp]),
    "cgnet_CGBN_forward_inference_supported": (ctypes.c_int, [_vp]),
    "cgnet_CGBN_forward_inference_reason": (ctypes.c_char_p, [_vp]),
    "cgnet_CGBN_forward_inference_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_CGBN_forward_inference": (ctypes.c_int, [_vp, _vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_float, ctypes.c_int,
                                                    _vp, ctypes.c_size_t, _vp]),
    "cgnet_CGBN_compact_supported": (ctypes.c_int, [_vp]),
    "cgnet_CGBN_internal_nFF": (ctypes.c_size_t, [_vp, ctypes.c_int]),
    "cgnet_CGBN_backward_gradw_workspace": (ctypes.c_size_t, [_vp, ctypes.c_int, ctypes.c_int]),
    "cgnet_CGBN_backward_gradw": (ctypes.c_int, [_vp, _vp, _vp, _vp, ctypes.c_int, _vp, ctypes.c_float, ctypes.c_int,
                                                 _vp, ctypes.c_size_t, _vp]),
    "cgnet_cg_plan_backward_lds": (ctypes.c_size_t, [_vp]),
    "cgnet_cg_plan_forward_lds": (ctypes.c_size_t, [_vp]),
    "cgnet_cg_plan_backward_groups": (ctypes.c_int, [_vp]),
    "cgnet_wmm_plan_gradw_lds": (ctypes.c_size_t, [_vp]),
    "cgnet_profile_enable": (ctypes.c_int, [ctypes.c_int]),
    "cgnet_profile_select": (ctypes.c_int, [ctypes.c_char_p]),
    "cgnet_profile_reset": (ctypes.c_int, []),
    "cgnet_profile_collect": (ctypes.c_int, []),
    "cgnet_profile_get": (ctypes.c_int, [ctypes.c_int, ctypes.c_char_p, ctypes.c_int,
                                         ctypes.POINTER(ctypes.c_double), _c_int_p]),
}

_lib = None


class CgnetError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("libcgnet_hip error %d: %s" % (code, message))
        self.code = code


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError("%s is missing: build it with `make -C cgnet_amd/csrc` "
                           "(or __graft_entry__.build()); there is no CPU fallback" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code):
    if code != OK:
        raise CgnetError(code, load().cgnet_last_error().decode("utf-8", "replace"))


def int_array(values):
    values = [int(v) for v in values]
    return (ctypes.c_int * max(1, len(values)))(*values)


def kernel_times():
    """{kernel name: (total milliseconds, launches)} gathered since the last reset.
    The caller must have synchronised the device first."""
    lib = load()
    n = lib.cgnet_profile_collect()
    out = {}
    buf = ctypes.create_string_buffer(128)
    for i in range(n):
        ms, cnt = ctypes.c_double(), ctypes.c_int()
        check(lib.cgnet_profile_get(i, buf, len(buf), ctypes.byref(ms), ctypes.byref(cnt)))
        name = buf.value.decode().split("<")[0]      # template instances of one kernel are added up
        prev = out.get(name, (0.0, 0))
        out[name] = (prev[0] + ms.value, prev[1] + cnt.value)
    return out
