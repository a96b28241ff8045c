"""CPU checks of the C ABI: the built library loads, exports every function the header declares,
the ctypes binding covers them all, and argument validation that needs no device works."""
import ctypes
import os
import re

import pytest

from cgnet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "cgnet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cgnet_[A-Za-z0-9_]+)\s*\(", text)))


def test_header_declares_the_reference_operator_set():
    names = declared_functions()
    for required in ("cgnet_sparse_precomputeCG", "cgnet_sparse_forward", "cgnet_sparse_backward",
                     "cgnet_sparse_maxL", "cgnet_FN_WMM_forward", "cgnet_FN_WMM_backward"):
        assert required in names


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), "libcgnet_hip.so does not export %s" % name
        assert name in _lib.SIGNATURES, "ctypes binding lacks %s" % name
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_no_torch_types_in_the_abi():
    text = open(os.path.join(ROOT, "include", "cgnet_hip.h")).read()
    assert "torch" not in text.replace("pytorch", "").lower().replace("the reference binds", "")
    assert "#include <torch" not in text and "at::" not in text


def test_host_side_argument_validation():
    lib = _lib.load()
    assert lib.cgnet_abi_version() == 1
    assert lib.cgnet_sparse_maxL() >= 20
    h = ctypes.c_void_p()
    taus = _lib.int_array([1, 1, 1])
    assert lib.cgnet_cg_plan_create(ctypes.byref(h), 999, taus, None, 0, None, None) == _lib.ERR_UNSUPPORTED
    assert b"lmax" in lib.cgnet_last_error()
    assert lib.cgnet_cg_plan_create(None, 2, taus, None, 0, None, None) == _lib.ERR_ARG
    assert lib.cgnet_cg_plan_create(ctypes.byref(h), 2, None, None, 0, None, None) == _lib.ERR_ARG
    # l1 < l2 is rejected before any device call: code (l=1, l1=0, l2=1) for lmax=2
    bad = _lib.int_array([(1 * 3 + 0) * 3 + 1])
    assert lib.cgnet_cg_plan_create(ctypes.byref(h), 2, taus, bad, 1, None, None) == _lib.ERR_ARG
    assert b"triangle" in lib.cgnet_last_error() or b"l1>=l2" in lib.cgnet_last_error()
    # triangle rule: (l=2, l1=0, l2=0)
    bad = _lib.int_array([(2 * 3 + 0) * 3 + 0])
    assert lib.cgnet_cg_plan_create(ctypes.byref(h), 2, taus, bad, 1, None, None) == _lib.ERR_ARG
    # unordered output degrees
    bad = _lib.int_array([(1 * 3 + 1) * 3 + 0, (0 * 3 + 0) * 3 + 0])
    assert lib.cgnet_cg_plan_create(ctypes.byref(h), 2, taus, bad, 2, None, None) == _lib.ERR_ARG
    # wrong t_offsets
    good = _lib.int_array([(0 * 3 + 0) * 3 + 0, (0 * 3 + 1) * 3 + 1])
    assert lib.cgnet_cg_plan_create(ctypes.byref(h), 2, taus, good, 2, _lib.int_array([0, 7]), None) == _lib.ERR_ARG
    assert lib.cgnet_wmm_plan_create(ctypes.byref(h), 2, None, None) == _lib.ERR_ARG
    assert lib.cgnet_wmm_plan_create(ctypes.byref(h), 2, _lib.int_array([1, -1, 1]), taus) == _lib.ERR_ARG
    assert lib.cgnet_sparse_precomputeCG(None, 2, good, 2, _lib.int_array([0, 1, 4]), None) == _lib.ERR_ARG
    assert lib.cgnet_sparse_forward(None, None, None, None, 1, None) == _lib.ERR_ARG
    assert lib.cgnet_FN_WMM_forward(None, None, None, None, 1, None, 1.0, 1e-5, 0, None, None, 0, None) == _lib.ERR_ARG
    assert h.value is None


def test_modules_hold_reference_parameter_layout_without_a_gpu():
    import math
    from cgnet_amd import CGNet
    lmax = 10
    taus = [int(math.ceil(12 / math.sqrt(2 * l + 1.0))) for l in range(lmax + 1)]
    net = CGNet.SphericalCNN(lmax, [[1] * (lmax + 1)] + [taus] * 5, device="cpu")
    shapes = [tuple(p.shape) for p in net.parameters() if p.requires_grad]
    assert shapes == [(1643, 2)] + [(31023, 2)] * 4          # MNIST/example.sh:12 of the reference
    # the state dictionary holds exactly the reference's entries (CGNet/CG_layers.py:89-91,116-122: three Parameters per
    # layer, nothing else), so checkpoints pass the reference's strict load_state_dict in both directions
    want = {"cgs.%d.bnWMM.%s" % (i, k) for i in range(5) for k in ("W", "bn_stds", "bn_eps")}
    assert set(net.state_dict().keys()) == want
    # opt-in: the moving-average count as a fourth entry (the reference loses it on a resume)
    from cgnet_amd import CG_layers
    net.cgs[2].bnWMM.persist_bn_cnt = True
    net.cgs[2].bnWMM.bn_cnt = 5.0
    sd = net.state_dict()
    assert set(sd.keys()) == want | {"cgs.2.bnWMM.bn_cnt"} and float(sd["cgs.2.bnWMM.bn_cnt"]) == 5.0
    net.cgs[2].bnWMM.bn_cnt = 1.0
    net.load_state_dict(sd)                                   # strict: the extra entry is consumed, not "unexpected"
    assert net.cgs[2].bnWMM.bn_cnt == 5.0
    net.cgs[2].bnWMM.persist_bn_cnt = False
    assert not CG_layers.MyBatchNormWeightMM_cuda.persist_bn_cnt
    net.load_state_dict({k: v for k, v in sd.items() if not k.endswith("bn_cnt")})   # a reference checkpoint
    assert net.cgs[2].bnWMM.bn_cnt == 5.0                     # ... leaves the count alone
    assert net.output_length == 122
    import torch
    with pytest.raises(AssertionError):
        net(torch.zeros(2, 121, 2))                           # no CPU path: GPU tensors only
    layer = net.cgs[1]
    assert not layer.sparse_flag and layer.bnWMM.bn_cnt == 1.0
    assert float(layer.bnWMM.W.min()) >= 0 and float(layer.bnWMM.W.max()) <= 0.05
