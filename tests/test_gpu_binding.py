"""The reference-side binding: ``cgnet_amd.CG_cuda_ops`` driven exactly the way the reference's own autograd
Functions drive their pybind11 module (CGNet/CG_layers.py:16-72,171-203; cudaCG_all.cpp:207-215) -- pre-zeroed
outputs, int32 GPU tensors for every piece of metadata, ``int(t_FF.sum())`` / ``int(cumu_tm_O[-1])`` sizes, the
``bn_eps`` tensor handed over as a dummy ``FN_stds`` when the fragment norm is off, flags 0x1 / 0x2 -- and the
reference's own differential case (CGNet/test.py:33-37,115-130).  Everything is compared with the CPU oracle."""
import math

import numpy as np
import pytest
import torch

from oracle import cg_coeff as OC
from oracle import cg_layer as OL
from oracle import triples as OT
from test_gpu_parity import F32, F64, assert_close, dev, make_oracle, oracle_step, rand_straight, randn32  # noqa: F401

pytestmark = pytest.mark.gpu


class RefStyleCG(torch.autograd.Function):
    """Call shape of the reference's ``_CG_sparse_cuda`` (CG_layers.py:171-203)."""

    @staticmethod
    def forward(ctx, Fs, output_length, t_F, cumu_tm_F, t_FF, cumu_tm_FF, llls, l_l1_to_lllidx_offsets, t_offsets,
                CG, CG_offsets):
        from cgnet_amd import CG_cuda_ops
        lmax = len(t_F) - 1
        assert lmax <= CG_cuda_ops.sparse_maxL()
        ctx.save_for_backward(Fs, t_F, cumu_tm_F, t_FF, cumu_tm_FF, llls, l_l1_to_lllidx_offsets, t_offsets, CG, CG_offsets)
        output = torch.zeros(Fs.shape[0], output_length, 2, device=Fs.device, dtype=torch.float)
        assert CG_cuda_ops.sparse_forward(Fs, output, t_F.shape[0] - 1, Fs.shape[0], t_F, cumu_tm_F, t_FF, cumu_tm_FF,
                                          llls, l_l1_to_lllidx_offsets, t_offsets, CG, CG_offsets) == 0
        return output

    @staticmethod
    def backward(ctx, grad_output):
        from cgnet_amd import CG_cuda_ops
        Fs, t_F, cumu_tm_F, t_FF, cumu_tm_FF, llls, _, t_offsets, CG, CG_offsets = ctx.saved_tensors
        grad_input = torch.zeros(Fs.shape, dtype=torch.float, device=grad_output.device)
        assert CG_cuda_ops.sparse_backward(Fs, grad_input, grad_output.contiguous(), t_F.shape[0] - 1, Fs.shape[0], t_F,
                                           cumu_tm_F, t_FF, cumu_tm_FF, llls, t_offsets, CG, CG_offsets) == 0
        return (grad_input,) + (None,) * 10


class RefStyleWMM(torch.autograd.Function):
    """Call shape of the reference's ``_MyBatchNormWeightMM_cuda`` (CG_layers.py:16-72)."""

    @staticmethod
    def forward(ctx, FF, W, t_FF, cumu_tm_FF, t_O, cumu_tm_O, cumu_tt_W, bn_stds, bn_cnt, bn_eps, bn_updateflag):
        from cgnet_amd import CG_cuda_ops
        ctx.lmax, ctx.B = t_FF.shape[0] - 1, FF.shape[0]
        output = torch.zeros(FF.shape[0], int(cumu_tm_O[-1]), 2, device=FF.device, dtype=torch.float)
        flags = (0x1 if bn_stds is not None else 0) + (0x2 if bn_updateflag else 0)
        assert CG_cuda_ops.FN_WMM_forward(FF, output, W, ctx.lmax, ctx.B, int(t_FF.sum()), int(cumu_tm_O[-1]), t_FF,
                                          cumu_tm_FF, cumu_tm_O, cumu_tt_W, bn_eps if bn_stds is None else bn_stds,
                                          bn_cnt, bn_eps, flags) == 0
        if bn_stds is not None:
            bn_stds = bn_stds.clone()
        ctx.bn_cnt, ctx.bn_eps, ctx.flags = bn_cnt, bn_eps, flags
        ctx.save_for_backward(FF, W, t_FF, cumu_tm_FF, t_O, cumu_tm_O, cumu_tt_W, bn_stds)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        from cgnet_amd import CG_cuda_ops
        FF, W, t_FF, cumu_tm_FF, t_O, cumu_tm_O, cumu_tt_W, bn_stds = ctx.saved_tensors
        grad_FF = torch.zeros(FF.shape, dtype=torch.float, device=grad_output.device)
        grad_W = torch.zeros(W.shape, dtype=torch.float, device=grad_output.device)
        assert CG_cuda_ops.FN_WMM_backward(grad_output.contiguous(), grad_FF, grad_W, FF, W, ctx.lmax, ctx.B,
                                           int(cumu_tm_FF[-1]), int(cumu_tt_W[-1]), t_FF, cumu_tm_FF, t_O, cumu_tm_O,
                                           cumu_tt_W, ctx.bn_eps if bn_stds is None else bn_stds, ctx.bn_cnt,
                                           ctx.bn_eps, ctx.flags) == 0
        return (grad_FF, grad_W) + (None,) * 9


def device_metadata(lmax, taus, tout, pairs, dev):
    """Every int32 GPU tensor the reference's modules build (CG_layers.py:86-98,218-250), from the oracle's lists."""
    i32 = dict(dtype=torch.int32, device=dev)
    codes, lookup = OT.encode_sorted(pairs)
    t_ff, t_off = OT.product_taus(lmax, codes, taus)
    table, cg_offs = OC.flat_cg_table(OT.decode(lmax, codes), dtype=np.float32)
    md = {
        "t_F": torch.tensor(taus, **i32), "cumu_tm_F": torch.tensor(OT.cumulative_tm(taus), **i32),
        "t_FF": torch.tensor(t_ff, **i32), "cumu_tm_FF": torch.tensor(OT.cumulative_tm(t_ff), **i32),
        "t_O": torch.tensor(tout, **i32), "cumu_tm_O": torch.tensor(OT.cumulative_tm(tout), **i32),
        "cumu_tt_W": torch.tensor(OT.cumulative_w(t_ff, tout), **i32),
        "llls": torch.tensor(codes, **i32), "t_offsets": torch.tensor(t_off, **i32),
        "CG_offsets": torch.tensor([int(v) for v in cg_offs], **i32),
        "ll1": torch.tensor(lookup, **i32),
    }
    return md, codes, t_ff, table, cg_offs


@pytest.mark.parametrize("bn,update", [(True, True), (True, False), (False, False)])
def test_six_functions_in_the_reference_call_shape(dev, monkeypatch, bn, update):
    from cgnet_amd import CG_cuda_ops
    built = {"cg": 0, "wmm": 0}
    real_cg, real_wmm = CG_cuda_ops.CGPlan, CG_cuda_ops.WMMPlan

    def counting(kind, cls):
        def make(*a, **k):
            built[kind] += 1
            return cls(*a, **k)
        return make
    monkeypatch.setattr(CG_cuda_ops, "CGPlan", counting("cg", real_cg))
    monkeypatch.setattr(CG_cuda_ops, "WMMPlan", counting("wmm", real_wmm))

    lmax, taus, tout, bsz = 4, [3, 2, 1, 2, 2], [2, 3, 1, 2, 1], 5
    md, codes, t_ff, table, cg_offs = device_metadata(lmax, taus, tout, OT.default_pairs(lmax), dev)
    assert CG_cuda_ops.sparse_maxL() >= lmax

    # 1. the table
    cg = torch.zeros(int(cg_offs[-1]), dtype=torch.float, device=dev)
    assert CG_cuda_ops.sparse_precomputeCG(cg, lmax, md["llls"], md["CG_offsets"]) == 0
    assert np.max(np.abs(cg.cpu().numpy() - table)) <= 1.2e-7

    # 2.-5. product and mixing, forward and backward, chained as the reference's CGBN_cuda.forward chains them
    g = torch.Generator().manual_seed(9)
    x64 = rand_straight(taus, bsz, seed=8)
    w64 = torch.cat([torch.randn(t_ff[l] * tout[l], 2, generator=g, dtype=torch.float64) / math.sqrt(t_ff[l])
                     for l in range(lmax + 1)]).float().double()
    stds = (0.05 + 0.2 * torch.rand(sum(t_ff), generator=g, dtype=torch.float64)).float()
    go64 = randn32((bsz, int(md["cumu_tm_O"][-1]), 2), g)
    bn_eps = torch.nn.Parameter(1e-5 * torch.ones(1, device=dev), requires_grad=False)
    cnt = 4.0

    def run_gpu():
        x = x64.float().to(dev).requires_grad_(True)
        w = w64.float().to(dev).requires_grad_(True)
        bn_stds = stds.clone().to(dev) if bn else None
        ff = RefStyleCG.apply(x, int(md["cumu_tm_FF"][-1]), md["t_F"], md["cumu_tm_F"], md["t_FF"], md["cumu_tm_FF"],
                              md["llls"], md["ll1"], md["t_offsets"], cg, md["CG_offsets"])
        out = RefStyleWMM.apply(ff, w, md["t_FF"], md["cumu_tm_FF"], md["t_O"], md["cumu_tm_O"], md["cumu_tt_W"],
                                bn_stds, cnt, bn_eps, update)
        out.backward(go64.float().to(dev))
        return out, x.grad, w.grad, bn_stds

    def run_oracle(dtype):
        ora = make_oracle(lmax, taus, tout, codes, bn, stds, dtype)
        ora.cnt, ora.training = cnt, update
        res = oracle_step(ora, x64, w64, go64, dtype)
        return res + ((torch.from_numpy(ora.stds_flat().astype(np.float64)),) if bn else (None,))

    out, gx, gw, new_stds = run_gpu()
    assert built == {"cg": 1, "wmm": 1}                   # the first call copied the metadata to the host once
    want, tw = run_oracle(F64), run_oracle(F32)
    assert_close(out, want[0], "binding forward", tw[0])
    assert_close(gx, want[1], "binding grad F", tw[1])
    assert_close(gw, want[2], "binding grad W", tw[2])
    if bn:
        assert_close(new_stds, want[3], "binding running stds", tw[3], rtol=5e-6, atol=1e-8)
        if not update:
            assert torch.equal(new_stds.cpu(), stds)

    # 6. the plan cache: same metadata tensors -> no new plan, no host copy ...
    copies = {"n": 0}
    real_host = CG_cuda_ops._host

    def counting_host(t):
        copies["n"] += 1
        return real_host(t)
    monkeypatch.setattr(CG_cuda_ops, "_host", counting_host)
    out2, gx2, gw2, _ = run_gpu()
    assert built == {"cg": 1, "wmm": 1} and copies["n"] == 0
    assert torch.equal(out2, out) and torch.equal(gx2, gx) and torch.equal(gw2, gw)
    # ... an in-place edit of a metadata tensor (same storage, new version) -> the plans are rebuilt from its new content
    md["t_offsets"].copy_(md["t_offsets"].clone())
    md["t_FF"].add_(0)
    out3, _, _, _ = run_gpu()
    assert built == {"cg": 2, "wmm": 2} and copies["n"] > 0
    assert torch.equal(out3, out)

    # size arguments that contradict the metadata are refused (the reference would read out of bounds)
    with pytest.raises(RuntimeError):
        CG_cuda_ops.FN_WMM_forward(torch.zeros(bsz, int(md["cumu_tm_FF"][-1]), 2, device=dev),
                                   torch.zeros(bsz, int(md["cumu_tm_O"][-1]), 2, device=dev), w64.float().to(dev), lmax, bsz,
                                   int(md["t_FF"].sum()) + 1, int(md["cumu_tm_O"][-1]), md["t_FF"], md["cumu_tm_FF"],
                                   md["cumu_tm_O"], md["cumu_tt_W"], bn_eps, cnt, bn_eps, 0)
    with pytest.raises(RuntimeError):                     # CPU tensor: CHECK_INPUT of cudaCG_all.cpp:34-36
        CG_cuda_ops.sparse_forward(torch.zeros(bsz, int(md["cumu_tm_F"][-1]), 2), torch.zeros(1, device=dev), lmax, bsz,
                                   md["t_F"], md["cumu_tm_F"], md["t_FF"], md["cumu_tm_FF"], md["llls"], md["ll1"],
                                   md["t_offsets"], cg, md["CG_offsets"])


def test_reference_differential_case(dev):
    """CGNet/test.py:115-130 and its __main__: B=2, taus=[2,1], two layers, norm=True, sparse=True (the MST
    list), inputs ``np.random.rand(B, tau, 2l+1, 2) * 10`` from seed 0 through the LIST interface, loss
    ``mse(out.sum(), 0)``; output, the gradient of every input fragment and of every layer's weights."""
    from cgnet_amd import CGNet
    bsz, taus, nlayers, lmax = 2, [2, 1], 2, 1
    torch.manual_seed(0)
    np.random.seed(0)
    net = CGNet.SphericalCNN(lmax, [taus] * (nlayers + 1), norm=True, skipconn=True, sparse_flag=True)
    oracles, twins, ws = [], [], []
    g = torch.Generator().manual_seed(1)
    for layer in net.cgs:
        assert layer.sparse_flag and layer.cg.lll_list == OT.encode_sorted(OT.mst_pairs(lmax, use_scipy=False))[0]
        t_ff = [int(v) for v in layer.t_FF]
        # the reference draws W ~ 0.05 U[0,1) on the CUDA generator (CG_layers.py:119-122): same law, injected values
        w64 = (0.05 * torch.rand(sum(a * b for a, b in zip(t_ff, taus)), 2, generator=g, dtype=torch.float64)).float().double()
        stds = torch.rand(sum(t_ff), generator=g, dtype=torch.float64).float()          # U[0,1) as CG_layers.py:116-117
        with torch.no_grad():
            layer.bnWMM.W.copy_(w64.float())
            layer.bnWMM.bn_stds.copy_(stds)
        oracles.append(make_oracle(lmax, taus, taus, layer.cg.lll_list, True, stds))
        twins.append(make_oracle(lmax, taus, taus, layer.cg.lll_list, True, stds, dtype=F32))
        ws.append(w64)
    np.random.seed(0)                                     # gen_fs(taus, B, seed=0)
    npv = [np.random.rand(bsz, taus[l], 2 * l + 1, 2) * 10 for l in range(lmax + 1)]

    def run_oracle(stack, dtype):
        fs = [torch.tensor(v, dtype=torch.float32).to(dtype).requires_grad_(True) for v in npv]
        wo = [w.to(dtype).clone().requires_grad_(True) for w in ws]
        out = OL.stack_forward(stack, wo, fs, taus, skipconn=True)
        loss = torch.nn.functional.mse_loss(out.sum(), torch.zeros((), dtype=dtype))
        return out.detach(), torch.autograd.grad(loss, fs + wo)
    want, want_g = run_oracle(oracles, F64)
    tw, tw_g = run_oracle(twins, F32)

    f0 = [torch.tensor(v, dtype=torch.float, device=dev, requires_grad=True) for v in npv]
    out = net(f0)
    assert out.shape == (bsz, 2 * 2 * (nlayers + 1))
    loss = torch.nn.functional.mse_loss(out.sum(), torch.zeros((), device=dev))
    loss.backward()
    assert_close(out, want, "reference case: out", tw)
    for l in range(lmax + 1):
        assert_close(f0[l].grad, want_g[l], "reference case: grad_F[%d]" % l, tw_g[l])
    for i, layer in enumerate(net.cgs):
        assert_close(layer.bnWMM.W.grad, want_g[lmax + 1 + i], "reference case: grad_W[%d]" % i, tw_g[lmax + 1 + i])
        assert layer.bnWMM.bn_cnt == 2.0


def test_plans_created_in_descending_lds_order(dev):
    """The dynamic-LDS limit of a kernel belongs to the process, not to the plan created last: a plan whose
    kernels need more LDS than a later plan's (here the forward's: its work-groups hold whole 16 x 16 x (2l+1)
    tiles, beyond the 64 KB a kernel gets by default) must still launch after that later plan was created."""
    from cgnet_amd import CG_layers
    shapes = [(20, [16] * 21), (15, [16] * 16), (13, [14] * 14), (11, [12] * 12)]
    mods = [CG_layers.CG_woFilter_cuda(lmax, taus, device=dev) for lmax, taus in shapes]
    need = [m.native_plan().forward_lds for m in mods]
    assert need[0] > 64 * 1024 and need[0] == max(need), need     # the first plan asks for the most, beyond the default limit
    assert need[-1] < 64 * 1024 and len(set(need)) > 1, need
    assert len(set(m.native_plan().backward_lds for m in mods)) > 1
    for k in (0, 1, 2, 3, 0):
        lmax, taus = shapes[k]
        x = rand_straight(taus, 1, seed=4).float().to(dev).requires_grad_(True)
        y = mods[k](x)
        y.backward(torch.ones_like(y))
        torch.cuda.synchronize()
        assert torch.isfinite(x.grad).all() and float(x.grad.abs().max()) > 0
