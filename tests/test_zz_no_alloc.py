"""The entry point that allocates nothing (cgnet_sparse_forward_stats_static) against the entry point it is a
variant of (cgnet_sparse_forward_stats, caller workspace): same product, same per-channel sums, bit for bit,
on two calls in a row, the second with a smaller input, so that whatever the first call left in the
library's fixed area must not leak into the second."""
import pytest
import torch

from oracle import triples as OT

pytestmark = pytest.mark.gpu


def _dev():
    if not torch.cuda.is_available():
        pytest.fail("GPU tests need a GPU: torch.cuda.is_available() is False")
    from cgnet_amd import _lib
    _lib.load()
    return torch.device("cuda:0")


def _table(plan, lmax, codes, dev):
    from cgnet_amd import _plans
    from oracle import cg_coeff as OC
    import numpy as np
    _, offs = OC.flat_cg_table(OT.decode(lmax, codes), dtype=np.float32)
    cg = torch.zeros(int(offs[-1]), device=dev)
    _plans.fill_cg_table(cg, lmax, codes, [int(v) for v in offs])
    return cg


def test_static_area_entry_point_matches_workspace_entry_point():
    from cgnet_amd import _lib, _plans
    dev = _dev()
    lib = _lib.load()
    lmax, taus = 6, [9, 8, 12, 10, 16, 8, 11]
    codes = OT.encode_sorted(OT.default_pairs(lmax))[0]
    plan = _plans.CGPlan(lmax, taus, codes)
    cg = _table(plan, lmax, codes, dev)
    g = torch.Generator().manual_seed(41)
    for bsz in (37, 5):                                   # the second call is the smaller one
        x = torch.randn(bsz, plan.nF, 2, generator=g).to(dev)
        want_ff = torch.full((bsz, plan.nFF, 2), float("nan"), device=dev)
        want_sums = torch.full((plan.sum_tFF, 2), float("nan"), device=dev, dtype=torch.float64)
        plan.forward_stats(x, want_ff, cg, bsz, want_sums)
        got_ff = torch.full_like(want_ff, float("nan"))
        got_sums = torch.full_like(want_sums, float("nan"))
        plan.forward_stats_static(x, got_ff, cg, bsz, got_sums)
        torch.cuda.synchronize()
        # the call allocates nothing: the device's free memory is the same before and after a second call on
        # the same buffers (torch's caching allocator is not involved: the binding passes raw pointers only)
        free_before, _ = torch.cuda.mem_get_info(dev)
        plan.forward_stats_static(x, got_ff, cg, bsz, got_sums)
        torch.cuda.synchronize()
        free_after, _ = torch.cuda.mem_get_info(dev)
        assert free_after == free_before, "the entry point changed the device's free memory by %d bytes" % (free_before - free_after)
        assert torch.isfinite(got_ff).all() and torch.isfinite(got_sums).all()
        assert torch.equal(got_ff, want_ff), "product differs at B=%d" % bsz
        assert torch.equal(got_sums, want_sums), "statistics differ at B=%d" % bsz
        # and the sums are what the product says they are
        mod = got_ff.double().pow(2).sum(-1).sqrt()
        chan = []
        o = 0
        for l, t in enumerate(plan.t_FF):
            n = t * (2 * l + 1)
            chan.append(mod[:, o:o + n].reshape(bsz, t, 2 * l + 1))
            o += n
        s1 = torch.cat([c.sum((0, 2)) for c in chan])
        s2 = torch.cat([c.pow(2).sum((0, 2)) for c in chan])
        assert torch.allclose(got_sums[:, 0], s1, rtol=1e-6) and torch.allclose(got_sums[:, 1], s2, rtol=1e-6)
    # a call whose partial sums exceed the fixed area is refused with a clear message, nothing is launched
    limit = int(lib.cgnet_sparse_forward_stats_static_limit())
    big_l, big_t = 11, [40] * 12
    big_codes = OT.encode_sorted(OT.default_pairs(big_l))[0]
    big = _plans.CGPlan(big_l, big_t, big_codes)
    bsz = 16
    assert lib.cgnet_sparse_forward_stats_workspace(big._h, bsz) > limit
    xb = torch.zeros(bsz, big.nF, 2, device=dev)
    ffb = torch.zeros(1, device=dev)                      # never touched: the size check comes first
    rc = lib.cgnet_sparse_forward_stats_static(big._h, xb.data_ptr(), ffb.data_ptr(), cg.data_ptr(), bsz,
                                               torch.zeros(big.sum_tFF, 2, device=dev, dtype=torch.float64).data_ptr(),
                                               None)
    assert rc == _lib.ERR_UNSUPPORTED
    assert b"static area" in lib.cgnet_last_error()
