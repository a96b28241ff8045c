#!/usr/bin/env python3
"""Headline benchmark: one Clebsch-Gordan layer (CG product -> fragment norm -> weight mixing),
forward + backward, at L=11, tau=12, B=100 (BASELINE.json configs[2]) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline]

Prints ONE JSON line.  A "step" is one training-mode forward (statistics update included) plus
one backward (input gradient and weight gradient) of the layer over one batch of synthetic
fragments that already reside in HBM.  `roofline` describes the kernel that takes the most
time inside the timed region (durations from HIP events the library records on the launch
stream; the timed steps bracket only that kernel, an untimed survey before them brackets every
kernel for the `kernels` table); `whole_step` prices the complete step against the five
compulsory passes over the materialised product tensor (the default backward skips two of them: it never
writes grad_FF; `--two-kernel-backward` runs all five).  `cpu_baseline` times the CPU oracle (a port of the reference's
python path) on a bounded sample of the same workload on the host cores.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published peak

WORKLOAD = {"lmax": 11, "tau": 12, "batch": 100}


def synthetic(lmax, tau, bsz, t_ff, seed=0):
    import torch
    g = torch.Generator().manual_seed(seed)
    x = torch.cat([torch.randn(bsz, tau * (2 * l + 1), 2, generator=g) / math.sqrt(2 * l + 1)
                   for l in range(lmax + 1)], dim=1)
    w = torch.cat([torch.randn(t_ff[l] * tau, 2, generator=g) / math.sqrt(t_ff[l]) for l in range(lmax + 1)])
    go = torch.randn(bsz, tau * (lmax + 1) ** 2, 2, generator=g)
    return x, w, go


TRAFFIC_PROFILE = os.path.join("profiles", "cg_layer_L11_tau12_B100_hbm_traffic_pmc.txt")


def profiled_traffic():
    """HBM bytes per launch of the streaming kernels as the committed rocprofv3 FETCH_SIZE / WRITE_SIZE
    summary states them (counters are not readable from inside a run; the summary names the command and
    the source revision it was measured on).  -> ({kernel: bytes}, description of the source)."""
    import re
    path = os.path.join(ROOT, TRAFFIC_PROFILE)
    table, rev = {}, "unknown revision"
    try:
        for line in open(path):
            m = re.match(r"^(\w+)(?:<\d+>)?\s+([\d.]+) MB\s+([\d.]+) MB\s+([\d.]+) MB\s+([\d.]+) MB\s+[\d.]+\s*$", line)
            if m:
                table[m.group(1)] = float(m.group(4)) * 1e6
            m = re.match(r"^source revision:\s*(\S+)", line)
            if m:
                rev = m.group(1)
    except OSError:
        return {}, "no traffic profile found"
    return table, "%s (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; measured at %s, not in this run)" % (TRAFFIC_PROFILE, rev)


SQ_PROFILE = os.path.join("profiles", "cg_layer_L11_tau12_B100_sq_counters_pmc.txt")


def profiled_issue(kernel, avg_launch_ms):
    """SIMD issue time of `kernel` from the committed SQ counter summary: vector and matrix instructions take turns
    on a SIMD of this GPU (2.7 cycles per vector instruction, 32 per v_mfma_f32_16x16x4_f32; measured, see the
    summary's header), so (2.7 N_vector + 32 N_matrix) / (1024 SIMDs x clock) bounds the kernel from below."""
    try:
        for line in open(os.path.join(ROOT, SQ_PROFILE)):
            f = line.split()
            if len(f) >= 7 and f[0].split("<")[0] == kernel:
                mhz, n_valu, n_mfma = float(f[2]), float(f[3]), float(f[6])
                bound_ms = (2.7 * (n_valu - n_mfma) + 32.0 * n_mfma) / (1024 * mhz * 1e6) * 1e3
                return {"bound_ms": round(bound_ms, 4), "frac": round(bound_ms / avg_launch_ms, 3), "clock_MHz": mhz,
                        "vector_instructions": n_valu - n_mfma, "matrix_instructions": n_mfma,
                        "source": SQ_PROFILE + " (counters of an earlier run, not of this one)"}
    except (OSError, ValueError):
        pass
    return None


def host_cpu():
    """(model name, physical cores, logical cpus) of the host, from /proc/cpuinfo."""
    model, cores, logical = "unknown", set(), 0
    try:
        phys = core = None
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "model name":
                model = val
            elif key == "processor":
                logical += 1
            elif key == "physical id":
                phys = val
            elif key == "core id":
                core = val
            elif not key and phys is not None:
                cores.add((phys, core))
                phys = core = None
        if phys is not None:
            cores.add((phys, core))
    except OSError:
        pass
    return model, (len(cores) or logical), logical


def cpu_baseline(lmax, tau, codes, t_ff, sample_batch, repeats):
    """The oracle's float32 layer (port of the reference's python path) on the host cores."""
    import numpy as np
    import torch
    from oracle import cg_layer as OL
    taus = [tau] * (lmax + 1)
    x, w, go = synthetic(lmax, tau, sample_batch, t_ff, seed=1)
    layer = OL.LayerOracle(lmax, taus, taus, codes, batchnorm=True)
    layer.set_stds_flat(np.ones(sum(t_ff), dtype=np.float32))

    def step():
        xx = x.clone().requires_grad_(True)
        ww = w.clone().requires_grad_(True)
        out = OL.join_straight(layer.forward(xx, ww))
        out.backward(go)
        return xx.grad, ww.grad
    step()                                            # warm-up (also builds the CG matrices)
    t0 = time.perf_counter()
    for _ in range(repeats):
        step()
    dt = (time.perf_counter() - t0) / repeats
    model, physical, logical = host_cpu()
    return {"value": sample_batch / dt, "unit": "samples/s", "cores": int(torch.get_num_threads()),
            "kind": "port", "cpu_model": model, "physical_cores": physical, "logical_cpus": logical,
            "threads_used": int(torch.get_num_threads()), "cpu_batch": sample_batch, "gpu_batch": WORKLOAD["batch"],
            "sample": "B=%d (the GPU line runs B=%d) of the same L=%d tau=%d layer fwd+bwd, float32 torch CPU oracle, "
                      "1 warm-up + %d timed steps, %.1f s per step; the per-sample cost of the oracle does not depend "
                      "on B" % (sample_batch, WORKLOAD["batch"], lmax, tau, repeats, dt)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--two-kernel-backward", action="store_true",
                    help="materialise grad_FF and run the mixing backward and the product backward as two kernels "
                         "(default: the one-kernel layer backward, which forms grad_FF tile by tile in LDS)")
    ap.add_argument("--cpu-batch", type=int, default=16)
    ap.add_argument("--cpu-repeats", type=int, default=8)
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 768 MiB read + 768 MiB write elementwise kernel before the warm-up "
                         "(a known-size reference for calibrating hardware byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build runs the CG layer on ONE GPU (no collectives, no sharding); "
                         "--gpus %d is not supported.\n" % args.gpus)
        sys.exit(2)

    import torch
    from cgnet_amd import CG_layers, _lib
    lib = _lib.load()
    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        sys.exit(1)
    dev = torch.device("cuda:0")
    lmax, tau, bsz = WORKLOAD["lmax"], WORKLOAD["tau"], WORKLOAD["batch"]
    taus = [tau] * (lmax + 1)
    layer = CG_layers.CGBN_cuda(lmax, taus, taus, batchnorm=True, sparse_flag=False, device=dev)
    layer.fused_backward = not args.two_kernel_backward
    t_ff = [int(v) for v in layer.t_FF]
    x, w, go = synthetic(lmax, tau, bsz, t_ff)
    with torch.no_grad():
        layer.bnWMM.W.copy_(w)
        layer.bnWMM.bn_stds.fill_(1.0)
    x = x.to(dev).requires_grad_(True)
    go = go.to(dev)
    layer.train()

    def step():
        x.grad = None
        layer.bnWMM.W.grad = None
        out = layer(x, straight_output=True)
        out.backward(go)

    if args.copy_probe:
        src = torch.ones(192 * 1024 * 1024, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # untimed: keep the GPU busy for a moment so that the timed steps run at the settled clock, whatever W was
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < 0.4:
        for _ in range(10):
            step()
        torch.cuda.synchronize()
    # untimed survey with every kernel bracketed by events: per-kernel table, and which kernel dominates
    lib.cgnet_profile_reset()
    lib.cgnet_profile_select(None)
    lib.cgnet_profile_enable(1)
    survey_steps = max(3, min(10, args.steps))
    for _ in range(survey_steps):
        step()
    torch.cuda.synchronize()
    lib.cgnet_profile_enable(0)
    survey = _lib.kernel_times()
    # timed region: only the dominant kernel is bracketed (each event pair costs a few microseconds)
    lib.cgnet_profile_reset()
    candidates = ("cg_forward_kernel", "cg_forward_mm_kernel", "wmm_forward_kernel", "wmm_gradw_kernel",
                  "wmm_gradff_mfma_kernel", "wmm_gradff_kernel", "cg_backward_unit_kernel", "cg_backward_hybrid_kernel",
                  "cg_backward_kernel", "cgbn_backward_fused_kernel")
    dominant = max((n for n in survey if n in candidates), key=lambda n: survey[n][0])
    lib.cgnet_profile_select(dominant.encode())
    lib.cgnet_profile_enable(1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    lib.cgnet_profile_enable(0)
    lib.cgnet_profile_select(None)
    times = _lib.kernel_times()
    assert torch.isfinite(x.grad).all() and torch.isfinite(layer.bnWMM.W.grad).all()

    n_f = tau * (lmax + 1) ** 2
    n_o = n_f
    n_ff = int(layer.cg.cumu_tm_FF[-1])
    n_w = int(layer.bnWMM.W.shape[0])
    sum_t = sum(t_ff)
    cg_len = int(layer.cg.CGspace.numel())
    # algorithmic bytes per launch of the five kernels that stream the product tensor
    algo = {
        "cg_forward_kernel": 8 * bsz * (n_f + n_ff),
        "cg_forward_mm_kernel": 8 * bsz * (n_f + n_ff),
        "wmm_forward_kernel": 8 * (bsz * n_ff + n_w + bsz * n_o) + 4 * sum_t,
        "wmm_gradw_kernel": 8 * (bsz * n_ff + bsz * n_o + n_w),
        "wmm_gradff_mfma_kernel": 8 * (bsz * n_o + n_w + bsz * n_ff),
        "wmm_gradff_kernel": 8 * (bsz * n_o + n_w + bsz * n_ff),
        "cg_backward_unit_kernel": 8 * (bsz * n_ff + 2 * bsz * n_f),
        "cg_backward_hybrid_kernel": 8 * (bsz * n_ff + 2 * bsz * n_f),
        "cg_backward_kernel": 8 * (bsz * n_ff + 2 * bsz * n_f),
    }
    # the one-kernel layer backward stands for two of the five passes (grad FF written, grad FF read); it is priced
    # against the bytes those passes would move although it moves neither (what it really moves: `traffic`)
    algo["cgbn_backward_fused_kernel"] = algo["wmm_gradff_mfma_kernel"] + algo["cg_backward_hybrid_kernel"]
    measured_traffic, traffic_source = profiled_traffic()
    step_bytes = 8 * (5 * bsz * n_ff + bsz * (3 * n_f + 3 * n_o) + 3 * n_w) + 4 * (2 * sum_t + cg_len)
    kernels = {}
    for name, (ms, cnt) in sorted(survey.items(), key=lambda kv: -kv[1][0]):
        avg = ms / max(cnt, 1)
        ent = {"avg_ms": round(avg, 4), "launches_per_step": cnt / survey_steps}
        if name in algo and avg > 0:
            ent["algorithmic_GBps"] = round(algo[name] / (avg * 1e-3) / 1e9, 1)
        kernels[name] = ent
    d_avg_s = times[dominant][0] / times[dominant][1] * 1e-3     # from the events of the timed region
    achieved = algo[dominant] / d_avg_s / 1e9
    ms_per_step = dt / args.steps * 1e3

    line = {
        "metric": "CG-layer fwd+bwd samples/sec at L=11,tau=12,B=100; % HBM roofline",
        "value": bsz * args.steps / dt,
        "unit": "samples/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "configs[2]: one CGNet layer fwd+bwd, Lmax=11, tau=12, B=100, fp32 complex, "
                               "CG product + fragment norm + weight mixing, default (l2<=l1) triples",
                   "lmax": lmax, "tau": tau, "batch": bsz, "triples": len(layer.cg.lll_list)},
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic.get(dominant),
                     "traffic_source": traffic_source,
                     "algorithmic_bytes_per_launch": algo[dominant], "avg_launch_ms": d_avg_s * 1e3,
                     "simd_issue": profiled_issue(dominant, d_avg_s * 1e3)},
        "whole_step": {"algorithmic_bytes": step_bytes, "achieved_GBps": step_bytes / (ms_per_step * 1e-3) / 1e9,
                       "frac_of_hbm_peak": step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "fused_backward": bool(layer.fused_backward and layer.native_layer_plan().fused_backward_supported),
        "kernels": kernels,
        "kernels_note": "per-kernel table from %d untimed steps with every launch bracketed by events; "
                        "in the timed steps only the dominant kernel is bracketed" % survey_steps,
    }
    if not args.no_cpu_baseline:
        del x, go
        torch.cuda.empty_cache()
        line["cpu_baseline"] = cpu_baseline(lmax, tau, layer.cg.lll_list, t_ff, args.cpu_batch, args.cpu_repeats)
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
