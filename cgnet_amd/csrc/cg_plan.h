// Types of the Clebsch-Gordan product plan shared by the translation units of libcgnet_hip:
// task / unit tables of the forward and backward kernels, the plan object, and the link between a
// product plan and a mixing plan that the one-kernel layer backward needs.
#pragma once
#include <vector>

#include "common.h"

namespace cgnet {

struct CgTask {
    int l, l1, l2;
    int tau1, tau2;
    int t1_begin, rows;   // range of t1 handled by this task
    int offF1;            // complex offset inside a sample's F of row t1_begin of degree l1
    int offF2;            // complex offset inside a sample's F of degree l2
    int offFF;            // complex offset inside a sample's FF of the tile
    int cg_off;           // float offset of the triple's table
    int chan0;            // index over all mid channels (all degrees) of the tile's first channel
    int nT1, nT2, TI, TJ; // forward register tiling: rows = nT1 x TI (strided), tau2 = nT2 x TJ
    int bTI[2], bRW[2];   // backward, per slot: output channels per thread, lanes sharing one output
    int sym;              // matrix-core forward only: 1 = the tile of a diagonal triple (l1 = l2, all rows) is stored in
                          // its compact form, the channels (t1 <= t2, t2) column after column; offFF / chan0 then count compact
                          // channels.  0 in every table of a product plan (the reference's layout).
};

// Backward, register-resident scheme: one work-group per (sample, unit), a unit being the
// triples that share l1 restricted to a range of t1 rows.
struct BwdUnit {
    int l1, rows;
    int offF1;                // complex offset inside a sample's F of the unit's first row
    int offF1p;               // the same inside a sample's padded fragments (rows of 2*l1+2 entries)
    int task_begin, task_end; // range in the unit-ordered task array (sorted by l2, then l)
    int nA;                   // waves that take slot 1; the other waves of the group take slot 2
    int TI, RW;               // slot-1 tiling: output rows per thread, lanes sharing one output
    int RM;                   // of those RW lanes, RM (1 or 2) split the reduced m range, RW / RM the reduced channels
    int p1off;                // slot-1 result: -1 = the unit's rows in the slot-1 area, else offset of its rows in the
                              // slot-2 partial area (a degree whose task list is split over several units)
};

struct BwdUTask {
    int l, l2, tau2;
    int offFF;                // complex offset inside a sample's gFF of the tile
    int offF2;                // complex offset inside a sample's F of degree l2
    int offF2p;               // the same inside a sample's padded fragments
    int cg_off;
    int cgp_off, cgp_len;     // float offset / length (multiple of 4) of the triple's zero-padded table
    int p2off;                // complex offset inside a sample's slot-2 partial area of this (unit, l2) slab
    int first_of_l2, last_of_l2;
    int TI, RW;               // slot-2 tiling for this run of equal l2
};

// Fused layer backward, packing kernels: what packing a task's weights needs to know (one entry per BwdUTask).
struct GenTask {
    int aoff;                 // float offset of the task's block in the packed conj(W)/div operand
    int nks;                  // k-steps of 4 over (output channel, re/im); 0 for a degree without output channels
    int tO;                   // output channels of degree l
    int chan0, nch;           // the tile's channels inside degree l: first, count (rows * tau2)
    int cumW, K, cumT;        // degree l: complex offset of its weights, mid channels, first mid channel among all
    int sym;                  // 0, or +-tau for a diagonal triple with tau x tau channels: channel (t1, t2) is packed as its own
                              // weight plus sign(sym) times that of channel (t2, t1)
};

// Fused layer backward, main kernel: everything a stage needs to know of its task, 12 ints that a wave reads
// with scalar loads one stage ahead.
struct FusedTask {
    int geom;                 // l | l2 << 8 | tau2 << 16 | first_of_l2 << 24 | last_of_l2 << 25
    int offF2p;               // complex offset of degree l2 inside a sample's padded fragments
    int cgp_off, cgp_len;     // the triple's zero-padded table (floats)
    int p2off;                // complex offset of the (unit, l2) slab in a sample's slot-2 partial area
    int aoff;                 // float offset of the task's packed A operand
    int shape;                // nks | tO << 8 | nch << 16
    int boff;                 // float offset inside a sample's packed B operand of degree l
    int chunks;               // 16-byte pieces: A block | B block << 16
    int pad[3];
};

}  // namespace cgnet

struct cgnet_cg_plan {
    int L = 0, nllls = 0;
    int nF = 0, nFF = 0, sumT = 0, cg_len = 0;
    std::vector<int> t_F, t_FF, t_off, cumF, cumFF, cumT;
    std::vector<cgnet::CgTask> fwd_tasks, bwd_tasks;
    std::vector<int> bwd_group_begin;            // task index ranges of the backward groups (max grouping)
    cgnet::CgTask* d_fwd_tasks = nullptr;
    cgnet::CgTask* d_bwd_tasks = nullptr;
    std::vector<int> bwd_group_table_off;        // for ng groups: first entry of its ng+1 boundaries
    int* d_bwd_group_table = nullptr;
    size_t fwd_lds = 0, bwd_lds = 0;
    bool fwd_mm = false;                         // the forward runs cg_forward_mm_kernel (product on the matrix cores)
    bool bwd_general_ok = true;                  // cg_backward_kernel's LDS need fits (else only the unit kernels serve)
    std::vector<int> fwd_class_begin;            // forward tasks by LDS class: class k = tasks [begin[k], begin[k+1])
    std::vector<size_t> fwd_class_lds;           // LDS bytes of a work-group of class k
    int bwd_threads = 256;                       // work-group size of the backward kernel
    // register-resident backward (used when every unit fits; otherwise the LDS-accumulator kernel)
    bool bwd_fast = false;
    bool bwd_hybrid = false;                     // units run cg_backward_hybrid_kernel (slot 2 on the matrix cores)
    int bwd_hyb_groups = 0;                      // ... with this many work-groups per compute unit (4, 3 or 2)
    std::vector<cgnet::BwdUnit> bwd_units;
    std::vector<cgnet::BwdUTask> bwd_utasks;
    cgnet::BwdUnit* d_bwd_units = nullptr;
    cgnet::BwdUTask* d_bwd_utasks = nullptr;
    int* d_bwd_combine = nullptr;                // [L+2] cumF | [L+1] own1 | [L+2] list begin | list of slab offsets
    int* d_bwd_padmeta = nullptr;                // [L+2] cumF | [L+2] cumFp | per triple {cg_off, cgp_off, cgp_len, M, M2, l1}
    int bwd_nFp = 0;                             // complex entries of one sample's padded fragments
    int bwd_cgp_len = 0;                         // floats of all padded tables
    int bwd_f1cap = 0, bwd_f2cap = 0, bwd_cgcap = 0, bwd_tcap = 0;   // LDS bytes of the staged operands
    int bwd_P2 = 0;                              // complex entries of one sample's slot-2 partial area
    size_t bwd_fast_lds = 0;
    int device = 0;
};


namespace cgnet {

// What the fused layer backward needs to know of a (product plan, mixing plan) pair: per-task metadata
// on the device and the sizes of its packed operands.  Built once (build_fused_link) and never
// changed afterwards, so calls that share it need no lock.
struct FusedLink {
    bool ok = false;                     // the fused kernel takes this pair of plans
    GenTask* d_gens = nullptr;
    FusedTask* d_ftasks = nullptr;
    int* d_packmap = nullptr;            // per (task, row tile) of the weight packing: task, row tile
    int* d_bmap = nullptr;               // per block of the gO packing: cumO, M, t_O, column tile | k-step << 8
    int npack = 0, nbmap = 0;
    size_t operand_floats = 0;           // packed A operand, all tasks
    int bop_floats = 0;                  // packed B operand of one sample
    int bcap = 0, acap = 0;              // LDS bytes of the B / A operand buffers
    int nO = 0;                          // complex entries of one sample's layer output
    size_t lds = 0;                      // LDS bytes of a work-group of the fused kernel
};

// Fused inference forward (product tile mixed while it lies in LDS; FF never exists): what the mixing half needs to
// know of a forward task, one entry per cgnet_cg_plan::fwd_tasks entry, in the same order.
struct FwdMixTask {
    int aoff;                 // float offset of the task's packed weights: float2 entry [ks * 64 + lane] = (W_re, W_im) / div of
                              // output channel lane % 16 and the tile's channel 4 ks + lane / 16 (zero past t_O / the tile)
    int nks;                  // k-steps of four channels over the tile; 0 for a degree without output channels
    int tO;                   // output channels of degree l
    int ooff;                 // complex offset of the task's t_O x (2l+1) block inside a sample's partial outputs
    int cumW, K, c0, cumT;    // degree l: complex offset of its weights, mid channels; the tile's first channel inside the degree;
                              // first mid channel of the degree among all
};

struct FwdLaunch {
    int T;                    // column tiles of 16 values of m of the launch's tasks
    int sel0, n;              // its tasks: entries [sel0, sel0 + n) of FwdLink::d_sel
    size_t lds;               // LDS bytes of a work-group
};

struct FwdLink {
    bool ok = false;
    FwdMixTask* d_mix = nullptr;
    int* d_sel = nullptr;                // indices into the forward tasks, launch by launch
    std::vector<FwdLaunch> launches;
    int* d_packmap = nullptr;            // per 64-lane block of the weight packing: task, k-step
    int* d_red = nullptr;                // [L+2] cumO | [L+1] t_O | [L+2] list begin | per degree the ooff of its tasks, in channel order
    int npack = 0;
    size_t a_floats = 0;                 // packed weights, all tasks
    int opart = 0;                       // complex entries of one sample's partial outputs
    int nO = 0, L = 0;
};

}  // namespace cgnet

namespace cgnet {

// Zero rows before / after a triple's table in the padded copy the unit backward stages.  The two m
// outputs of a thread and the two-step unrolled loop touch table rows -1 .. M+1; there the coefficient
// is zero, so whatever finite value the tile holds at the matching position does not count.
constexpr int kTabLo = 1, kTabHi = 2;

// One lane's share of the packed A operand of the fused layer backward, for row tile `rt` of the task `g`:
// k-steps in pairs (nkp = (nks+1)/2 pairs, an odd last one padded with zeros), float2 entry
// [(rt * nkp + kp) * 64 + lane] = (A[c][4(2kp) + kk], A[c][4(2kp+1) + kk]) for c = chan0 + 16 * rt + lane % 16,
// kk = lane / 16, A[c][(to, re/im)] = W[to][c] / max(eps, stds[c]); rows past the tile's last channel and k past
// 2 t_O are zero.
__device__ __forceinline__ void pack_w_gen_lane(const float2* __restrict__ W, const float* __restrict__ stds, float eps,
                                                const GenTask& g, int rt, int lane, float* __restrict__ Ag) {
    const int i = lane & 15, kk = lane >> 4;
    const int cl = 16 * rt + i;
    const bool on = cl < g.nch;
    const int c = g.chan0 + cl;
    const int nkp = (g.nks + 1) >> 1;
    float* dst = Ag + g.aoff + ((size_t)rt * nkp * 64 + lane) * 2;       // float2 entry [(rt * nkp + kp) * 64 + lane]
    const float r = (on && stds) ? fmaxf(eps, stds[g.cumT + c]) : 1.f;
    // the mirror channel (t2, t1) of a diagonal triple's channel (t1, t2)
    const int tau = g.sym < 0 ? -g.sym : g.sym;
    int cm = c;
    if (tau) {
        const int t1 = cl / tau, t2 = cl - t1 * tau;
        cm = g.chan0 + t2 * tau + t1;
    }
    const float rm = (on && stds && tau) ? fmaxf(eps, stds[g.cumT + cm]) : 1.f;
    for (int kp = 0; kp < nkp; ++kp) {
        float pair[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int ks = 2 * kp + h;
            const int k = 4 * ks + kk, to = k >> 1;
            float v = 0.f;
            if (on && ks < g.nks && to < g.tO) {
                const float2 w = W[g.cumW + (size_t)to * g.K + c];
                v = (k & 1) ? w.y : w.x;
                if (stds) v = v / r;
                if (tau) {
                    const float2 wm = W[g.cumW + (size_t)to * g.K + cm];
                    float vm = (k & 1) ? wm.y : wm.x;
                    if (stds) vm = vm / rm;
                    v = g.sym < 0 ? v - vm : v + vm;
                }
            }
            pair[h] = v;
        }
        *reinterpret_cast<float2*>(dst + (size_t)kp * 128) = make_float2(pair[0], pair[1]);
    }
}

// One lane's share of the packed weights of the fused inference forward (layout: FwdMixTask::aoff).
__device__ __forceinline__ void pack_w_mix_lane(const float2* __restrict__ W, const float* __restrict__ stds, float eps,
                                                const FwdMixTask& g, int nch, int ks, int lane, float* __restrict__ Af) {
    const int to = lane & 15, cl = 4 * ks + (lane >> 4);
    float2 v = make_float2(0.f, 0.f);
    if (to < g.tO && cl < nch) {
        const float2 w = W[g.cumW + (size_t)to * g.K + g.c0 + cl];
        v = w;
        if (stds) {
            const float r = fmaxf(eps, stds[g.cumT + g.c0 + cl]);
            v = make_float2(w.x / r, w.y / r);
        }
    }
    *reinterpret_cast<float2*>(Af + g.aoff + ((size_t)ks * 64 + lane) * 2) = v;
}

// Work-group `blk` (256 threads, every thread must call) of the padded fragments: Fp = F with one zero behind
// every row.  meta: [L+2] cumF | [L+2] cumFp | ...
__device__ __forceinline__ void pad_fragments_block(const float2* __restrict__ F, float2* __restrict__ Fp,
                                                    const int* __restrict__ meta, int L, int nF, int nFp, int B,
                                                    int blk, int* s_tab) {
    const int* cumF = meta;                 // L+2
    const int* cumFp = meta + (L + 2);      // L+2
    const size_t idx = (size_t)blk * blockDim.x + threadIdx.x;
    const int b = (int)(idx / nFp), e = (int)(idx % nFp);
    const int lam = lookup_in_group(L + 1, e, [&](int k) { return cumFp[k]; }, s_tab);
    if (idx >= (size_t)B * nFp) return;
    const int rel = e - cumFp[lam], Mq = 2 * lam + 2;
    const int t = rel / Mq, x = rel - t * Mq;
    float2 v = make_float2(0.f, 0.f);
    if (x < Mq - 1) v = F[(size_t)b * nF + cumF[lam] + t * (Mq - 1) + x];
    Fp[idx] = v;
}

// One triple's table between kTabLo / kTabHi zero rows, by one work-group.  m: {cg_off, cgp_off, cgp_len, M, M2, l1}.
// Entries whose m1 = m - m2 is no valid index of degree l1 become zeros whatever the caller's table holds there: the
// matrix-core half of the backward multiplies them with neighbouring fragment entries and relies on the product
// being zero.
constexpr int kPadMetaInts = 6;
__device__ __forceinline__ void pad_table_block(const float* __restrict__ CG, float* __restrict__ CGP,
                                                const int* __restrict__ m) {
    const int cg_off = m[0], cgp_off = m[1], len = m[2], M = m[3], M2 = m[4], l1 = m[5];
    const int l = (M - 1) >> 1, l2 = (M2 - 1) >> 1;
    for (int e = threadIdx.x; e < len; e += blockDim.x) {
        const int x = e - kTabLo * M2;
        float v = 0.f;
        if (x >= 0 && x < M * M2) {
            const int r = x / M2, c = x - r * M2;
            const int m1 = (r - l) - (c - l2);
            if (m1 >= -l1 && m1 <= l1) v = CG[cg_off + x];
        }
        CGP[cgp_off + e] = v;
    }
}

}  // namespace cgnet
