// Clebsch-Gordan product of a set of fragments with itself, forward and backward, for gfx950.
//
// Work decomposition.  A "task" is one kept triple (l, l1, l2) restricted to a range of t1
// rows, so that its output tile  FF[b, l, t_off + t1*tau2 + t2, m]  (t1 in the range, all t2,
// all m) is one contiguous run of a sample's FF and fits in LDS.
//
// Forward: one work-group per (task, group of samples).  The CG table of the triple is staged
// in LDS once, then per sample the two input slabs are staged, every thread accumulates a
// TI x TJ register tile of channels for one m (the m = m1 + m2 rule leaves at most 2*l2+1
// terms), the tile is written to LDS in output order and streamed out with contiguous stores.
// Optionally the per-channel sums of |z| and |z|^2 are taken from the staged tile.
//
// Backward: one work-group per (sample, group of tasks).  The gradient of the whole sample's
// fragments is accumulated in LDS while the group's gFF tiles stream through LDS once; each
// output element is owned by one 2^k-lane row of threads that splits the channel reduction
// and combines with a fixed DPP tree, so the result does not depend on scheduling.  Groups
// write partial gradients that a second kernel adds in a fixed order.
#include <algorithm>
#include <memory>
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
    int device = 0;
};

namespace cgnet {
namespace {

constexpr int kThreads = 256;
constexpr int kFwdTileBytes = 32 * 1024;
constexpr int kBwdTileBytes = 16 * 1024;
constexpr int kMaxTileChannels = 4 * kThreads;   // statistics: at most four channels per thread
constexpr int kMaxBwdGroups = 32;
constexpr size_t kMaxLds = 160 * 1024;

__host__ __device__ inline size_t fwd_task_lds(const CgTask& t) {
    const size_t M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
    return 8 * ((size_t)t.rows * t.tau2 * M + (size_t)t.rows * M1 + (size_t)t.tau2 * M2) + 4 * M * M2;
}

// ------------------------------------------------------------------------------------ forward
template <int TI, int TJ>
__device__ __forceinline__ void fwd_tiles(const CgTask& t, const float* __restrict__ cg,
                                          const float2* __restrict__ f1, const float2* __restrict__ f2,
                                          float2* __restrict__ out) {
    const int l = t.l, l1 = t.l1, l2 = t.l2;
    const int M = 2 * l + 1, M1 = 2 * l1 + 1, M2 = 2 * l2 + 1;
    const int nT1 = t.nT1, nT2 = t.nT2, rows = t.rows, tau2 = t.tau2;
    const int nitems = nT1 * nT2 * M;
    for (int item = threadIdx.x; item < nitems; item += kThreads) {
        const int mm = item % M;
        const int tt = item / M;
        const int tj = tt % nT2, ti = tt / nT2;
        const int m = mm - l;
        const int lo = max(-l2, m - l1), hi = min(l2, m + l1);
        float ar[TI][TJ], ai[TI][TJ];
        int r1[TI], r2[TJ];
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            r1[i] = min(ti + nT1 * i, rows - 1) * M1 + (m + l1);
#pragma unroll
            for (int j = 0; j < TJ; ++j) ar[i][j] = ai[i][j] = 0.f;
        }
#pragma unroll
        for (int j = 0; j < TJ; ++j) r2[j] = min(tj + nT2 * j, tau2 - 1) * M2 + l2;
        const float* cgrow = cg + mm * M2 + l2;
        for (int m2 = lo; m2 <= hi; ++m2) {
            const float c = cgrow[m2];
            float2 b[TJ];
#pragma unroll
            for (int j = 0; j < TJ; ++j) b[j] = f2[r2[j] + m2];
#pragma unroll
            for (int i = 0; i < TI; ++i) {
                float2 a = f1[r1[i] - m2];
                a.x *= c;
                a.y *= c;
#pragma unroll
                for (int j = 0; j < TJ; ++j) {
                    ar[i][j] = fmaf(a.x, b[j].x, ar[i][j]);
                    ar[i][j] = fmaf(-a.y, b[j].y, ar[i][j]);
                    ai[i][j] = fmaf(a.x, b[j].y, ai[i][j]);
                    ai[i][j] = fmaf(a.y, b[j].x, ai[i][j]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            const int t1 = ti + nT1 * i;
#pragma unroll
            for (int j = 0; j < TJ; ++j) {
                const int t2 = tj + nT2 * j;
                if (t1 < rows && t2 < tau2) out[(t1 * tau2 + t2) * M + mm] = make_float2(ar[i][j], ai[i][j]);
            }
        }
    }
}

template <int TI>
__device__ __forceinline__ void fwd_dispatch_j(const CgTask& t, const float* cg, const float2* f1,
                                               const float2* f2, float2* out) {
    switch (t.TJ) {
        case 1: fwd_tiles<TI, 1>(t, cg, f1, f2, out); break;
        case 2: fwd_tiles<TI, 2>(t, cg, f1, f2, out); break;
        case 3: fwd_tiles<TI, 3>(t, cg, f1, f2, out); break;
        default: fwd_tiles<TI, 4>(t, cg, f1, f2, out); break;
    }
}

__global__ void __launch_bounds__(kThreads)
cg_forward_kernel(const float2* __restrict__ F, float2* __restrict__ FF, const float* __restrict__ CG,
                  const CgTask* __restrict__ tasks, int nF, int nFF, int B, int samples_per_group,
                  double* __restrict__ stats_part, int sumT) {
    extern __shared__ __align__(16) unsigned char smem[];
    const CgTask t = tasks[blockIdx.x];
    const int M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
    const int nch = t.rows * t.tau2;
    const int nout = nch * M, n1 = t.rows * M1, n2 = t.tau2 * M2, ncg = M * M2;
    float2* out = reinterpret_cast<float2*>(smem);
    float2* f1 = out + nout;
    float2* f2 = f1 + n1;
    float* cg = reinterpret_cast<float*>(f2 + n2);
    const int tid = threadIdx.x;

    for (int e = tid; e < ncg; e += kThreads) cg[e] = CG[t.cg_off + e];

    double s1[4] = {0., 0., 0., 0.}, s2[4] = {0., 0., 0., 0.};
    const int b0 = blockIdx.y * samples_per_group;
    const int b1 = min(B, b0 + samples_per_group);
    for (int b = b0; b < b1; ++b) {
        const float2* Fb = F + (size_t)b * nF;
        for (int e = tid; e < n1; e += kThreads) f1[e] = Fb[t.offF1 + e];
        for (int e = tid; e < n2; e += kThreads) f2[e] = Fb[t.offF2 + e];
        __syncthreads();
        switch (t.TI) {
            case 1: fwd_dispatch_j<1>(t, cg, f1, f2, out); break;
            case 2: fwd_dispatch_j<2>(t, cg, f1, f2, out); break;
            case 3: fwd_dispatch_j<3>(t, cg, f1, f2, out); break;
            default: fwd_dispatch_j<4>(t, cg, f1, f2, out); break;
        }
        __syncthreads();
        float2* dst = FF + (size_t)b * nFF + t.offFF;
        for (int e = tid; e < nout; e += kThreads) dst[e] = out[e];
        if (stats_part) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int ch = tid + kThreads * k;
                if (ch < nch) {
                    float a = 0.f, q = 0.f;
                    for (int mm = 0; mm < M; ++mm) {
                        const float2 z = out[ch * M + mm];
                        const float n = fmaf(z.x, z.x, z.y * z.y);
                        q += n;
                        a += sqrtf(n);
                    }
                    s1[k] += (double)a;
                    s2[k] += (double)q;
                }
            }
        }
        __syncthreads();
    }
    if (stats_part) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int ch = tid + kThreads * k;
            if (ch < nch) {
                double* p = stats_part + ((size_t)blockIdx.y * sumT + t.chan0 + ch) * 2;
                p[0] = s1[k];
                p[1] = s2[k];
            }
        }
    }
}

__global__ void __launch_bounds__(256)
stats_reduce_kernel(const double* __restrict__ part, double* __restrict__ sums, int n2, int ngroups) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n2) return;
    double s = 0.;
    for (int g = 0; g < ngroups; ++g) s += part[(size_t)g * n2 + i];
    sums[i] = s;
}

// ----------------------------------------------------------------------------------- backward
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xF, 0xF, true));
}

// Sum over aligned groups of RW consecutive lanes; every lane of the group receives the sum.
// Must be executed by all lanes of the wave.
template <int RW>
__device__ __forceinline__ float row_sum(float v) {
    if (RW >= 2) v += dpp_move<0xB1>(v);    // quad_perm [1,0,3,2]
    if (RW >= 4) v += dpp_move<0x4E>(v);    // quad_perm [2,3,0,1]
    if (RW >= 8) v += dpp_move<0x141>(v);   // row_half_mirror
    if (RW >= 16) v += dpp_move<0x140>(v);  // row_mirror
    return v;
}

constexpr int kBT = 4;   // output rows per thread in the backward phases

// Gradient with respect to the slot that is NOT reduced over.
//   SLOT == 1: outputs (t1 in the task's rows, m1), reduced over (t2, m2)
//   SLOT == 2: outputs (t2, m2),                    reduced over (t1 in rows, m1)
// g is the staged gFF tile [rows][tau2][M]; fr the staged fragments of the reduced slot;
// acc the sample-wide gradient accumulator; out_base the complex offset of the output slab.
template <int SLOT, int RW>
__device__ __forceinline__ void bwd_phase(const CgTask& t, const float* __restrict__ cg,
                                          const float2* __restrict__ g, const float2* __restrict__ fr,
                                          float2* __restrict__ acc) {
    const int l = t.l, l1 = t.l1, l2 = t.l2;
    const int M = 2 * l + 1, M1 = 2 * l1 + 1, M2 = 2 * l2 + 1;
    const int rows = t.rows, tau2 = t.tau2;
    // geometry of the output slot (o) and the reduced slot (r)
    const int n_o = (SLOT == 1) ? rows : tau2;        // output channels
    const int n_r = (SLOT == 1) ? tau2 : rows;        // reduced channels
    const int l_o = (SLOT == 1) ? l1 : l2, l_r = (SLOT == 1) ? l2 : l1;
    const int M_o = (SLOT == 1) ? M1 : M2, M_r = (SLOT == 1) ? M2 : M1;
    const int g_so = (SLOT == 1) ? tau2 * M : M;      // stride in g between output channels
    const int g_sr = (SLOT == 1) ? M : tau2 * M;      // stride in g between reduced channels
    const int out_base = (SLOT == 1) ? t.offF1 : t.offF2;

    constexpr int nrows_blk = kThreads / RW;
    const int row_id = threadIdx.x / RW, lane_r = threadIdx.x % RW;
    const int nT = (n_o + kBT - 1) / kBT;
    const int nitems = nT * M_o;
    const int npass = (nitems + nrows_blk - 1) / nrows_blk;
    for (int pass = 0; pass < npass; ++pass) {
        const int item = pass * nrows_blk + row_id;
        const bool valid = item < nitems;
        float ax[kBT], ay[kBT];
#pragma unroll
        for (int i = 0; i < kBT; ++i) ax[i] = ay[i] = 0.f;
        int mmo = 0, to = 0;
        if (valid) {
            mmo = item % M_o;
            to = item / M_o;
            const int mo = mmo - l_o;
            const int lo = max(-l_r, -l - mo), hi = min(l_r, l - mo);
            int go[kBT];
#pragma unroll
            for (int i = 0; i < kBT; ++i) go[i] = min(to + nT * i, n_o - 1) * g_so;
            for (int r = lane_r; r < n_r; r += RW) {
                const float2* frow = fr + r * M_r + l_r;
                const float2* grow = g + r * g_sr + (mo + l);
                for (int mr = lo; mr <= hi; ++mr) {
                    // table entry [m + l][m2 + l2] with m = mo + mr
                    const float c = (SLOT == 1) ? cg[(mo + mr + l) * M2 + (mr + l2)]
                                                : cg[(mo + mr + l) * M2 + mmo];
                    const float2 f = frow[mr];
                    const float cx = c * f.x, cy = -c * f.y;   // c * conj(f)
#pragma unroll
                    for (int i = 0; i < kBT; ++i) {
                        const float2 gv = grow[go[i] + mr];
                        ax[i] = fmaf(gv.x, cx, ax[i]);
                        ax[i] = fmaf(-gv.y, cy, ax[i]);
                        ay[i] = fmaf(gv.x, cy, ay[i]);
                        ay[i] = fmaf(gv.y, cx, ay[i]);
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kBT; ++i) {
            ax[i] = row_sum<RW>(ax[i]);
            ay[i] = row_sum<RW>(ay[i]);
        }
        if (valid && lane_r == 0) {
#pragma unroll
            for (int i = 0; i < kBT; ++i) {
                const int ch = to + nT * i;
                if (ch < n_o) {
                    float2* p = acc + out_base + ch * M_o + mmo;
                    float2 v = *p;
                    v.x += ax[i];
                    v.y += ay[i];
                    *p = v;
                }
            }
        }
    }
}

template <int SLOT>
__device__ __forceinline__ void bwd_phase_dispatch(int n_reduce, const CgTask& t, const float* cg,
                                                   const float2* g, const float2* fr, float2* acc) {
    if (n_reduce <= 1) bwd_phase<SLOT, 1>(t, cg, g, fr, acc);
    else if (n_reduce <= 2) bwd_phase<SLOT, 2>(t, cg, g, fr, acc);
    else if (n_reduce <= 4) bwd_phase<SLOT, 4>(t, cg, g, fr, acc);
    else if (n_reduce <= 8) bwd_phase<SLOT, 8>(t, cg, g, fr, acc);
    else bwd_phase<SLOT, 16>(t, cg, g, fr, acc);
}

__global__ void __launch_bounds__(kThreads)
cg_backward_kernel(const float2* __restrict__ F, const float2* __restrict__ gFF,
                   const float* __restrict__ CG, float2* __restrict__ dst,
                   const CgTask* __restrict__ tasks, const int* __restrict__ group_begin,
                   int nF, int nFF, int B, int tile_floats2) {
    extern __shared__ __align__(16) unsigned char smem[];
    float2* acc = reinterpret_cast<float2*>(smem);
    float2* g = acc + nF;
    const int tid = threadIdx.x;
    const int b = blockIdx.y, grp = blockIdx.x;
    for (int e = tid; e < nF; e += kThreads) acc[e] = make_float2(0.f, 0.f);
    const float2* Fb = F + (size_t)b * nF;
    const float2* Gb = gFF + (size_t)b * nFF;
    const int tbeg = group_begin[grp], tend = group_begin[grp + 1];
    for (int ti = tbeg; ti < tend; ++ti) {
        const CgTask t = tasks[ti];
        const int M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
        const int nout = t.rows * t.tau2 * M, n1 = t.rows * M1, n2 = t.tau2 * M2, ncg = M * M2;
        float2* f1 = g + nout;
        float2* f2 = f1 + n1;
        float* cg = reinterpret_cast<float*>(f2 + n2);
        __syncthreads();   // previous task (and the zeroing) done before the staging area is reused
        for (int e = tid; e < nout; e += kThreads) g[e] = Gb[t.offFF + e];
        for (int e = tid; e < n1; e += kThreads) f1[e] = Fb[t.offF1 + e];
        for (int e = tid; e < n2; e += kThreads) f2[e] = Fb[t.offF2 + e];
        for (int e = tid; e < ncg; e += kThreads) cg[e] = CG[t.cg_off + e];
        __syncthreads();
        bwd_phase_dispatch<1>(t.tau2, t, cg, g, f2, acc);
        __syncthreads();   // a diagonal triple writes the same slab in both phases
        bwd_phase_dispatch<2>(t.rows, t, cg, g, f1, acc);
    }
    __syncthreads();
    float2* out = dst + ((size_t)grp * B + b) * nF;
    for (int e = tid; e < nF; e += kThreads) out[e] = acc[e];
    (void)tile_floats2;
}

__global__ void __launch_bounds__(256)
partial_sum_kernel(const float2* __restrict__ part, float2* __restrict__ out, size_t n, int ngroups) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float2 s = part[i];
    for (int gidx = 1; gidx < ngroups; ++gidx) {
        const float2 v = part[(size_t)gidx * n + i];
        s.x += v.x;
        s.y += v.y;
    }
    out[i] = s;
}

// ------------------------------------------------------------------------------------- host
int samples_per_group_for(int B, int ntasks) {
    // enough work-groups to fill 256 CUs a few times over, while each group amortises the
    // staging of its CG table over several samples
    int groups = std::max(1, std::min(B, (4096 + ntasks - 1) / std::max(1, ntasks)));
    return (B + groups - 1) / groups;
}

int bwd_groups_for(const cgnet_cg_plan* p, int B) {
    const int maxg = (int)p->bwd_group_begin.size() - 1;
    if (maxg <= 0) return 0;
    int want = (1024 + B - 1) / std::max(1, B);
    return std::max(1, std::min(maxg, want));
}

}  // namespace
}  // namespace cgnet

using namespace cgnet;

static void free_plan(cgnet_cg_plan* plan) {
    if (!plan) return;
    if (plan->d_fwd_tasks) (void)hipFree(plan->d_fwd_tasks);
    if (plan->d_bwd_tasks) (void)hipFree(plan->d_bwd_tasks);
    if (plan->d_bwd_group_table) (void)hipFree(plan->d_bwd_group_table);
    delete plan;
}

extern "C" int cgnet_cg_plan_create(cgnet_cg_plan** plan, int L, const int* h_t_F, const int* h_llls,
                                    int nllls, const int* h_t_offsets, const int* h_CG_offsets) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    *plan = nullptr;
    CGNET_REQUIRE(L >= 0 && L <= kMaxL, CGNET_ERR_UNSUPPORTED, "lmax=%d outside [0, %d]", L, kMaxL);
    CGNET_REQUIRE(h_t_F, CGNET_ERR_ARG, "t_F is NULL");
    CGNET_REQUIRE(nllls >= 0 && (nllls == 0 || h_llls), CGNET_ERR_ARG, "llls is NULL or nllls negative");
    cgnet_cg_plan* p = new cgnet_cg_plan();
    std::unique_ptr<cgnet_cg_plan, void (*)(cgnet_cg_plan*)> guard(p, free_plan);
    p->L = L;
    p->nllls = nllls;
    const int n1 = L + 1;
    p->t_F.assign(h_t_F, h_t_F + n1);
    p->cumF.assign(n1 + 1, 0);
    for (int l = 0; l < n1; ++l) {
        CGNET_REQUIRE(h_t_F[l] >= 0 && h_t_F[l] <= kMaxTau, CGNET_ERR_UNSUPPORTED,
                      "t_F[%d]=%d outside [0, %d]", l, h_t_F[l], kMaxTau);
        p->cumF[l + 1] = p->cumF[l] + h_t_F[l] * (2 * l + 1);
    }
    p->nF = p->cumF[n1];
    p->t_FF.assign(n1, 0);
    p->t_off.assign(nllls, 0);
    std::vector<int> tl(nllls), tl1(nllls), tl2(nllls), cgo(nllls + 1, 0);
    int prev_l = 0;
    for (int i = 0; i < nllls; ++i) {
        const int c = h_llls[i];
        CGNET_REQUIRE(c >= 0 && c < n1 * n1 * n1, CGNET_ERR_ARG, "llls[%d]=%d is not a triple code for lmax=%d", i, c, L);
        tl[i] = c / (n1 * n1);
        tl1[i] = (c / n1) % n1;
        tl2[i] = c % n1;
        CGNET_REQUIRE(tl1[i] >= tl2[i] && tl1[i] - tl2[i] <= tl[i] && tl[i] <= tl1[i] + tl2[i], CGNET_ERR_ARG,
                      "triple %d = (l=%d, l1=%d, l2=%d) violates l1>=l2 or the triangle rule", i, tl[i], tl1[i], tl2[i]);
        CGNET_REQUIRE(tl[i] >= prev_l, CGNET_ERR_ARG, "llls must be ordered by output degree (entry %d)", i);
        prev_l = tl[i];
        const int width = h_t_F[tl1[i]] * h_t_F[tl2[i]];
        p->t_off[i] = p->t_FF[tl[i]];
        if (h_t_offsets)
            CGNET_REQUIRE(h_t_offsets[i] == p->t_off[i], CGNET_ERR_ARG,
                          "t_offsets[%d]=%d is not the running channel count %d of degree %d", i,
                          h_t_offsets[i], p->t_off[i], tl[i]);
        p->t_FF[tl[i]] += width;
        cgo[i + 1] = cgo[i] + (2 * tl[i] + 1) * (2 * tl2[i] + 1);
        if (h_CG_offsets)
            CGNET_REQUIRE(h_CG_offsets[i] == cgo[i] && h_CG_offsets[i + 1] == cgo[i + 1], CGNET_ERR_ARG,
                          "CG_offsets[%d] is not the running sum of (2l+1)(2l2+1)", i);
    }
    p->cg_len = cgo[nllls];
    p->cumFF.assign(n1 + 1, 0);
    p->cumT.assign(n1 + 1, 0);
    for (int l = 0; l < n1; ++l) {
        const long long next = (long long)p->cumFF[l] + (long long)p->t_FF[l] * (2 * l + 1);
        CGNET_REQUIRE(next < (1LL << 30), CGNET_ERR_UNSUPPORTED, "product has more than 2^30 complex entries per sample");
        p->cumFF[l + 1] = (int)next;
        p->cumT[l + 1] = p->cumT[l] + p->t_FF[l];
    }
    p->nFF = p->cumFF[n1];
    p->sumT = p->cumT[n1];

    auto build = [&](int tile_bytes, std::vector<CgTask>* out) -> int {
        for (int i = 0; i < nllls; ++i) {
            const int l = tl[i], l1 = tl1[i], l2 = tl2[i];
            const int tau1 = h_t_F[l1], tau2 = h_t_F[l2];
            if (tau1 == 0 || tau2 == 0) continue;
            const int M = 2 * l + 1;
            const long long row_bytes = 8LL * tau2 * M;
            int max_rows = (int)std::min<long long>(tau1, std::max<long long>(1, tile_bytes / row_bytes));
            max_rows = std::max(1, std::min(max_rows, kMaxTileChannels / tau2));
            const int nchunks = (tau1 + max_rows - 1) / max_rows;
            const int rows_per = (tau1 + nchunks - 1) / nchunks;
            for (int r0 = 0; r0 < tau1; r0 += rows_per) {
                CgTask t;
                t.l = l; t.l1 = l1; t.l2 = l2; t.tau1 = tau1; t.tau2 = tau2;
                t.t1_begin = r0;
                t.rows = std::min(rows_per, tau1 - r0);
                t.offF1 = p->cumF[l1] + r0 * (2 * l1 + 1);
                t.offF2 = p->cumF[l2];
                t.offFF = p->cumFF[l] + (p->t_off[i] + r0 * tau2) * M;
                t.cg_off = cgo[i];
                t.chan0 = p->cumT[l] + p->t_off[i] + r0 * tau2;
                t.nT1 = (t.rows + 3) / 4;
                t.TI = (t.rows + t.nT1 - 1) / t.nT1;
                t.nT2 = (tau2 + 3) / 4;
                t.TJ = (tau2 + t.nT2 - 1) / t.nT2;
                out->push_back(t);
            }
        }
        return 0;
    };
    build(kFwdTileBytes, &p->fwd_tasks);
    build(kBwdTileBytes, &p->bwd_tasks);
    // heaviest forward tasks first: a short tail when the grid drains
    std::stable_sort(p->fwd_tasks.begin(), p->fwd_tasks.end(), [](const CgTask& a, const CgTask& b) {
        return (long long)a.rows * a.tau2 * (2 * a.l + 1) * (2 * a.l2 + 1) >
               (long long)b.rows * b.tau2 * (2 * b.l + 1) * (2 * b.l2 + 1);
    });
    size_t fl = 0, bl = 0;
    for (const CgTask& t : p->fwd_tasks) fl = std::max(fl, fwd_task_lds(t));
    for (const CgTask& t : p->bwd_tasks) bl = std::max(bl, fwd_task_lds(t));
    p->fwd_lds = align_up(fl, 16);
    p->bwd_lds = align_up(bl, 16) + 8 * (size_t)p->nF;
    CGNET_REQUIRE(p->fwd_lds <= kMaxLds, CGNET_ERR_UNSUPPORTED,
                  "a single output row needs %zu bytes of LDS (limit %zu)", p->fwd_lds, kMaxLds);
    CGNET_REQUIRE(p->bwd_lds <= kMaxLds, CGNET_ERR_UNSUPPORTED,
                  "backward needs %zu bytes of LDS (limit %zu): too many input channels", p->bwd_lds, kMaxLds);

    // backward groups: contiguous task ranges of roughly equal cost, at most kMaxBwdGroups
    {
        const int nt = (int)p->bwd_tasks.size();
        const int ng = std::min(kMaxBwdGroups, nt);
        std::vector<double> cost(nt);
        double total = 0;
        for (int i = 0; i < nt; ++i) {
            const CgTask& t = p->bwd_tasks[i];
            cost[i] = (double)t.rows * t.tau2 * (2 * t.l + 1) * (2.0 * t.l1 + 2.0 * t.l2 + 2.0) + 2000.0;
            total += cost[i];
        }
        p->bwd_group_begin.clear();
        p->bwd_group_begin.push_back(0);
        double run = 0;
        for (int i = 0, gcount = 1; i < nt; ++i) {
            run += cost[i];
            if (gcount < ng && run >= total * gcount / ng && i + 1 < nt) {
                p->bwd_group_begin.push_back(i + 1);
                ++gcount;
            }
        }
        p->bwd_group_begin.push_back(nt);
        if (nt == 0) p->bwd_group_begin.assign(1, 0);
    }
    // boundaries of every coarser grouping (ng = 1 .. finest), concatenated
    std::vector<int> gtab;
    {
        const int ng_max = (int)p->bwd_group_begin.size() - 1;
        p->bwd_group_table_off.assign(ng_max + 1, 0);
        for (int ng = 1; ng <= ng_max; ++ng) {
            p->bwd_group_table_off[ng] = (int)gtab.size();
            for (int g = 0; g <= ng; ++g) gtab.push_back(p->bwd_group_begin[(size_t)g * ng_max / ng]);
        }
    }

    CGNET_HIP(hipGetDevice(&p->device));
    if (!p->fwd_tasks.empty()) {
        CGNET_HIP(hipMalloc((void**)&p->d_fwd_tasks, sizeof(CgTask) * p->fwd_tasks.size()));
        CGNET_HIP(hipMemcpy(p->d_fwd_tasks, p->fwd_tasks.data(), sizeof(CgTask) * p->fwd_tasks.size(), hipMemcpyHostToDevice));
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_tasks, sizeof(CgTask) * p->bwd_tasks.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_tasks, p->bwd_tasks.data(), sizeof(CgTask) * p->bwd_tasks.size(), hipMemcpyHostToDevice));
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_group_table, sizeof(int) * gtab.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_group_table, gtab.data(), sizeof(int) * gtab.size(), hipMemcpyHostToDevice));
    }
    if (p->fwd_lds > 64 * 1024)
        CGNET_HIP(hipFuncSetAttribute((const void*)cg_forward_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)p->fwd_lds));
    if (p->bwd_lds > 64 * 1024)
        CGNET_HIP(hipFuncSetAttribute((const void*)cg_backward_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)p->bwd_lds));
    *plan = guard.release();
    return CGNET_OK;
}

extern "C" int cgnet_cg_plan_destroy(cgnet_cg_plan* plan) {
    clear_error();
    free_plan(plan);
    return CGNET_OK;
}

extern "C" int cgnet_cg_plan_sizes(const cgnet_cg_plan* plan, int sizes[5]) {
    clear_error();
    CGNET_REQUIRE(plan && sizes, CGNET_ERR_ARG, "null pointer argument");
    sizes[0] = plan->nF;
    sizes[1] = plan->nFF;
    sizes[2] = plan->sumT;
    sizes[3] = plan->cg_len;
    sizes[4] = plan->nllls;
    return CGNET_OK;
}

extern "C" int cgnet_cg_plan_channels(const cgnet_cg_plan* plan, int* h_t_FF, int* h_t_offsets) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    if (h_t_FF) std::copy(plan->t_FF.begin(), plan->t_FF.end(), h_t_FF);
    if (h_t_offsets) std::copy(plan->t_off.begin(), plan->t_off.end(), h_t_offsets);
    return CGNET_OK;
}

static int launch_forward(const cgnet_cg_plan* p, const float* d_F, float* d_FF, const float* d_CG, int B,
                          double* d_part, int spg, hipStream_t s) {
    const int ntasks = (int)p->fwd_tasks.size();
    if (ntasks == 0 || B == 0) return CGNET_OK;
    const int ngroups = (B + spg - 1) / spg;
    CGNET_REQUIRE(ngroups <= 65535, CGNET_ERR_UNSUPPORTED, "batch of %d needs %d sample groups (limit 65535)", B, ngroups);
    CGNET_LAUNCH(cg_forward_kernel, dim3(ntasks, ngroups), dim3(kThreads), p->fwd_lds, s,
                       (const float2*)d_F, (float2*)d_FF, d_CG, p->d_fwd_tasks, p->nF, p->nFF, B, spg, d_part, p->sumT);
    CGNET_HIP(hipGetLastError());
    return CGNET_OK;
}

extern "C" int cgnet_sparse_forward(const cgnet_cg_plan* plan, const float* d_F, float* d_FF,
                                    const float* d_CG, int B, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (B == 0 || plan->nFF == 0) return CGNET_OK;
    CGNET_REQUIRE(d_F && d_FF && d_CG, CGNET_ERR_ARG, "null device pointer");
    const int spg = samples_per_group_for(B, (int)plan->fwd_tasks.size());
    return launch_forward(plan, d_F, d_FF, d_CG, B, nullptr, spg, (hipStream_t)stream);
}

extern "C" size_t cgnet_sparse_forward_stats_workspace(const cgnet_cg_plan* plan, int B) {
    if (!plan || B <= 0) return 0;
    const int spg = samples_per_group_for(B, (int)plan->fwd_tasks.size());
    const int ngroups = (B + spg - 1) / spg;
    return align_up(sizeof(double) * 2 * (size_t)plan->sumT * ngroups, 256);
}

extern "C" int cgnet_sparse_forward_stats(const cgnet_cg_plan* plan, const float* d_F, float* d_FF,
                                          const float* d_CG, int B, double* d_sums, void* d_workspace,
                                          size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (plan->sumT == 0) return CGNET_OK;
    CGNET_REQUIRE(d_sums, CGNET_ERR_ARG, "d_sums is NULL");
    hipStream_t s = (hipStream_t)stream;
    if (B == 0 || plan->nFF == 0) {
        CGNET_HIP(hipMemsetAsync(d_sums, 0, sizeof(double) * 2 * plan->sumT, s));
        return CGNET_OK;
    }
    CGNET_REQUIRE(d_F && d_FF && d_CG, CGNET_ERR_ARG, "null device pointer");
    const size_t need = cgnet_sparse_forward_stats_workspace(plan, B);
    CGNET_REQUIRE(d_workspace && workspace_bytes >= need, CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    const int spg = samples_per_group_for(B, (int)plan->fwd_tasks.size());
    const int ngroups = (B + spg - 1) / spg;
    int rc = launch_forward(plan, d_F, d_FF, d_CG, B, (double*)d_workspace, spg, s);
    if (rc != CGNET_OK) return rc;
    const int n2 = 2 * plan->sumT;
    CGNET_LAUNCH(stats_reduce_kernel, dim3((n2 + 255) / 256), dim3(256), 0, s,
                       (const double*)d_workspace, d_sums, n2, ngroups);
    CGNET_HIP(hipGetLastError());
    return CGNET_OK;
}

extern "C" size_t cgnet_sparse_backward_workspace(const cgnet_cg_plan* plan, int B) {
    if (!plan || B <= 0) return 0;
    const int ng = bwd_groups_for(plan, B);
    if (ng <= 1) return 0;
    return align_up(sizeof(float) * 2 * (size_t)plan->nF * B * ng, 256);
}

extern "C" int cgnet_sparse_backward(const cgnet_cg_plan* plan, const float* d_F, float* d_gF,
                                     const float* d_gFF, const float* d_CG, int B, void* d_workspace,
                                     size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (B == 0 || plan->nF == 0) return CGNET_OK;
    CGNET_REQUIRE(d_gF, CGNET_ERR_ARG, "d_gF is NULL");
    CGNET_REQUIRE(B <= 65535, CGNET_ERR_UNSUPPORTED, "B=%d above 65535", B);
    hipStream_t s = (hipStream_t)stream;
    const int ng_max = (int)plan->bwd_group_begin.size() - 1;
    if (ng_max <= 0 || plan->bwd_tasks.empty()) {
        CGNET_HIP(hipMemsetAsync(d_gF, 0, sizeof(float) * 2 * (size_t)plan->nF * B, s));
        return CGNET_OK;
    }
    CGNET_REQUIRE(d_F && d_gFF && d_CG, CGNET_ERR_ARG, "null device pointer");
    const int ng = bwd_groups_for(plan, B);
    const size_t need = cgnet_sparse_backward_workspace(plan, B);
    CGNET_REQUIRE(need == 0 || (d_workspace && workspace_bytes >= need), CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    const int* d_gb = plan->d_bwd_group_table + plan->bwd_group_table_off[ng];
    float2* dst = ng > 1 ? (float2*)d_workspace : (float2*)d_gF;
    CGNET_LAUNCH(cg_backward_kernel, dim3(ng, B), dim3(kThreads), plan->bwd_lds, s,
                       (const float2*)d_F, (const float2*)d_gFF, d_CG, dst, plan->d_bwd_tasks, d_gb,
                       plan->nF, plan->nFF, B, 0);
    CGNET_HIP(hipGetLastError());
    if (ng > 1) {
        const size_t n = (size_t)plan->nF * B;
        CGNET_LAUNCH(partial_sum_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                           (const float2*)d_workspace, (float2*)d_gF, n, ng);
        CGNET_HIP(hipGetLastError());
    }
    return CGNET_OK;
}
