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
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <mutex>
#include <vector>

#include "internal.h"

namespace cgnet {
namespace {

constexpr int kThreads = 256;
constexpr int kFwdTileBytes = 32 * 1024;
constexpr int kFwdMmTileBytes = 128 * 1024;      // matrix-core forward: 16 x 16 channels x 95 values of m = 190 KB at
                                                 // most, the largest that leaves room for the operands
constexpr int kBwdTileBytes = 14 * 1024;
constexpr int kMaxTileChannels = 4 * kThreads;   // statistics: at most four channels per thread
constexpr int kMaxBwdGroups = 32;
constexpr size_t kMaxLds = 160 * 1024;
constexpr int kBwdPieces = 40;                   // unit backward: a unit holds at most this fraction of a sample's work
constexpr size_t kMaxHybLds = 80 * 1024;        // hybrid unit backward: two groups of eight waves per CU
constexpr size_t kHybLds4 = 39 * 1024;          // ... four groups per CU
constexpr size_t kHybLds3 = 53 * 1024;          // ... three groups per CU
constexpr long long kHybTileBytes = 28 * 1024;
constexpr size_t kMaxUnitLds = 64 * 1024;       // unit backward: LDS-direct copies address the first 64 KB


// ---------------------------------------------------------------------------- LDS addressing
// LDS byte address of a pointer into shared memory, and typed reads through such addresses.
typedef float v2f_t __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(3))) v2f_t* lds_f2_ptr;
typedef const __attribute__((address_space(3))) float* lds_f_ptr;
__device__ __forceinline__ unsigned lds_addr(const void* p) {
    return (unsigned)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
// complex entry k behind LDS byte address a
__device__ __forceinline__ float2 lds_c(unsigned a, int k) {
    const v2f_t v = ((lds_f2_ptr)(uintptr_t)a)[k];
    return make_float2(v.x, v.y);
}
__device__ __forceinline__ lds_f_ptr lds_f(unsigned a) { return (lds_f_ptr)(uintptr_t)a; }
// Keeps a per-lane value in one register: the optimiser may not split it into base + offset again.
__device__ __forceinline__ unsigned opaque(unsigned v) {
    asm volatile("" : "+v"(v));
    return v;
}




__device__ __forceinline__ void lds_barrier() {      // this wave's LDS accesses are complete, then the group's barrier
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ------------------------------------------------------------------------------------ forward
// The hardware square root (one instruction, error within one ulp).  The statistics use the same
// rounded modulus in both of their sums, so its last bit does not matter to the variance.
__device__ __forceinline__ float sqrt_hw(float n) { return __builtin_amdgcn_sqrtf(n); }

// One item = one m of a TI x TJ tile of channels.  Items are ordered m-major, so the lanes of a
// wave work on a few m with similar numbers of terms, for all channel tiles.  What an item needs
// to know does not depend on the sample: it is worked out once per group.
template <int TI, int TJ>
struct FwdItem {
    unsigned pa[TI], pb[TJ];   // LDS byte addresses in fragment buffer 0: slot-1 rows (walked down), slot-2 rows (up)
    unsigned pc, pc_end;       // table entries of the first / last term
    int obase;                 // index in the output tile of (first channel of the tile, m)
    int valid;                 // bit i*TJ+j: channel (i, j) of the tile exists
};

template <int TI, int TJ>
__device__ __forceinline__ void fwd_item_setup(const CgTask& t, int item, const float* cg, const float2* f1,
                                               const float2* f2, FwdItem<TI, TJ>& it) {
    const int l = t.l, l1 = t.l1, l2 = t.l2;
    const int M = 2 * l + 1, M1 = 2 * l1 + 1, M2 = 2 * l2 + 1;
    const int nT1 = t.nT1, nT2 = t.nT2, rows = t.rows, tau2 = t.tau2;
    const int ntiles = nT1 * nT2;
    // m numbered from the middle of the axis outwards: the waves with the many-term middle m are
    // full, the last (partly filled) wave gets the outer m with few terms
    const int mslot = item / ntiles;
    const int tt = item - mslot * ntiles;
    const int mm = (mslot & 1) ? l + ((mslot + 1) >> 1) : l - (mslot >> 1);
    const int tj = tt % nT2, ti = tt / nT2;
    const int m = mm - l;
    const int lo = max(-l2, m - l1), hi = min(l2, m + l1);
    it.valid = 0;
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        it.pa[i] = lds_addr(f1 + min(ti + nT1 * i, rows - 1) * M1 + (m + l1) - lo);
#pragma unroll
        for (int j = 0; j < TJ; ++j)
            if (ti + nT1 * i < rows && tj + nT2 * j < tau2) it.valid |= 1 << (i * TJ + j);
    }
#pragma unroll
    for (int j = 0; j < TJ; ++j) it.pb[j] = lds_addr(f2 + min(tj + nT2 * j, tau2 - 1) * M2 + l2 + lo);
    it.pc = lds_addr(cg + mm * M2 + l2 + lo);
    it.pc_end = it.pc + 4u * (unsigned)(hi - lo);   // hi >= lo: the plan only admits triples that obey the triangle rule
    it.obase = (ti * tau2 + tj) * M + mm;
}

// The item's TI x TJ sums for the sample whose fragments lie `bufofs` bytes behind buffer 0.
template <int TI, int TJ>
__device__ __forceinline__ void fwd_item_run(const CgTask& t, const FwdItem<TI, TJ>& it, unsigned bufofs,
                                             float2* __restrict__ out) {
    float ar[TI][TJ], ai[TI][TJ];
    unsigned pa[TI], pb[TJ];
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        pa[i] = opaque(it.pa[i] + bufofs);
#pragma unroll
        for (int j = 0; j < TJ; ++j) ar[i][j] = ai[i][j] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < TJ; ++j) pb[j] = opaque(it.pb[j] + bufofs);
    unsigned pc = opaque(it.pc);
    const unsigned pc_end = it.pc_end;
    {
        // every m has at least one term (pc <= pc_end on entry)
#pragma unroll 2
        do {
            const float c = lds_f(pc)[0];
            float2 b[TJ];
#pragma unroll
            for (int j = 0; j < TJ; ++j) { b[j] = lds_c(pb[j], 0); pb[j] += 8u; }
#pragma unroll
            for (int i = 0; i < TI; ++i) {
                float2 a = lds_c(pa[i], 0);
                pa[i] -= 8u;
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
            pc += 4u;
        } while (pc <= pc_end);
    }
    const int M = 2 * t.l + 1;
    const int si = t.nT1 * t.tau2 * M, sj = t.nT2 * M;
#pragma unroll
    for (int i = 0; i < TI; ++i)
#pragma unroll
        for (int j = 0; j < TJ; ++j)
            if (it.valid & (1 << (i * TJ + j))) out[it.obase + i * si + j * sj] = make_float2(ar[i][j], ai[i][j]);
}

// LDS of the forward kernel: two fragment buffers (slab of l1 rows, slab of l2) | output tile | table
__host__ __device__ inline size_t fwd_frag_lds(const CgTask& t) {
    const size_t M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
    return ((8 * (size_t)t.rows * M1 + 15) & ~(size_t)15) + ((8 * (size_t)t.tau2 * M2 + 15) & ~(size_t)15);
}

__host__ __device__ inline size_t fwd_task_lds(const CgTask& t) {
    const size_t M = 2 * t.l + 1, M2 = 2 * t.l2 + 1;
    return ((8 * (size_t)t.rows * t.tau2 * M + 15) & ~(size_t)15) + 2 * fwd_frag_lds(t) + 4 * M * M2;
}

template <int TI, int TJ>
__device__ __forceinline__ void fwd_group(const CgTask& t, const float2* __restrict__ F, float2* __restrict__ FF,
                                          const float* __restrict__ CG, int nF, int nFF, int B,
                                          int samples_per_group, int group, double* __restrict__ stats_part, int sumT,
                                          unsigned char* smem) {
    const int M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
    const int nch = t.rows * t.tau2;
    const int nout = nch * M, n1 = t.rows * M1, n2 = t.tau2 * M2, ncg = M * M2;
    const size_t out_bytes = (8 * (size_t)nout + 15) & ~(size_t)15;
    const size_t f1_bytes = (8 * (size_t)n1 + 15) & ~(size_t)15;
    const size_t frag_bytes = fwd_frag_lds(t);
    unsigned char* frag = smem;                                   // [2][frag_bytes], the LDS-direct copy targets
    float2* out = reinterpret_cast<float2*>(smem + 2 * frag_bytes);
    float* cg = reinterpret_cast<float*>(smem + 2 * frag_bytes + out_bytes);
    const int tid = threadIdx.x;
    const float2* f1_0 = reinterpret_cast<const float2*>(frag);
    const float2* f2_0 = reinterpret_cast<const float2*>(frag + f1_bytes);

    // fragments of sample b -> buffer `par`, straight into LDS
    auto issue = [&](int b, int par) {
        const float2* Fb = F + (size_t)b * nF;
        unsigned char* d1 = frag + par * frag_bytes;
        unsigned char* d2 = d1 + f1_bytes;
        dma16<kThreads>(Fb + t.offF1, d1, n1 >> 1, tid);
        if (n1 & 1) dma8(Fb + t.offF1 + (n1 - 1), d1 + 8 * (size_t)(n1 - 1), tid);
        dma16<kThreads>(Fb + t.offF2, d2, n2 >> 1, tid);
        if (n2 & 1) dma8(Fb + t.offF2 + (n2 - 1), d2 + 8 * (size_t)(n2 - 1), tid);
    };

    const int nitems = t.nT1 * t.nT2 * M;
    const bool single = nitems <= kThreads;                       // one item per thread: set up once
    FwdItem<TI, TJ> mine;
    if (single && tid < nitems) fwd_item_setup<TI, TJ>(t, tid, cg, f1_0, f2_0, mine);

    double s1[4] = {0., 0., 0., 0.}, s2[4] = {0., 0., 0., 0.};
    const int b0 = group * samples_per_group;
    const int b1 = min(B, b0 + samples_per_group);
    if (b0 < b1) issue(b0, 0);
    for (int e = tid; e < ncg; e += kThreads) cg[e] = CG[t.cg_off + e];
    int par = 0;
    for (int b = b0; b < b1; ++b, par ^= 1) {
        dma_wait();
        __syncthreads();       // this sample's fragments landed; the previous tile has been copied out
        if (b + 1 < b1) issue(b + 1, par ^ 1);
        const unsigned bufofs = (unsigned)(par * frag_bytes);
        if (single) {
            if (tid < nitems) fwd_item_run<TI, TJ>(t, mine, bufofs, out);
        } else {
            for (int item = tid; item < nitems; item += kThreads) {
                FwdItem<TI, TJ> it;
                fwd_item_setup<TI, TJ>(t, item, cg, f1_0, f2_0, it);
                fwd_item_run<TI, TJ>(t, it, bufofs, out);
            }
        }
        __syncthreads();
        // tile -> FF with 16-byte stores from the first 16-byte boundary on
        float2* dst = FF + (size_t)b * nFF + t.offFF;
        const int head = min(nout, (int)((reinterpret_cast<uintptr_t>(dst) >> 3) & 1));
        const int npair = (nout - head) >> 1;
        float4* dst4 = reinterpret_cast<float4*>(dst + head);
        for (int e = tid; e < npair; e += kThreads) {
            const float2 u = out[head + 2 * e], v = out[head + 2 * e + 1];
            stream_store16(dst4 + e, u.x, u.y, v.x, v.y);
        }
        if (tid == 0 && head) dst[0] = out[0];
        if (tid == 1 && ((nout - head) & 1)) dst[nout - 1] = out[nout - 1];
        if (stats_part) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int ch = tid + kThreads * k;
                if (ch < nch) {
                    // both sums run over the same rounded |z| in double: the variance formed from them
                    // later is then free of cancellation between inconsistently rounded terms
                    double a = s1[k], q = s2[k];
                    for (int mm = 0; mm < M; ++mm) {
                        const float2 z = out[ch * M + mm];
                        const double r = (double)sqrt_hw(fmaf(z.x, z.x, z.y * z.y));
                        a += r;
                        q = fma(r, r, q);
                    }
                    s1[k] = a;
                    s2[k] = q;
                }
            }
        }
    }
    if (stats_part) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int ch = tid + kThreads * k;
            if (ch < nch) {
                double* p = stats_part + ((size_t)group * sumT + t.chan0 + ch) * 2;
                p[0] = s1[k];
                p[1] = s2[k];
            }
        }
    }
}

__global__ void __launch_bounds__(kThreads)
cg_forward_kernel(const float2* __restrict__ F, float2* __restrict__ FF, const float* __restrict__ CG,
                  const CgTask* __restrict__ tasks, int nF, int nFF, int B, int samples_per_group,
                  double* __restrict__ stats_part, int sumT) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = part_major((B + samples_per_group - 1) / samples_per_group);
    const CgTask t = tasks[up.unit];
    const int group = up.part;
#define CGNET_FWD(TI_, TJ_) \
    case (TI_) * 8 + (TJ_): fwd_group<TI_, TJ_>(t, F, FF, CG, nF, nFF, B, samples_per_group, group, stats_part, sumT, smem); break;
    switch (min(t.TI, 4) * 8 + min(t.TJ, 4)) {
        CGNET_FWD(1, 1) CGNET_FWD(1, 2) CGNET_FWD(1, 3) CGNET_FWD(1, 4)
        CGNET_FWD(2, 1) CGNET_FWD(2, 2) CGNET_FWD(2, 3) CGNET_FWD(2, 4)
        CGNET_FWD(3, 1) CGNET_FWD(3, 2) CGNET_FWD(3, 3) CGNET_FWD(3, 4)
        CGNET_FWD(4, 1) CGNET_FWD(4, 2) CGNET_FWD(4, 3)
        default: fwd_group<4, 4>(t, F, FF, CG, nF, nFF, B, samples_per_group, group, stats_part, sumT, smem); break;
    }
#undef CGNET_FWD
}

// ---- forward on the matrix cores ---------------------------------------------------------------
// For a fixed output m the tile's channels are a small matrix product:
//   FF_m[t1, t2] = sum_m2 (C[m][m2] F1[t1][m - m2]) * F2[t2][m2]              (rows x terms) . (terms x tau2)
// rows of the accumulator = the up to 16 rows of the task, columns = the up to 16 channels of degree l2, the
// reduction runs over the valid m2 in steps of four (v_mfma_f32_16x16x4_f32; complex numbers as four real
// products per step).  Only the left operand needs arithmetic (one coefficient times one fragment entry per lane
// and step); the right operand is read as it lies in the staged l2 slab.  No masking: the table is staged with three
// zeros behind every row, and holds zeros where m - m2 is no valid m1 (every table this library fills does), so the
// steps past the last valid m2 multiply whatever finite fragment entries lie next to the rows by zero (LDS is
// cleared once, the slabs have 32 spare bytes on either side).  The eight waves take the values of m in turn,
// numbered from the middle outwards, and write their 16 x 16 results into the output tile; the tile then leaves as
// in the vector-ALU kernel.  Used when every channel count is in 8..16.
constexpr int kFwdMmPad = 32;     // bytes before / between / behind the fragment buffers
constexpr size_t kFwdMmStatsLds = 8 * 256 * sizeof(double);   // eight waves x four values x 64 lanes

__host__ __device__ inline size_t fwd_task_lds_mm(const CgTask& t) {
    const size_t M = 2 * t.l + 1, M2 = 2 * t.l2 + 1;
    const size_t need = kFwdMmPad + 2 * (fwd_frag_lds(t) + kFwdMmPad) +
                        ((8 * (size_t)t.rows * t.tau2 * M + 15) & ~(size_t)15) + ((4 * M * (M2 + 3) + 15) & ~(size_t)15);
    return need > kFwdMmStatsLds ? need : kFwdMmStatsLds;     // the statistics' final reduction runs through LDS
}

// One sample of a task: the waves take the values of m in turn (from the middle outwards, so that every wave gets
// long and short ones); for one m the accumulator D[t1][t2] gathers the steps of four m2.
// STATS: the lane also adds |z| and |z|^2 of its four results (channels (4 kk + v, i)) to its own sums.
template <bool STATS>
__device__ __forceinline__ void fwd_mm_sample(const CgTask& t, const float* __restrict__ cg, int P,
                                              const float2* __restrict__ f1, const float2* __restrict__ f2,
                                              float2* __restrict__ out, int wave, int nwaves, int lane,
                                              double (&s1)[4], double (&s2)[4]) {
    const int l = t.l, l1 = t.l1, l2 = t.l2;
    const int M = 2 * l + 1, M1 = 2 * l1 + 1, M2 = 2 * l2 + 1;
    const int rows = t.rows, tau2 = t.tau2;
    const int i = lane & 15, kk = lane >> 4;
    // Channel of the result (row r = 4 kk + v, column i): r tau2 + i.  In the compact tile of a diagonal triple only
    // the columns i >= r exist, column after column: i (i + 1) / 2 + r -- so that in both layouts the four results
    // of a lane lie a constant number of channels apart.
    const int r0 = 4 * kk;
    const int chan_lane = t.sym ? i * (i + 1) / 2 + r0 : r0 * tau2 + i;
    const int chan_step = t.sym ? 1 : tau2;
    const int last_row = t.sym ? min(rows - 1, i) : rows - 1;     // rows r0 + v <= last_row are stored
    // rows / channels past the end repeat the last one (their results are not stored)
    const unsigned a_row = lds_addr(f1 + min(i, rows - 1) * M1);
    const unsigned b_row = lds_addr(f2 + min(i, tau2 - 1) * M2);
    const unsigned c_lane = lds_addr(cg + kk);
    for (int mslot = wave; mslot < M; mslot += nwaves) {
        const int mm = (mslot & 1) ? l + ((mslot + 1) >> 1) : l - (mslot >> 1);
        const int m = mm - l;
        const int lo = max(-l2, m - l1), hi = min(l2, m + l1);
        const int nsteps = (hi - lo + 4) >> 2;
        // lane kk of a step takes m2 = lo + 4 s + kk, i.e. m1 = m - m2; past hi the table pitch holds zeros and the
        // fragment reads stay inside the padded buffers
        unsigned pa = opaque(a_row + 8u * (unsigned)(m - lo + l1 - kk));
        unsigned pb = opaque(b_row + 8u * (unsigned)(lo + l2 + kk));
        unsigned pc = opaque(c_lane + 4u * (unsigned)(mm * P + lo + l2));
        // the first step starts from constant zero accumulators (every m has at least one step: the plan only
        // admits triples that obey the triangle rule)
        f32x4 dre, dim;
        {
            const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
            const float c = lds_f(pc)[0];
            const float2 fa = lds_c(pa, 0), fb = lds_c(pb, 0);
            pa -= 32u;
            pb += 32u;
            pc += 16u;
            const float ar = c * fa.x, ai = c * fa.y, nai = -ai;
            dre = mfma4(ar, fb.x, zero);
            dim = mfma4(ar, fb.y, zero);
            dre = mfma4(nai, fb.y, dre);
            dim = mfma4(ai, fb.x, dim);
        }
        for (int s = 1; s < nsteps; ++s) {
            const float c = lds_f(pc)[0];
            const float2 fa = lds_c(pa, 0), fb = lds_c(pb, 0);
            pa -= 32u;
            pb += 32u;
            pc += 16u;
            const float ar = c * fa.x, ai = c * fa.y, nai = -ai;
            dre = mfma4(ar, fb.x, dre);
            dim = mfma4(ar, fb.y, dim);
            dre = mfma4(nai, fb.y, dre);
            dim = mfma4(ai, fb.x, dim);
        }
        if (i < tau2) {
            // re and im go out as two 4-byte writes (one two-address LDS instruction): an 8-byte write would first
            // copy the pair into adjacent registers
            float* o = reinterpret_cast<float*>(out + chan_lane * M + mm);
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (r0 + v <= last_row) {
                    o[2 * v * chan_step * M] = dre[v];
                    o[2 * v * chan_step * M + 1] = dim[v];
                }
        }
        if (STATS) {
            // both sums run over the same rounded |z| in double (see cg_forward_kernel); lanes past the task's
            // channels add up values nobody reads
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const double r = (double)sqrt_hw(fmaf(dre[v], dre[v], dim[v] * dim[v]));
                s1[v] += r;
                s2[v] = fma(r, r, s2[v]);
            }
        }
    }
}

constexpr int kFwdMmThreads = 512;

__global__ void __launch_bounds__(kFwdMmThreads, 8)    // 64 registers: four work-groups per compute unit
cg_forward_mm_kernel(const float2* __restrict__ F, float2* __restrict__ FF, const float* __restrict__ CG,
                     const CgTask* __restrict__ tasks, int nF, int nFF, int B, int samples_per_group,
                     double* __restrict__ stats_part, int sumT, int lds_bytes) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = part_major((B + samples_per_group - 1) / samples_per_group);
    const CgTask t = tasks[up.unit];
    const int group = up.part;
    const int M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
    const int P = M2 + 3;
    // channels the tile holds in memory: all rows x tau2, or the upper triangle of a compact diagonal tile (the LDS
    // is laid out for the full tile either way)
    const int nch = t.sym ? t.rows * (t.rows + 1) / 2 : t.rows * t.tau2;
    const int nout = nch * M, n1 = t.rows * M1, n2 = t.tau2 * M2;
    const size_t out_bytes = (8 * (size_t)t.rows * t.tau2 * M + 15) & ~(size_t)15;
    const size_t f1_bytes = (8 * (size_t)n1 + 15) & ~(size_t)15;
    const size_t frag_bytes = fwd_frag_lds(t) + kFwdMmPad;          // one buffer and the pad behind it
    unsigned char* frag = smem + kFwdMmPad;                        // [2][frag_bytes]
    float2* out = reinterpret_cast<float2*>(frag + 2 * frag_bytes);
    float* cg = reinterpret_cast<float*>(frag + 2 * frag_bytes + out_bytes);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    {
        float4* z = reinterpret_cast<float4*>(smem);
        for (int e = tid; e < (lds_bytes >> 4); e += kFwdMmThreads) z[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();                                               // the clearing stores precede every copy
    auto issue = [&](int b, int par) {
        const float2* Fb = F + (size_t)b * nF;
        unsigned char* d1 = frag + par * frag_bytes;
        unsigned char* d2 = d1 + f1_bytes;
        dma16<kFwdMmThreads>(Fb + t.offF1, d1, n1 >> 1, tid);
        if (n1 & 1) dma8(Fb + t.offF1 + (n1 - 1), d1 + 8 * (size_t)(n1 - 1), tid);
        dma16<kFwdMmThreads>(Fb + t.offF2, d2, n2 >> 1, tid);
        if (n2 & 1) dma8(Fb + t.offF2 + (n2 - 1), d2 + 8 * (size_t)(n2 - 1), tid);
    };
    double s1[4] = {0., 0., 0., 0.}, s2[4] = {0., 0., 0., 0.};   // of the lane's channels, over its m and all samples
    const int b0 = group * samples_per_group;
    const int b1 = min(B, b0 + samples_per_group);
    if (b0 < b1) issue(b0, 0);
    // the table with three zeros behind every row (the zeros are the cleared LDS); entries whose m1 = m - m2 is no
    // valid index of degree l1 are staged as zeros whatever the caller's table holds there (the kernel multiplies
    // them with neighbouring fragment entries and relies on the product being zero)
    for (int e = tid; e < M * M2; e += kFwdMmThreads) {
        const int r = e / M2, c = e - r * M2;
        const int m1 = (r - t.l) - (c - t.l2);
        cg[r * P + c] = (m1 >= -t.l1 && m1 <= t.l1) ? CG[t.cg_off + e] : 0.f;
    }
    int par = 0;
    for (int b = b0; b < b1; ++b, par ^= 1) {
        dma_wait();
        __syncthreads();       // this sample's fragments landed; the previous tile has been copied out
        if (b + 1 < b1) issue(b + 1, par ^ 1);
        const float2* f1 = reinterpret_cast<const float2*>(frag + par * frag_bytes);
        const float2* f2 = reinterpret_cast<const float2*>(frag + par * frag_bytes + f1_bytes);
        if (stats_part) fwd_mm_sample<true>(t, cg, P, f1, f2, out, wave, kFwdMmThreads / 64, lane, s1, s2);
        else fwd_mm_sample<false>(t, cg, P, f1, f2, out, wave, kFwdMmThreads / 64, lane, s1, s2);
        __syncthreads();
        // tile -> FF with 16-byte stores from the first 16-byte boundary on
        float2* dst = FF + (size_t)b * nFF + t.offFF;
        const int head = min(nout, (int)((reinterpret_cast<uintptr_t>(dst) >> 3) & 1));
        const int npair = (nout - head) >> 1;
        float4* dst4 = reinterpret_cast<float4*>(dst + head);
        for (int e = tid; e < npair; e += kFwdMmThreads) {
            const float2 u = out[head + 2 * e], v = out[head + 2 * e + 1];
            stream_store16(dst4 + e, u.x, u.y, v.x, v.y);
        }
        if (tid == 0 && head) dst[0] = out[0];
        if (tid == 1 && ((nout - head) & 1)) dst[nout - 1] = out[nout - 1];
    }
    if (stats_part) {
        // The eight waves hold partial sums of the same channels (each over its own m).  They go through LDS
        // (everything else in it is no longer needed) in two rounds of four values per lane, and one thread
        // per channel adds the waves in order.
        double* red = reinterpret_cast<double*>(smem);            // [wave][value 0..3][lane]
#pragma unroll
        for (int round = 0; round < 2; ++round) {
            __syncthreads();                                       // the last tile has left / round 0 has been read
#pragma unroll
            for (int v = 0; v < 4; ++v) red[(wave * 4 + v) * 64 + lane] = round == 0 ? s1[v] : s2[v];
            __syncthreads();
            // thread -> channel (row r, column c) of the task; its value lies at lane (r / 4) * 16 + c, slot r % 4
            for (int ch = tid; ch < nch; ch += kFwdMmThreads) {
                int r = ch / t.tau2, c = ch - r * t.tau2;
                if (t.sym) {                                       // compact tile: column c holds the rows 0 .. c
                    c = 0;
                    r = ch;
                    while (r > c) {
                        r -= c + 1;
                        ++c;
                    }
                }
                const int src = (r & 3) * 64 + (r >> 2) * 16 + c;
                double sum = 0.;
#pragma unroll
                for (int w = 0; w < kFwdMmThreads / 64; ++w) sum += red[w * 256 + src];
                stats_part[((size_t)group * sumT + t.chan0 + ch) * 2 + round] = sum;
            }
        }
    }
}

// ---- inference forward of the whole layer: the product tile is mixed while it lies in LDS -------------------------
// cg_forward_mm_kernel whose tile never leaves for memory: when a sample's tile of a task is complete, the eight waves
// multiply it with the task's slice of the weights, O_part[to, m] = sum over the tile's channels c of
// (W[to, c] / div[c]) FF[c, m], on the matrix cores (rows = the up to 16 output channels, columns = T tiles of 16
// values of m with re / im of a column in one lane, reduction over the channels in steps of four), and what leaves
// is the task's t_O x (2l+1) partial output, a twelfth of the tile.  cgbn_forward_reduce_kernel adds the partial
// outputs of a degree's tasks in channel order.  A wave has a role (column tile, share of the reduction steps) and
// keeps its share of the packed weights in registers for all samples of the group; the shares meet in LDS.
// Statistics cannot be taken on this route (the mixing needs the stds of the whole batch before the first tile): it
// serves evaluation mode and layers without fragment norm.
constexpr int kMixMaxK = 16;                   // reduction steps of one wave (64 channels)
constexpr int kMixShares = 4;                  // shares of the reduction steps of a column tile: one wave per SIMD
constexpr size_t kMixShareBytes = 2048;        // a share's 16 x 16 complex partial sums

__host__ __device__ constexpr size_t mix_red_bytes(int T) { return (size_t)T * (kMixShares - 1) * kMixShareBytes; }

template <int T>
__global__ void __launch_bounds__(kFwdMmThreads, 6)
cgbn_forward_fused_kernel(const float2* __restrict__ F, const float* __restrict__ CG, const CgTask* __restrict__ tasks,
                          const FwdMixTask* __restrict__ mix, const int* __restrict__ sel, const float* __restrict__ Af,
                          float2* __restrict__ Opart, int nF, int B, int samples_per_group, int opart, int lds_bytes) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = part_major((B + samples_per_group - 1) / samples_per_group);
    const int unit = sel[up.unit];                                 // the launch's tasks: those with T column tiles
    const CgTask t = tasks[unit];
    const FwdMixTask g = mix[unit];
    const int group = up.part;
    const int M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
    const int P = M2 + 3;
    const int nch = t.rows * t.tau2;
    const int nout = nch * M, n1 = t.rows * M1, n2 = t.tau2 * M2;
    const size_t out_bytes = (8 * (size_t)nout + 15) & ~(size_t)15;
    const size_t f1_bytes = (8 * (size_t)n1 + 15) & ~(size_t)15;
    const size_t frag_bytes = fwd_frag_lds(t) + kFwdMmPad;
    unsigned char* frag = smem + kFwdMmPad;                        // [2][frag_bytes]
    float2* out = reinterpret_cast<float2*>(frag + 2 * frag_bytes);
    float* cg = reinterpret_cast<float*>(frag + 2 * frag_bytes + out_bytes);
    float4* red = reinterpret_cast<float4*>(smem + lds_bytes - mix_red_bytes(T));   // [share - 1][column tile][2][64]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    {
        float4* z = reinterpret_cast<float4*>(smem);
        for (int e = tid; e < (lds_bytes >> 4); e += kFwdMmThreads) z[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();                                               // the clearing stores precede every copy
    auto issue = [&](int b, int par) {
        const float2* Fb = F + (size_t)b * nF;
        unsigned char* d1 = frag + par * frag_bytes;
        unsigned char* d2 = d1 + f1_bytes;
        dma16<kFwdMmThreads>(Fb + t.offF1, d1, n1 >> 1, tid);
        if (n1 & 1) dma8(Fb + t.offF1 + (n1 - 1), d1 + 8 * (size_t)(n1 - 1), tid);
        dma16<kFwdMmThreads>(Fb + t.offF2, d2, n2 >> 1, tid);
        if (n2 & 1) dma8(Fb + t.offF2 + (n2 - 1), d2 + 8 * (size_t)(n2 - 1), tid);
    };
    const int b0 = group * samples_per_group;
    const int b1 = min(B, b0 + samples_per_group);
    if (b0 < b1) issue(b0, 0);
    for (int e = tid; e < M * M2; e += kFwdMmThreads) {            // the table, as in cg_forward_mm_kernel
        const int r = e / M2, c = e - r * M2;
        const int m1 = (r - t.l) - (c - t.l2);
        cg[r * P + c] = (m1 >= -t.l1 && m1 <= t.l1) ? CG[t.cg_off + e] : 0.f;
    }
    // role of the wave in the mixing: column tile tcol, share kh of the reduction steps.  Four shares put one wave of
    // a column tile on every SIMD; with one column tile the other four waves only take part in the product.
    const int tcol = wave % T, kh = wave / T;
    const bool mixing = kh < kMixShares && g.nks > 0;
    const int ks0 = mixing ? (kh * g.nks) / kMixShares : 0, ks1 = mixing ? ((kh + 1) * g.nks) / kMixShares : 0;
    const int cnt = ks1 - ks0;                                     // <= kMixMaxK (the plan checks)
    float2 a[kMixMaxK];
#pragma unroll
    for (int j = 0; j < kMixMaxK; ++j)
        a[j] = j < cnt ? reinterpret_cast<const float2*>(Af + g.aoff)[(size_t)(ks0 + j) * 64 + lane] : make_float2(0.f, 0.f);
    const int i = lane & 15, kk = lane >> 4;
    const int col = 16 * tcol + i;
    const unsigned pb_last = lds_addr(out + (nch - 1) * M + min(col, M - 1));
    const unsigned pb_first = lds_addr(out + (4 * ks0 + kk) * M + min(col, M - 1));
    const unsigned pb_step = 32u * (unsigned)M;                    // four channels further
    double dummy1[4] = {0., 0., 0., 0.}, dummy2[4] = {0., 0., 0., 0.};   // the statistics half of fwd_mm_sample's interface
    int par = 0;
    for (int b = b0; b < b1; ++b, par ^= 1) {
        dma_wait();
        __syncthreads();       // this sample's fragments landed; the previous sample's partial sums have been read
        if (b + 1 < b1) issue(b + 1, par ^ 1);
        const float2* f1 = reinterpret_cast<const float2*>(frag + par * frag_bytes);
        const float2* f2 = reinterpret_cast<const float2*>(frag + par * frag_bytes + f1_bytes);
        fwd_mm_sample<false>(t, cg, P, f1, f2, out, wave, kFwdMmThreads / 64, lane, dummy1, dummy2);
        lds_barrier();         // the tile is complete
        f32x4 xr = {0.f, 0.f, 0.f, 0.f}, yr = xr, xi = xr, yi = xr;
        if (mixing) {
            unsigned pb = pb_first;
#pragma unroll
            for (int j = 0; j < kMixMaxK; ++j) {
                if (j < cnt) {
                    const float2 v = lds_c(min(pb, pb_last), 0);   // channels past the tile's last meet zero weights
                    pb += pb_step;
                    xr = mfma4(a[j].x, v.x, xr);
                    yr = mfma4(a[j].x, v.y, yr);
                    xi = mfma4(a[j].y, v.x, xi);
                    yi = mfma4(a[j].y, v.y, yi);
                }
            }
        }
        // (W_re + i W_im)(x + i y): re = W_re x - W_im y, im = W_re y + W_im x
        float4 ore = make_float4(xr[0] - yi[0], xr[1] - yi[1], xr[2] - yi[2], xr[3] - yi[3]);
        float4 oim = make_float4(yr[0] + xi[0], yr[1] + xi[1], yr[2] + xi[2], yr[3] + xi[3]);
        if (mixing && kh > 0) {
            float4* mine = red + ((kh - 1) * T + tcol) * 128;
            mine[lane] = ore;
            mine[64 + lane] = oim;
        }
        lds_barrier();         // the shares have been written; nobody reads the tile any more
        if (kh == 0 && g.tO > 0) {
            // the wave that holds share 0 of its column tile adds the others in order and stores the partial output
            if (g.nks > 0) {
#pragma unroll
                for (int k = 1; k < kMixShares; ++k) {
                    const float4* theirs = red + ((k - 1) * T + tcol) * 128;
                    const float4 r = theirs[lane], q = theirs[64 + lane];
                    ore.x += r.x; ore.y += r.y; ore.z += r.z; ore.w += r.w;
                    oim.x += q.x; oim.y += q.y; oim.z += q.z; oim.w += q.w;
                }
            }
            float2* dst = Opart + (size_t)b * opart + g.ooff + (4 * kk) * M + col;
            if (col < M) {
                if (4 * kk + 0 < g.tO) dst[0] = make_float2(ore.x, oim.x);
                if (4 * kk + 1 < g.tO) dst[M] = make_float2(ore.y, oim.y);
                if (4 * kk + 2 < g.tO) dst[2 * M] = make_float2(ore.z, oim.z);
                if (4 * kk + 3 < g.tO) dst[3 * M] = make_float2(ore.w, oim.w);
            }
        }
    }
}

// O[b][degree l][to][m] = sum of the partial outputs of the degree's tasks, in channel order.
// meta: [L+2] cumO | [L+1] t_O | [L+2] list begin | the ooff of every task, degree by degree
__global__ void __launch_bounds__(256)
cgbn_forward_reduce_kernel(const float2* __restrict__ Opart, float2* __restrict__ O, const int* __restrict__ meta,
                           int L, int nO, int opart, int B) {
    __shared__ int s_tab[kMaxLookup];
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int b = (int)(idx / nO), e = (int)(idx % nO);
    const int* cumO = meta;                 // L+2
    const int* lbeg = meta + (L + 2) + (L + 1);
    const int* loff = lbeg + (L + 2);
    const int lam = lookup_in_group(L + 1, e, [&](int k) { return cumO[k]; }, s_tab);
    if (idx >= (size_t)B * nO) return;
    const int rel = e - cumO[lam];
    const float2* p = Opart + (size_t)b * opart;
    float2 sum = make_float2(0.f, 0.f);
#pragma unroll 8
    for (int k = lbeg[lam]; k < lbeg[lam + 1]; ++k) {
        const float2 v = p[loff[k] + rel];
        sum.x += v.x;
        sum.y += v.y;
    }
    O[idx] = sum;
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

// Zero padding of the m axis of the staged gFF tile and of the CG table rows: the two m
// outputs of a thread and the two-step unrolled loop may touch one index below and two above.
constexpr int kPadLo = 1, kPadHi = 3;

__host__ __device__ inline size_t bwd_task_lds(const CgTask& t) {
    const size_t M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
    const size_t Mp = M + kPadLo + kPadHi;
    return 8 * ((size_t)t.rows * t.tau2 * Mp + (size_t)t.rows * M1 + (size_t)t.tau2 * M2) + 4 * Mp * M2;
}

// Gradient with respect to the slot that is NOT reduced over.
//   SLOT == 1: outputs (t1 in the task's rows, m1), reduced over (t2, m2)
//   SLOT == 2: outputs (t2, m2),                    reduced over (t1 in rows, m1)
// A thread owns TI output channels x 2 consecutive m; RW lanes share one such item and split
// the reduced channels, then add up over a fixed DPP tree.  Along the reduced m the two
// outputs read a sliding two-element window of the staged gFF tile (g, rows padded with zeros),
// so a step costs TI + 1 + 2 LDS reads for 2*TI complex multiply-adds.
template <int SLOT, int TI, int RW>
__device__ __forceinline__ void bwd_phase(const CgTask& t, const float* __restrict__ cgp,
                                          const float2* __restrict__ g, const float2* __restrict__ fr,
                                          float2* __restrict__ acc, int nthreads) {
    const int l = t.l, l1 = t.l1, l2 = t.l2;
    const int M = 2 * l + 1, M1 = 2 * l1 + 1, M2 = 2 * l2 + 1;
    const int Mp = M + kPadLo + kPadHi;
    const int rows = t.rows, tau2 = t.tau2;
    const int n_o = (SLOT == 1) ? rows : tau2;        // output channels
    const int n_r = (SLOT == 1) ? tau2 : rows;        // reduced channels
    const int M_o = (SLOT == 1) ? M1 : M2, M_r = (SLOT == 1) ? M2 : M1;
    const int g_so = (SLOT == 1) ? tau2 * Mp : Mp;    // stride in g between output channels
    const int g_sr = (SLOT == 1) ? Mp : tau2 * Mp;    // stride in g between reduced channels
    const int out_base = (SLOT == 1) ? t.offF1 : t.offF2;
    const int d = l1 + l2 - l;                        // m index of g = mo + mr - d (all 0-based)

    const int nrows_blk = nthreads / RW;
    const int row_id = threadIdx.x / RW, lane_r = threadIdx.x % RW;
    const int nT = (n_o + TI - 1) / TI;
    const int nWin = (M_o + 1) >> 1;
    const int nitems = nT * nWin;
    const int npass = (nitems + nrows_blk - 1) / nrows_blk;
    for (int pass = 0; pass < npass; ++pass) {
        const int item = pass * nrows_blk + row_id;
        const bool valid = item < nitems;
        float ax[TI][2], ay[TI][2];
#pragma unroll
        for (int i = 0; i < TI; ++i) ax[i][0] = ax[i][1] = ay[i][0] = ay[i][1] = 0.f;
        int mo0 = 0, to = 0;
        if (valid) {
            const int w = item % nWin;
            to = item / nWin;
            mo0 = 2 * w;
            // reduced-m range in which at least one of the two outputs has 0 <= m index < M
            const int ir_lo = max(0, d - mo0 - 1);
            const int ir_hi = min(M_r - 1, M - 1 + d - mo0);
            int go[TI];
#pragma unroll
            for (int i = 0; i < TI; ++i) go[i] = min(to + nT * i, n_o - 1) * g_so;
            const int col0 = min(mo0, M2 - 1), col1 = min(mo0 + 1, M2 - 1);   // SLOT 2: table columns
            for (int r = lane_r; r < n_r; r += RW) {
                const float2* frow = fr + r * M_r;
                const float2* gb = g + r * g_sr + (kPadLo + mo0 - d);          // gb[ch + ir] = g[.., m = mo0+ir-d]
                const float* cb = cgp + (kPadLo + mo0 - d) * M2;               // cb[ir*M2 + col] = table row mo0+ir-d
                float2 e0[TI], e1[TI];
#pragma unroll
                for (int i = 0; i < TI; ++i) e0[i] = gb[go[i] + ir_lo];
                for (int ir = ir_lo; ir <= ir_hi; ir += 2) {
                    // ---- step ir: outputs (mo0, mo0+1) read (e0, e1)
#pragma unroll
                    for (int i = 0; i < TI; ++i) e1[i] = gb[go[i] + ir + 1];
                    {
                        const float2 f = frow[ir];
                        const float c0 = (SLOT == 1) ? cb[ir * M2 + ir] : cb[ir * M2 + col0];
                        const float c1 = (SLOT == 1) ? cb[(ir + 1) * M2 + ir] : cb[(ir + 1) * M2 + col1];
                        const float c0x = c0 * f.x, c0y = -c0 * f.y, c1x = c1 * f.x, c1y = -c1 * f.y;
#pragma unroll
                        for (int i = 0; i < TI; ++i) {
                            ax[i][0] = fmaf(e0[i].x, c0x, ax[i][0]);
                            ax[i][0] = fmaf(-e0[i].y, c0y, ax[i][0]);
                            ay[i][0] = fmaf(e0[i].x, c0y, ay[i][0]);
                            ay[i][0] = fmaf(e0[i].y, c0x, ay[i][0]);
                            ax[i][1] = fmaf(e1[i].x, c1x, ax[i][1]);
                            ax[i][1] = fmaf(-e1[i].y, c1y, ax[i][1]);
                            ay[i][1] = fmaf(e1[i].x, c1y, ay[i][1]);
                            ay[i][1] = fmaf(e1[i].y, c1x, ay[i][1]);
                        }
                    }
                    // ---- step ir+1: the window has moved by one, roles of e0 / e1 swap
#pragma unroll
                    for (int i = 0; i < TI; ++i) e0[i] = gb[go[i] + ir + 2];
                    {
                        const int ir1 = ir + 1;
                        const int irc = min(ir1, M_r - 1);
                        float2 f = frow[irc];
                        if (ir1 > ir_hi) f = make_float2(0.f, 0.f);
                        const float c0 = (SLOT == 1) ? cb[ir1 * M2 + irc] : cb[ir1 * M2 + col0];
                        const float c1 = (SLOT == 1) ? cb[(ir1 + 1) * M2 + irc] : cb[(ir1 + 1) * M2 + col1];
                        const float c0x = c0 * f.x, c0y = -c0 * f.y, c1x = c1 * f.x, c1y = -c1 * f.y;
#pragma unroll
                        for (int i = 0; i < TI; ++i) {
                            ax[i][0] = fmaf(e1[i].x, c0x, ax[i][0]);
                            ax[i][0] = fmaf(-e1[i].y, c0y, ax[i][0]);
                            ay[i][0] = fmaf(e1[i].x, c0y, ay[i][0]);
                            ay[i][0] = fmaf(e1[i].y, c0x, ay[i][0]);
                            ax[i][1] = fmaf(e0[i].x, c1x, ax[i][1]);
                            ax[i][1] = fmaf(-e0[i].y, c1y, ax[i][1]);
                            ay[i][1] = fmaf(e0[i].x, c1y, ay[i][1]);
                            ay[i][1] = fmaf(e0[i].y, c1x, ay[i][1]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int i = 0; i < TI; ++i) {
            ax[i][0] = row_sum<RW>(ax[i][0]);
            ay[i][0] = row_sum<RW>(ay[i][0]);
            ax[i][1] = row_sum<RW>(ax[i][1]);
            ay[i][1] = row_sum<RW>(ay[i][1]);
        }
        if (valid) {
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                if (lane_r != (k % RW)) continue;        // lane k of the row stores output k
                const int mo = mo0 + k;
                if (mo >= M_o) continue;
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const int ch = to + nT * i;
                    if (ch < n_o) {
                        float2* p = acc + out_base + ch * M_o + mo;
                        float2 v = *p;
                        v.x += ax[i][k];
                        v.y += ay[i][k];
                        *p = v;
                    }
                }
            }
        }
    }
}

template <int SLOT, int TI>
__device__ __forceinline__ void bwd_phase_rw(int rw, const CgTask& t, const float* cgp, const float2* g,
                                             const float2* fr, float2* acc, int nthreads) {
    switch (rw) {
        case 1: bwd_phase<SLOT, TI, 1>(t, cgp, g, fr, acc, nthreads); break;
        case 2: bwd_phase<SLOT, TI, 2>(t, cgp, g, fr, acc, nthreads); break;
        case 4: bwd_phase<SLOT, TI, 4>(t, cgp, g, fr, acc, nthreads); break;
        case 8: bwd_phase<SLOT, TI, 8>(t, cgp, g, fr, acc, nthreads); break;
        default: bwd_phase<SLOT, TI, 16>(t, cgp, g, fr, acc, nthreads); break;
    }
}

template <int SLOT>
__device__ __forceinline__ void bwd_phase_dispatch(const CgTask& t, const float* cgp, const float2* g,
                                                   const float2* fr, float2* acc, int nthreads) {
    const int ti = t.bTI[SLOT - 1], rw = t.bRW[SLOT - 1];
    switch (ti) {
        case 1: bwd_phase_rw<SLOT, 1>(rw, t, cgp, g, fr, acc, nthreads); break;
        case 2: bwd_phase_rw<SLOT, 2>(rw, t, cgp, g, fr, acc, nthreads); break;
        case 3: bwd_phase_rw<SLOT, 3>(rw, t, cgp, g, fr, acc, nthreads); break;
        default: bwd_phase_rw<SLOT, 4>(rw, t, cgp, g, fr, acc, nthreads); break;
    }
}

__global__ void __launch_bounds__(kThreads)
cg_backward_kernel(const float2* __restrict__ F, const float2* __restrict__ gFF,
                   const float* __restrict__ CG, float2* __restrict__ dst,
                   const CgTask* __restrict__ tasks, const int* __restrict__ group_begin,
                   int nF, int nFF, int B) {
    extern __shared__ __align__(16) unsigned char smem[];
    float2* acc = reinterpret_cast<float2*>(smem);
    float2* g = acc + nF;
    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int b = blockIdx.y, grp = blockIdx.x;
    for (int e = tid; e < nF; e += nthreads) acc[e] = make_float2(0.f, 0.f);
    const float2* Fb = F + (size_t)b * nF;
    const float2* Gb = gFF + (size_t)b * nFF;
    const int tbeg = group_begin[grp], tend = group_begin[grp + 1];
    for (int ti = tbeg; ti < tend; ++ti) {
        const CgTask t = tasks[ti];
        const int M = 2 * t.l + 1, M1 = 2 * t.l1 + 1, M2 = 2 * t.l2 + 1;
        const int Mp = M + kPadLo + kPadHi;
        const int nch = t.rows * t.tau2;
        const int n1 = t.rows * M1, n2 = t.tau2 * M2;
        float2* f1 = g + nch * Mp;
        float2* f2 = f1 + n1;
        float* cgp = reinterpret_cast<float*>(f2 + n2);
        __syncthreads();   // previous task (and the zeroing) done before the staging area is reused
        {
            const float inv = 1.0f / (float)Mp;
            const float2* src = Gb + t.offFF;
            for (int e = tid; e < nch * Mp; e += nthreads) {
                const int ch = (int)(((float)e + 0.5f) * inv);
                const int x = e - ch * Mp - kPadLo;
                float2 v = make_float2(0.f, 0.f);
                if (x >= 0 && x < M) v = src[ch * M + x];
                g[e] = v;
            }
        }
        for (int e = tid; e < n1; e += nthreads) f1[e] = Fb[t.offF1 + e];
        for (int e = tid; e < n2; e += nthreads) f2[e] = Fb[t.offF2 + e];
        for (int e = tid; e < Mp * M2; e += nthreads) {
            const int x = e - kPadLo * M2;
            cgp[e] = (x >= 0 && x < M * M2) ? CG[t.cg_off + x] : 0.f;
        }
        __syncthreads();
        bwd_phase_dispatch<1>(t, cgp, g, f2, acc, nthreads);
        __syncthreads();   // a diagonal triple writes the same slab in both phases
        bwd_phase_dispatch<2>(t, cgp, g, f1, acc, nthreads);
    }
    __syncthreads();
    float2* out = dst + ((size_t)grp * B + b) * nF;
    for (int e = tid; e < nF; e += nthreads) out[e] = acc[e];
}

// ---- register-resident backward ------------------------------------------------------------
// diagonal triples in the fused layer backward: of the NK reduction steps of four rows the vector waves take the
// first CGNET_DIAG_C0(NK), the matrix waves the others (rounding up instead of down measured the same)
#ifndef CGNET_DIAG_C0
#define CGNET_DIAG_C0(NK_) ((NK_) / 2)
#endif
struct BwdGeom {
    int l, l1, l2, rows, tau2;
    int nr1;      // slot 1: how many of the tau2 reduced channels this call takes (the first nr1)
};

// Item -> (window of two m, first output channel).  Windows are numbered from the middle of the m
// axis outwards and the channel groups of one window are neighbours, so the lanes of a wave have
// similar numbers of terms and the waves with the short (outer) windows finish early.
__device__ __forceinline__ void bwd_item(int item, int nT, int nWin, int& w, int& to) {
    const int widx = item / nT;
    to = item - widx * nT;
    const int c = (nWin - 1) >> 1;
    w = (widx & 1) ? c + ((widx + 1) >> 1) : c - (widx >> 1);
}
constexpr int kBwdMaxTI = 4;   // output channels per thread

// Adds one task's contribution to the calling thread's accumulators.  Same arithmetic and item
// layout as bwd_phase, one item per thread (rtid = thread index inside its role), no reduction.
// g: the tile exactly as it lies in gFF ([t1][t2][m], no padding); cgp: the table with kTabLo /
// kTabHi zero rows; fr: fragment rows of the reduced slot with one trailing zero each.
template <int SLOT, int TI, int RW, int RM = 1>
__device__ __forceinline__ void bwd_accum(const BwdGeom& q, const float* __restrict__ cgp,
                                          const float2* __restrict__ g, const float2* __restrict__ fr,
                                          int rtid, float (&ax)[kBwdMaxTI][2], float (&ay)[kBwdMaxTI][2]) {
    const int l = q.l, l1 = q.l1, l2 = q.l2;
    const int M = 2 * l + 1, M1 = 2 * l1 + 1, M2 = 2 * l2 + 1;
    const int rows = q.rows, tau2 = q.tau2;
    const int n_o = (SLOT == 1) ? rows : tau2;
    const int n_r = (SLOT == 1) ? q.nr1 : rows;
    const int M_o = (SLOT == 1) ? M1 : M2, M_r = (SLOT == 1) ? M2 : M1;
    const int g_so = (SLOT == 1) ? tau2 * M : M;
    const int g_sr = (SLOT == 1) ? M : tau2 * M;
    const int d = l1 + l2 - l;
    // the RW lanes of an item: RM of them split the reduced m range (the first takes an even number of steps, so
    // that its two-step loop ends exactly where the second begins), RW / RM split the reduced channels
    constexpr int RC = RW / RM;
    static_assert(RM == 1 || (RM == 2 && RW % 2 == 0), "the reduced m range is split in two at most");
    const int item = rtid / RW, lane_r = (rtid % RW) % RC, lane_m = (rtid % RW) / RC;
    const int nT = (n_o + TI - 1) / TI;
    const int nWin = (M_o + 1) >> 1;
    if (item >= nT * nWin) return;
    int w, to;
    bwd_item(item, nT, nWin, w, to);
    const int mo0 = 2 * w;
    int ir_lo = max(0, d - mo0 - 1);
    int ir_hi = min(M_r - 1, M - 1 + d - mo0);
    if (RM == 2) {
        const int first = (((ir_hi - ir_lo + 1) >> 1) + 1) & ~1;      // about half, even
        if (lane_m == 0) ir_hi = min(ir_hi, ir_lo + first - 1);
        else ir_lo = ir_lo + first;
    }
    int go[TI];
#pragma unroll
    for (int i = 0; i < TI; ++i) go[i] = min(to + nT * i, n_o - 1) * g_so;
    const int col0 = min(mo0, M2 - 1), col1 = min(mo0 + 1, M2 - 1);
    // Per-lane LDS byte addresses, advanced by constants inside the loop.  Coefficients of the
    // step pair (ir, ir+1):  c0 = T[p][k0], c1 = T[p+1][k1], c0' = T[p+1][k0'], c1' = T[p+2][k1']
    // with p the table row of (mo0, ir); slot 1: k = ir (k0' = k1' = ir+1), slot 2: k0 = col0, k1 = col1.
    const unsigned c_step = (SLOT == 1) ? 8u * (M2 + 1) : 8u * M2;     // two rows (and two columns) per pair
    for (int r = lane_r; r < n_r; r += RC) {
        unsigned gp[TI];
#pragma unroll
        for (int i = 0; i < TI; ++i) gp[i] = lds_addr(g + r * g_sr + (mo0 - d) + go[i] + ir_lo);
        unsigned fp = lds_addr(fr + r * (M_r + 1) + ir_lo);           // rows carry one trailing zero
        const float* cb = cgp + (kTabLo + mo0 - d + ir_lo) * M2;       // table row of (mo0, ir_lo)
        unsigned ca = lds_addr(cb + ((SLOT == 1) ? ir_lo : col0));     // c0
        unsigned cbn = lds_addr(cb + M2 + ((SLOT == 1) ? ir_lo : col1));   // c1 (slot 1: c0' is the next float)
        unsigned cc = lds_addr(cb + 2 * M2 + ((SLOT == 1) ? ir_lo + 1 : col1));  // c1'
        unsigned cd = lds_addr(cb + M2 + col0);                        // slot 2: c0'
        const unsigned f_end = fp + 8u * (unsigned)(ir_hi - ir_lo);
        const bool any = ir_hi >= ir_lo;
#pragma unroll
        for (int i = 0; i < TI; ++i) gp[i] = opaque(gp[i]);
        fp = opaque(fp); ca = opaque(ca); cbn = opaque(cbn); cc = opaque(cc);
        if (SLOT == 2) cd = opaque(cd);
        float2 e0[TI], e1[TI];
#pragma unroll
        for (int i = 0; i < TI; ++i) e0[i] = lds_c(gp[i], 0);
        if (any) {
#pragma unroll 2
            for (; fp <= f_end; ) {
                float2 e2[TI];
#pragma unroll
                for (int i = 0; i < TI; ++i) { e1[i] = lds_c(gp[i], 1); e2[i] = lds_c(gp[i], 2); }
                const float2 fa = lds_c(fp, 0), fb = lds_c(fp, 1);
                const float c0 = lds_f(ca)[0];
                const float c1 = lds_f(cbn)[0];
                const float d0 = (SLOT == 1) ? lds_f(cbn)[1] : lds_f(cd)[0];
                const float d1 = lds_f(cc)[0];
                {
                    const float c0x = c0 * fa.x, c0y = -c0 * fa.y, c1x = c1 * fa.x, c1y = -c1 * fa.y;
#pragma unroll
                    for (int i = 0; i < TI; ++i) {
                        ax[i][0] = fmaf(e0[i].x, c0x, ax[i][0]);
                        ax[i][0] = fmaf(-e0[i].y, c0y, ax[i][0]);
                        ay[i][0] = fmaf(e0[i].x, c0y, ay[i][0]);
                        ay[i][0] = fmaf(e0[i].y, c0x, ay[i][0]);
                        ax[i][1] = fmaf(e1[i].x, c1x, ax[i][1]);
                        ax[i][1] = fmaf(-e1[i].y, c1y, ax[i][1]);
                        ay[i][1] = fmaf(e1[i].x, c1y, ay[i][1]);
                        ay[i][1] = fmaf(e1[i].y, c1x, ay[i][1]);
                    }
                }
                {
                    // past the valid range either the fragment (padded row) or the table row
                    // (padded) is zero, so no masking is needed
                    const float c0x = d0 * fb.x, c0y = -d0 * fb.y, c1x = d1 * fb.x, c1y = -d1 * fb.y;
#pragma unroll
                    for (int i = 0; i < TI; ++i) {
                        ax[i][0] = fmaf(e1[i].x, c0x, ax[i][0]);
                        ax[i][0] = fmaf(-e1[i].y, c0y, ax[i][0]);
                        ay[i][0] = fmaf(e1[i].x, c0y, ay[i][0]);
                        ay[i][0] = fmaf(e1[i].y, c0x, ay[i][0]);
                        ax[i][1] = fmaf(e2[i].x, c1x, ax[i][1]);
                        ax[i][1] = fmaf(-e2[i].y, c1y, ax[i][1]);
                        ay[i][1] = fmaf(e2[i].x, c1y, ay[i][1]);
                        ay[i][1] = fmaf(e2[i].y, c1x, ay[i][1]);
                    }
                }
#pragma unroll
                for (int i = 0; i < TI; ++i) { e0[i] = e2[i]; gp[i] += 16u; }
                fp += 16u;
                ca += c_step; cbn += c_step; cc += c_step;
                if (SLOT == 2) cd += c_step;
            }
        }
    }
}

// Adds up the RW lanes of every item (all lanes of the wave take part) and stores the slab
// dst[n_o][M_o]; every element of the slab has exactly one owner.  Clears the accumulators.
template <int TI, int RW>
__device__ __forceinline__ void bwd_flush(int n_o, int M_o, int rtid, float (&ax)[kBwdMaxTI][2],
                                          float (&ay)[kBwdMaxTI][2], float2* __restrict__ dst) {
#pragma unroll
    for (int i = 0; i < TI; ++i) {
        ax[i][0] = row_sum<RW>(ax[i][0]);
        ay[i][0] = row_sum<RW>(ay[i][0]);
        ax[i][1] = row_sum<RW>(ax[i][1]);
        ay[i][1] = row_sum<RW>(ay[i][1]);
    }
    const int item = rtid / RW, lane_r = rtid % RW;
    const int nT = (n_o + TI - 1) / TI;
    const int nWin = (M_o + 1) >> 1;
    if (item < nT * nWin) {
        int w, to;
        bwd_item(item, nT, nWin, w, to);
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            const int mo = 2 * w + k;
            if (lane_r == (k % RW) && mo < M_o) {
#pragma unroll
                for (int i = 0; i < TI; ++i) {
                    const int ch = to + nT * i;
                    if (ch < n_o) dst[ch * M_o + mo] = make_float2(ax[i][k], ay[i][k]);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kBwdMaxTI; ++i) ax[i][0] = ax[i][1] = ay[i][0] = ay[i][1] = 0.f;
}

#define CGNET_BWD_SWITCH(TI_, RW_, CALL)                                         \
    switch ((TI_) * 32 + (RW_)) {                                                \
        case 1 * 32 + 1: { CALL(1, 1); } break;                                  \
        case 1 * 32 + 2: { CALL(1, 2); } break;                                  \
        case 1 * 32 + 4: { CALL(1, 4); } break;                                  \
        case 1 * 32 + 8: { CALL(1, 8); } break;                                  \
        case 1 * 32 + 16: { CALL(1, 16); } break;                                \
        case 2 * 32 + 1: { CALL(2, 1); } break;                                  \
        case 2 * 32 + 2: { CALL(2, 2); } break;                                  \
        case 2 * 32 + 4: { CALL(2, 4); } break;                                  \
        case 2 * 32 + 8: { CALL(2, 8); } break;                                  \
        case 2 * 32 + 16: { CALL(2, 16); } break;                                \
        case 3 * 32 + 1: { CALL(3, 1); } break;                                  \
        case 3 * 32 + 2: { CALL(3, 2); } break;                                  \
        case 3 * 32 + 4: { CALL(3, 4); } break;                                  \
        case 3 * 32 + 8: { CALL(3, 8); } break;                                  \
        case 3 * 32 + 16: { CALL(3, 16); } break;                                \
        case 4 * 32 + 1: { CALL(4, 1); } break;                                  \
        case 4 * 32 + 2: { CALL(4, 2); } break;                                  \
        case 4 * 32 + 4: { CALL(4, 4); } break;                                  \
        case 4 * 32 + 8: { CALL(4, 8); } break;                                  \
        default: { CALL(4, 16); } break;                                         \
    }

// slot-1 tilings: as above, plus the variants whose lanes also split the reduced m range in two
#define CGNET_BWD_SWITCH_A(TI_, RW_, RM_, CALL)                                  \
    if ((RM_) == 2) {                                                            \
        switch ((TI_) * 32 + (RW_)) {                                            \
            case 2 * 32 + 4: { CALL(2, 4, 2); } break;                           \
            case 2 * 32 + 8: { CALL(2, 8, 2); } break;                           \
            case 2 * 32 + 16: { CALL(2, 16, 2); } break;                         \
            case 3 * 32 + 4: { CALL(3, 4, 2); } break;                           \
            case 3 * 32 + 8: { CALL(3, 8, 2); } break;                           \
            case 3 * 32 + 16: { CALL(3, 16, 2); } break;                         \
            case 4 * 32 + 4: { CALL(4, 4, 2); } break;                           \
            case 4 * 32 + 8: { CALL(4, 8, 2); } break;                           \
            default: { CALL(4, 16, 2); } break;                                  \
        }                                                                        \
    } else {                                                                     \
        switch ((TI_) * 32 + (RW_)) {                                            \
            case 1 * 32 + 1: { CALL(1, 1, 1); } break;                           \
            case 1 * 32 + 2: { CALL(1, 2, 1); } break;                           \
            case 1 * 32 + 4: { CALL(1, 4, 1); } break;                           \
            case 1 * 32 + 8: { CALL(1, 8, 1); } break;                           \
            case 1 * 32 + 16: { CALL(1, 16, 1); } break;                         \
            case 2 * 32 + 1: { CALL(2, 1, 1); } break;                           \
            case 2 * 32 + 2: { CALL(2, 2, 1); } break;                           \
            case 2 * 32 + 4: { CALL(2, 4, 1); } break;                           \
            case 2 * 32 + 8: { CALL(2, 8, 1); } break;                           \
            case 2 * 32 + 16: { CALL(2, 16, 1); } break;                         \
            case 3 * 32 + 1: { CALL(3, 1, 1); } break;                           \
            case 3 * 32 + 2: { CALL(3, 2, 1); } break;                           \
            case 3 * 32 + 4: { CALL(3, 4, 1); } break;                           \
            case 3 * 32 + 8: { CALL(3, 8, 1); } break;                           \
            case 3 * 32 + 16: { CALL(3, 16, 1); } break;                         \
            case 4 * 32 + 1: { CALL(4, 1, 1); } break;                           \
            case 4 * 32 + 2: { CALL(4, 2, 1); } break;                           \
            case 4 * 32 + 4: { CALL(4, 4, 1); } break;                           \
            case 4 * 32 + 8: { CALL(4, 8, 1); } break;                           \
            default: { CALL(4, 16, 1); } break;                                  \
        }                                                                        \
    }

// slot-1 tilings of the hybrid kernel: at most two output rows per thread (64 registers)
#define CGNET_BWD_SWITCH_A2(TI_, RW_, RM_, CALL)                                 \
    if ((RM_) == 2) {                                                            \
        switch ((TI_) * 32 + (RW_)) {                                            \
            case 2 * 32 + 4: { CALL(2, 4, 2); } break;                           \
            case 2 * 32 + 8: { CALL(2, 8, 2); } break;                           \
            default: { CALL(2, 16, 2); } break;                                  \
        }                                                                        \
    } else {                                                                     \
        switch ((TI_) * 32 + (RW_)) {                                            \
            case 1 * 32 + 1: { CALL(1, 1, 1); } break;                           \
            case 1 * 32 + 2: { CALL(1, 2, 1); } break;                           \
            case 1 * 32 + 4: { CALL(1, 4, 1); } break;                           \
            case 1 * 32 + 8: { CALL(1, 8, 1); } break;                           \
            case 1 * 32 + 16: { CALL(1, 16, 1); } break;                         \
            case 2 * 32 + 1: { CALL(2, 1, 1); } break;                           \
            case 2 * 32 + 2: { CALL(2, 2, 1); } break;                           \
            case 2 * 32 + 4: { CALL(2, 4, 1); } break;                           \
            case 2 * 32 + 8: { CALL(2, 8, 1); } break;                           \
            default: { CALL(2, 16, 1); } break;                                  \
        }                                                                        \
    }

// ... at most three output rows per thread (80 registers)
#define CGNET_BWD_SWITCH_A3(TI_, RW_, RM_, CALL)                                 \
    if ((TI_) == 3) {                                                            \
        if ((RM_) == 2) {                                                        \
            switch (RW_) {                                                       \
                case 4: { CALL(3, 4, 2); } break;                                \
                case 8: { CALL(3, 8, 2); } break;                                \
                default: { CALL(3, 16, 2); } break;                              \
            }                                                                    \
        } else {                                                                 \
            switch (RW_) {                                                       \
                case 1: { CALL(3, 1, 1); } break;                                \
                case 2: { CALL(3, 2, 1); } break;                                \
                case 4: { CALL(3, 4, 1); } break;                                \
                case 8: { CALL(3, 8, 1); } break;                                \
                default: { CALL(3, 16, 1); } break;                              \
            }                                                                    \
        }                                                                        \
    } else {                                                                     \
        CGNET_BWD_SWITCH_A2(TI_, RW_, RM_, CALL)                                 \
    }

struct BwdCtx {
    const float2* Fp;          // this sample's fragments, rows padded with one zero
    const float2* Gb;          // this sample's gFF
    const float* CGP;          // zero-padded tables of all triples
    const BwdUTask* tasks;
    float2* f1;                // LDS: rows x (M1+1) slab of degree l1 (fixed for the unit)
    char* f2;                  // LDS: two slabs of degree l2 (current run / next run), f2cap bytes each
    char* cg;                  // LDS: two tables, cgcap bytes each
    char* tile;                // LDS: the tile buffers (two, or one in the hybrid kernel), tcap + 16 bytes each
    int f2cap, cgcap, tcap;
    int tid, rtid;
};

// Starts the copy of task t's tile into tile buffer `buf`.
template <int NT>
__device__ __forceinline__ void bwd_issue_tile(const BwdCtx& c, const BwdUnit& u, const BwdUTask& t, int buf) {
    const int ntile = u.rows * t.tau2 * (2 * t.l + 1);
    char* tile = c.tile + buf * (c.tcap + 16);
    dma16<NT>(c.Gb + t.offFF, tile, ntile >> 1, c.tid);
    if (ntile & 1) dma8(c.Gb + t.offFF + (ntile - 1), tile + 8 * (size_t)(ntile - 1), c.tid);
}

// Starts the copies of task t: table into buffer `par`, the l2 slab (first task of a run only) into slab buffer
// `f2par`, and with two tile buffers (TWO) the tile into buffer `par`.
template <int NT, bool TWO>
__device__ __forceinline__ void bwd_issue(const BwdCtx& c, const BwdUnit& u, const BwdUTask& t, int par, int f2par) {
    const int M2 = 2 * t.l2 + 1;
    if (TWO) bwd_issue_tile<NT>(c, u, t, par);
    dma16<NT>(c.CGP + t.cgp_off, c.cg + par * c.cgcap, t.cgp_len >> 2, c.tid);
    if (t.first_of_l2) dma16<NT>(c.Fp + t.offF2p, c.f2 + f2par * c.f2cap, (t.tau2 * (M2 + 1)) >> 1, c.tid);
}

// Per-task prologue of both roles.  On entry `t` is the task whose copies were started one
// task earlier into buffer `par`; on exit they are visible, `cur` holds that task and the
// copies of the following task are in flight.  One barrier per task, executed by every thread.
// With one tile buffer (TWO = false) the following task's tile is not among those copies: bwd_stage_end starts it
// when every wave has finished with the current tile (a second barrier per task).
template <int NT, bool TWO>
__device__ __forceinline__ void bwd_stage(const BwdCtx& c, const BwdUnit& u, int ti, BwdUTask& t, BwdUTask& cur,
                                          int& par, int& f2par, const float*& cgp, const float2*& g,
                                          const float2*& f2) {
    dma_wait();
    __syncthreads();           // copies of every wave landed; nobody still reads the other buffers
    cur = t;
    cgp = reinterpret_cast<const float*>(c.cg + par * c.cgcap);
    g = reinterpret_cast<const float2*>(c.tile + (TWO ? par : 0) * (c.tcap + 16));
    f2 = reinterpret_cast<const float2*>(c.f2 + f2par * c.f2cap);
    par ^= 1;
    if (ti + 1 < u.task_end) {
        t = c.tasks[ti + 1];
        if (t.first_of_l2) f2par ^= 1;
        bwd_issue<NT, TWO>(c, u, t, par, f2par);
    }
}

// Per-task epilogue of both roles with one tile buffer; `t` is the following task (as bwd_stage left it).
template <int NT, bool TWO>
__device__ __forceinline__ void bwd_stage_end(const BwdCtx& c, const BwdUnit& u, int ti, const BwdUTask& t) {
    if (TWO) return;
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");     // every wave's reads of the tile are complete
    if (ti + 1 < u.task_end) bwd_issue_tile<NT>(c, u, t, 0);
}

// Waves of role A: gradient of slot 1 (rows of degree l1), kept in registers for the whole unit.
template <int NT, bool TWO, int TI, int RW, int RM>
__device__ __forceinline__ void bwd_unit_loop_a(const BwdCtx& c, const BwdUnit& u, BwdUTask t,
                                                float2* __restrict__ dst) {
    float ax[kBwdMaxTI][2], ay[kBwdMaxTI][2], tx[kBwdMaxTI][2], ty[kBwdMaxTI][2];
#pragma unroll
    for (int i = 0; i < kBwdMaxTI; ++i) {
        ax[i][0] = ax[i][1] = ay[i][0] = ay[i][1] = 0.f;
        tx[i][0] = tx[i][1] = ty[i][0] = ty[i][1] = 0.f;
    }
    int par = 0, f2par = 0;
    for (int ti = u.task_begin; ti < u.task_end; ++ti) {
        BwdUTask cur;
        const float* cgp;
        const float2 *g, *f2;
        bwd_stage<NT, TWO>(c, u, ti, t, cur, par, f2par, cgp, g, f2);
        const BwdGeom q{cur.l, u.l1, cur.l2, u.rows, cur.tau2, cur.tau2};
        bwd_accum<1, TI, RW, RM>(q, cgp, g, f2, c.rtid, ax, ay);
        bwd_stage_end<NT, TWO>(c, u, ti, t);
        if (cur.last_of_l2) {
            // blocked summation: the running sum of one l2 is folded into the unit's total
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    tx[i][k] += ax[i][k];
                    ty[i][k] += ay[i][k];
                    ax[i][k] = ay[i][k] = 0.f;
                }
        }
    }
    bwd_flush<TI, RW>(u.rows, 2 * u.l1 + 1, c.rtid, tx, ty, dst);
}

// Waves of role B: gradient of slot 2, kept in registers across the tasks that share l2.
__device__ __forceinline__ void bwd_unit_loop_b(const BwdCtx& c, const BwdUnit& u, BwdUTask t,
                                                float2* __restrict__ part2_b) {
    float ax[kBwdMaxTI][2], ay[kBwdMaxTI][2];
#pragma unroll
    for (int i = 0; i < kBwdMaxTI; ++i) ax[i][0] = ax[i][1] = ay[i][0] = ay[i][1] = 0.f;
    int par = 0, f2par = 0;
    for (int ti = u.task_begin; ti < u.task_end; ++ti) {
        BwdUTask cur;
        const float* cgp;
        const float2 *g, *f2;
        bwd_stage<kThreads, true>(c, u, ti, t, cur, par, f2par, cgp, g, f2);
        const BwdGeom q{cur.l, u.l1, cur.l2, u.rows, cur.tau2, cur.tau2};
#define CGNET_CALL_B(TI_, RW_) bwd_accum<2, TI_, RW_>(q, cgp, g, c.f1, c.rtid, ax, ay)
        CGNET_BWD_SWITCH(cur.TI, cur.RW, CGNET_CALL_B)
#undef CGNET_CALL_B
        if (cur.last_of_l2) {
            float2* dst = part2_b + cur.p2off;
#define CGNET_FLUSH_B(TI_, RW_) bwd_flush<TI_, RW_>(cur.tau2, 2 * cur.l2 + 1, c.rtid, ax, ay, dst)
            CGNET_BWD_SWITCH(cur.TI, cur.RW, CGNET_FLUSH_B)
#undef CGNET_FLUSH_B
        }
    }
}

// LDS map (bytes): [16 zero] f1 (f1cap) | f2 x2 (f2cap each) | table x2 (cgcap each) | [16 zero]
// tile 0 (tcap) [16 zero] tile 1 (tcap) [16 zero]; the hybrid kernel has tile 0 only.  Everything is cleared
// once, so positions a tile read may touch just outside the tile hold finite values.
__host__ __device__ inline size_t bwd_unit_lds(int f1cap, int f2cap, int cgcap, int tcap, int ntiles = 2) {
    return 16 + (size_t)f1cap + 2 * (size_t)f2cap + 2 * (size_t)cgcap + 16 + ntiles * ((size_t)tcap + 16);
}

__global__ void __launch_bounds__(kThreads, 4)
cg_backward_unit_kernel(const float2* __restrict__ Fp, const float2* __restrict__ gFF,
                        const float* __restrict__ CGP, float2* __restrict__ part1, float2* __restrict__ part2,
                        const BwdUnit* __restrict__ units, const BwdUTask* __restrict__ tasks,
                        int nF, int nFp, int nFF, int P2, int f1cap, int f2cap, int cgcap, int tcap, int B) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = unit_major(B);
    const BwdUnit u = units[up.unit];
    const int b = up.part;
    const int tid = threadIdx.x, wave = tid >> 6;
    const int M1 = 2 * u.l1 + 1;
    const bool roleA = wave < u.nA;                  // wave-uniform
    BwdCtx c;
    c.Fp = Fp + (size_t)b * nFp;
    c.Gb = gFF + (size_t)b * nFF;
    c.CGP = CGP;
    c.tasks = tasks;
    c.f1 = reinterpret_cast<float2*>(smem + 16);
    c.f2 = reinterpret_cast<char*>(smem) + 16 + f1cap;
    c.cg = c.f2 + 2 * f2cap;
    c.tile = c.cg + 2 * cgcap + 16;
    c.f2cap = f2cap; c.cgcap = cgcap; c.tcap = tcap;
    c.tid = tid;
    c.rtid = roleA ? tid : tid - 64 * u.nA;

    {
        const int n16 = (int)(bwd_unit_lds(f1cap, f2cap, cgcap, tcap) >> 4);
        float4* z = reinterpret_cast<float4*>(smem);
        for (int e = tid; e < n16; e += kThreads) z[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();                                 // the clearing stores precede every copy
    const BwdUTask t0 = tasks[u.task_begin];
    dma16<kThreads>(c.Fp + u.offF1p, c.f1, (u.rows * (M1 + 1)) >> 1, tid);
    bwd_issue<kThreads, true>(c, u, t0, 0, 0);

    // The two roles run the same sequence of barriers (one per task) from different code paths.
    if (roleA) {
        float2* dst = u.p1off < 0 ? part1 + (size_t)b * nF + u.offF1 : part2 + (size_t)b * P2 + u.p1off;
#define CGNET_LOOP_A(TI_, RW_, RM_) bwd_unit_loop_a<kThreads, true, TI_, RW_, RM_>(c, u, t0, dst)
        CGNET_BWD_SWITCH_A(u.TI, u.RW, u.RM, CGNET_LOOP_A)
#undef CGNET_LOOP_A
    } else {
        bwd_unit_loop_b(c, u, t0, part2 + (size_t)b * P2);
    }
}

// ---- unit backward, slot 2 on the matrix cores ----------------------------------------------
// For a fixed m of the tile, G_m = gFF[t1, t2, m] is a rows x tau2 complex matrix and
//   gF2[t2, m2] += sum_t1 G_m[t1, t2] * (C[m][m2] conj F1[t1][m - m2])       (tau2 x rows)(rows x window of m2)
// is a small matrix product: rows of the accumulator = the up to 16 channels of degree l2, columns
// = up to three tiles of 16 values of m2, reduction over the up to 16 rows of the unit in steps of 4.
// Work-groups of eight waves: the first nA keep the slot-1 gradient on the vector ALUs exactly as in
// cg_backward_unit_kernel, the others take slot 2 here, each every (8 - nA)-th m.  A matrix instruction costs
// the SIMD fewer issue cycles per useful product than the vector route does (the two kinds take turns on a SIMD,
// they do not run side by side), so the vector ALUs carry about half the arithmetic.  The partial slot-2 gradients
// of the matrix waves leave as separate slabs; cg_backward_combine_kernel adds them.  The kernel keeps one tile
// buffer and few registers, so that three or four work-groups share a compute unit: its waves wait for LDS reads
// and for each other (two barriers per task), and it is other work-groups that fill those waits.
constexpr int kHybThreads = 512;
constexpr int kHybWaves = 8;        // the first BwdUnit::nA of them take slot 1, the others (= partial slabs per
                                    // slot-2 gradient) slot 2 on the matrix cores
constexpr int kHybMaxRows = 16;     // reduction steps: at most 4 x 4 rows
constexpr int kHybMaxTI = 3;        // slot 1: output rows per thread (two where four groups share a compute unit)
constexpr int kHybMaxTiles = 3;     // 16-column tiles of the m2 axis: degrees up to 23
// Plan: weight of a vector-ALU step of slot 1 against the matrix-core cost of slot 2 in the same
// work-group.  Measured, not derived: below one because the matrix waves also wait on their operand
// loads, so a unit is better off with one vector wave fewer than the instruction counts suggest.
constexpr double kHybSlot1Scale = 0.6;

// x mod n for 0 <= x < 2^20, n < 2^10 (wave-uniform; inv = 1 / n)
__device__ __forceinline__ int small_mod(int x, int n, float inv) {
    int r = x - (int)(((float)x + 0.5f) * inv) * n;
    if (r < 0) r += n;
    if (r >= n) r -= n;
    return r;
}

// NK = reduction steps of four rows; KFULL: the rows fill every step.  One loop per 16-column tile of the m2 axis,
// over the m indices (of those congruent to `part` modulo `split`) at which one of the tile's columns has a valid
// m1 = m - m2: a tile outside the window of an m costs nothing, and no branch joins paths that hold the accumulators
// in different registers (there the compiler copied them, and every copy waits for the matrix pipeline to drain).
// All addresses are explicit LDS byte addresses advanced by constants from one m to the next.  The table holds zeros
// where m - m2 is no valid m1 (every table this library fills does), so only the columns past the end of the m2
// axis are masked; the fragment column of such an entry is clamped into its row and multiplied by that zero.
// C0: the reduction skips its first C0 steps (rows below 4 * C0 belong to somebody else: diagonal triples, below).
template <int NK, bool KFULL, int C0 = 0>
__device__ __forceinline__ void bwd_mm_task(const BwdGeom& q, const float* __restrict__ cgp,
                                            const float2* __restrict__ g, const float2* __restrict__ f1, int part,
                                            int split, float inv_split, int lane, f32x4 (&dre)[kHybMaxTiles],
                                            f32x4 (&dim)[kHybMaxTiles]) {
    const int l = q.l, l1 = q.l1, l2 = q.l2;
    const int M = 2 * l + 1, M1 = 2 * l1 + 1, M2 = 2 * l2 + 1;
    const int rows = q.rows, tau2 = q.tau2;
    const int i = lane & 15, kk = lane >> 4;
    const int io = min(i, tau2 - 1);                              // rows past the last channel repeat it (never stored)
    const int d = l1 + l2 - l;
    // per reduction step: LDS address of the lane's tile entry at m index 0, base of its fragment row; rows past
    // the end of the unit repeat the last one and get a zero coefficient
    unsigned gbase[NK], fbase[NK];
    float kmask[NK];
#pragma unroll
    for (int c = 0; c < NK; ++c) {
        const int k = 4 * c + kk;
        const int kc = min(k, rows - 1);
        kmask[c] = k < rows ? 1.f : 0.f;
        gbase[c] = lds_addr(g + (kc * tau2 + io) * M);
        fbase[c] = lds_addr(f1 + kc * (M1 + 1));
    }
    const int nt = (M2 + 15) >> 4;
    const unsigned gstep = 8u * (unsigned)split, cstep = 4u * (unsigned)(split * M2);
#pragma unroll
    for (int t = 0; t < kHybMaxTiles; ++t) {
        const int col = 16 * t + i;
        const int colc = min(col, M2 - 1);
        const bool colok = col < M2;
        // column c of the m2 axis is valid at m index mi iff mi - l - (c - l2) lies in [-l1, l1]
        const int lo = max(0, 16 * t - d);
        const int hi = t < nt ? min(M - 1, 16 * t + 15 - d + 2 * l1) : -1;
        const int mi0 = lo + small_mod(part - lo + 1024 * split, split, inv_split);
        unsigned ga[NK];
#pragma unroll
        for (int c = 0; c < NK; ++c) ga[c] = opaque(gbase[c] + 8u * (unsigned)mi0);
        unsigned ca = opaque(lds_addr(cgp + (kTabLo + mi0) * M2 + colc));
        int fc = mi0 - l - (colc - l2) + l1;                      // fragment column of slot 1 = m - m2 + l1
        for (int mi = mi0; mi <= hi; mi += split) {
            float2 gq[NK], fq[NK];
            const float cc = lds_f(ca)[0];
            ca += cstep;
            const int fcol = max(0, min(M1 - 1, fc));             // clamped where the coefficient is zero anyway
            fc += split;
#pragma unroll
            for (int c = C0; c < NK; ++c) {
                gq[c] = lds_c(ga[c], 0);
                ga[c] += gstep;
                fq[c] = lds_c(fbase[c] + 8u * (unsigned)fcol, 0);
            }
            const float cv = colok ? cc : 0.f;
#pragma unroll
            for (int c = C0; c < NK; ++c) {
                const float w = KFULL ? cv : cv * kmask[c];
                const float bx = w * fq[c].x, by = -w * fq[c].y;  // C conj(f)
                const float ngy = -gq[c].y;
                dre[t] = mfma4(gq[c].x, bx, dre[t]);
                dim[t] = mfma4(gq[c].x, by, dim[t]);
                dre[t] = mfma4(ngy, by, dre[t]);
                dim[t] = mfma4(gq[c].y, bx, dim[t]);
            }
        }
    }
}

// Stores the wave's accumulator tiles: rows = channels, columns of an m axis of length Mo.
__device__ __forceinline__ void bwd_mm_store(const f32x4 (&dre)[kHybMaxTiles], const f32x4 (&dim)[kHybMaxTiles], int n_out, int Mo, int lane,
                                             float2* __restrict__ dst) {
    const int j = lane & 15, kk = lane >> 4;
#pragma unroll
    for (int tile = 0; tile < kHybMaxTiles; ++tile) {
        const int col = 16 * tile + j;
        if (col < Mo) {
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int ch = 4 * kk + v;
                if (ch < n_out) dst[ch * Mo + col] = make_float2(dre[tile][v], dim[tile][v]);
            }
        }
    }
}

template <int NK, bool KFULL>
__device__ __forceinline__ void bwd_hybrid_loop_b(const BwdCtx& c, const BwdUnit& u, BwdUTask t, int part, int split,
                                                  int lane, float2* __restrict__ part2_b) {
    f32x4 dre[kHybMaxTiles], dim[kHybMaxTiles];
#pragma unroll
    for (int k = 0; k < kHybMaxTiles; ++k) dre[k] = dim[k] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const float inv_split = 1.0f / (float)split;
    int par = 0, f2par = 0;
    for (int ti = u.task_begin; ti < u.task_end; ++ti) {
        BwdUTask cur;
        const float* cgp;
        const float2 *g, *f2;
        bwd_stage<kHybThreads, false>(c, u, ti, t, cur, par, f2par, cgp, g, f2);
        const BwdGeom q{cur.l, u.l1, cur.l2, u.rows, cur.tau2, cur.tau2};
        bwd_mm_task<NK, KFULL>(q, cgp, g, c.f1, part, split, inv_split, lane, dre, dim);
        bwd_stage_end<kHybThreads, false>(c, u, ti, t);
        if (cur.last_of_l2) {
            const int M2 = 2 * cur.l2 + 1;
            bwd_mm_store(dre, dim, cur.tau2, M2, lane, part2_b + cur.p2off + (size_t)part * cur.tau2 * M2);
#pragma unroll
            for (int k = 0; k < kHybMaxTiles; ++k) dre[k] = dim[k] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
    }
}

// the matrix-core role for a unit of `rows` rows: reduction steps and whether the rows fill them are fixed per unit
#define CGNET_HYB_ROLE_B(ROWS_, CALL)                                    \
    switch ((((ROWS_) + 3) >> 2) * 2 + (((ROWS_) & 3) ? 0 : 1)) {        \
        case 2: { CALL(1, false); } break;                               \
        case 3: { CALL(1, true); } break;                                \
        case 4: { CALL(2, false); } break;                               \
        case 5: { CALL(2, true); } break;                                \
        case 6: { CALL(3, false); } break;                               \
        case 7: { CALL(3, true); } break;                                \
        case 8: { CALL(4, false); } break;                               \
        default: { CALL(4, true); } break;                               \
    }

// G4: 64 registers and at most two output rows per slot-1 thread, so that four work-groups share a compute unit;
// otherwise 80 registers, three rows, three work-groups (shapes whose tiles would shrink below four rows with four).
template <bool G4>
__global__ void __launch_bounds__(kHybThreads, G4 ? 8 : 6)
cg_backward_hybrid_kernel(const float2* __restrict__ Fp, const float2* __restrict__ gFF,
                          const float* __restrict__ CGP, float2* __restrict__ part1, float2* __restrict__ part2,
                          const BwdUnit* __restrict__ units, const BwdUTask* __restrict__ tasks,
                          int nF, int nFp, int nFF, int P2, int f1cap, int f2cap, int cgcap, int tcap, int B) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = unit_major(B);
    const BwdUnit u = units[up.unit];
    const int b = up.part;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M1 = 2 * u.l1 + 1;
    const bool roleA = wave < u.nA;                  // wave-uniform
    BwdCtx c;
    c.Fp = Fp + (size_t)b * nFp;
    c.Gb = gFF + (size_t)b * nFF;
    c.CGP = CGP;
    c.tasks = tasks;
    c.f1 = reinterpret_cast<float2*>(smem + 16);
    c.f2 = reinterpret_cast<char*>(smem) + 16 + f1cap;
    c.cg = c.f2 + 2 * f2cap;
    c.tile = c.cg + 2 * cgcap + 16;
    c.f2cap = f2cap; c.cgcap = cgcap; c.tcap = tcap;
    c.tid = tid;
    c.rtid = tid;                                    // role A: threads 0 .. 64 * nA - 1
    {
        const int n16 = (int)(bwd_unit_lds(f1cap, f2cap, cgcap, tcap, 1) >> 4);
        float4* z = reinterpret_cast<float4*>(smem);
        for (int e = tid; e < n16; e += kHybThreads) z[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();                                 // the clearing stores precede every copy
    const BwdUTask t0 = tasks[u.task_begin];
    dma16<kHybThreads>(c.Fp + u.offF1p, c.f1, (u.rows * (M1 + 1)) >> 1, tid);
    bwd_issue<kHybThreads, false>(c, u, t0, 0, 0);
    bwd_issue_tile<kHybThreads>(c, u, t0, 0);
    // The two roles run the same sequence of barriers (one per task) from different code paths.
    if (roleA) {
        float2* dst = u.p1off < 0 ? part1 + (size_t)b * nF + u.offF1 : part2 + (size_t)b * P2 + u.p1off;
#define CGNET_LOOP_A(TI_, RW_, RM_) bwd_unit_loop_a<kHybThreads, false, TI_, RW_, RM_>(c, u, t0, dst)
        if (G4) {
            CGNET_BWD_SWITCH_A2(u.TI, u.RW, u.RM, CGNET_LOOP_A)
        } else {
            CGNET_BWD_SWITCH_A3(u.TI, u.RW, u.RM, CGNET_LOOP_A)
        }
#undef CGNET_LOOP_A
    } else {
#define CGNET_LOOP_B(NK_, KF_) \
    bwd_hybrid_loop_b<NK_, KF_>(c, u, t0, wave - u.nA, kHybWaves - u.nA, tid & 63, part2 + (size_t)b * P2)
        CGNET_HYB_ROLE_B(u.rows, CGNET_LOOP_B)
#undef CGNET_LOOP_B
    }
}

// ---- the layer's backward in one kernel: gFF tiles made in LDS ------------------------------------
// cg_backward_hybrid_kernel whose work-groups make every task's gFF tile themselves instead of copying it from
// memory:   gFF[c, (m, re/im)] = sum_k A[c][k] B[k][(m, re/im)],  k = (output channel to, re/im),
//   A[c][(to,0)] = W_re[to][c]/div[c], A[c][(to,1)] = W_im[to][c]/div[c]
//   B[(to,0)][(m,0)] = gO_re, B[(to,1)][(m,0)] = gO_im, B[(to,0)][(m,1)] = gO_im, B[(to,1)][(m,1)] = -gO_re
// the arithmetic of wmm_gradff_mfma_kernel, instruction for instruction, so the tile holds the values that kernel
// would have written to memory and the result equals the two-kernel route bit for bit.
//
// Both operands are packed beforehand in the order the lanes of a wave read them (pack_w_gen_kernel: one block per
// task; pack_go_gen_kernel: one block per sample and degree), so that making the tile costs LDS reads and
// matrix instructions but next to no vector-ALU work, which is what the kernel is short of.
//
// A stage (one task) has two phases.  Phase 1: all eight waves make the tile -- it is cut into units of 16 channels
// x 16 real columns (one accumulator each), numbered column-tile major, and every wave takes a contiguous share.
// Phase 2: the tile is used exactly as in the hybrid kernel (slot 1 on the vector ALUs, slot 2 on the matrix
// cores).  The two operands of the next task's tile are copied into LDS during phase 2 (their buffers are only read
// in phase 1); the task's own coefficient table and l2 slab, which only phase 2 reads, are copied during its phase 1.
// Every buffer exists once, which keeps the work-group small enough for three to share a compute unit.  A wave
// learns about the task after the next one through scalar loads that are in flight for a whole stage.

struct FusedCtx {
    const float2* Fp;          // this sample's fragments, rows padded with one zero
    const float* Bg;           // this sample's packed B operand
    const float* Ag;           // packed A operand, one block per task
    const float* CGP;          // zero-padded tables of all triples
    float2* f1;                // LDS: rows x (M1+1) slab of degree l1
    char* f2;                  // LDS: two slabs of degree l2, f2cap bytes each
    char* cg;                  // LDS: two tables, cgcap bytes each
    float* bl;                 // LDS: the task's B operand
    float* al;                 // LDS: the task's A operand
    float* tile;               // LDS: the gFF tile
    int f2cap, cgcap;
    int tid, lane, wave;
};

__device__ __forceinline__ int ft_l(const FusedTask& t) { return t.geom & 255; }
__device__ __forceinline__ int ft_l2(const FusedTask& t) { return (t.geom >> 8) & 255; }
__device__ __forceinline__ int ft_tau2(const FusedTask& t) { return (t.geom >> 16) & 255; }
__device__ __forceinline__ bool ft_first(const FusedTask& t) { return (t.geom >> 24) & 1; }
__device__ __forceinline__ bool ft_last(const FusedTask& t) { return (t.geom >> 25) & 1; }
__device__ __forceinline__ int ft_c0(const FusedTask& t) { return (t.geom >> 26) & 3; }   // diagonal triple: matrix waves skip this many steps
__device__ __forceinline__ int ft_nks(const FusedTask& t) { return t.shape & 255; }
__device__ __forceinline__ int ft_nch(const FusedTask& t) { return t.shape >> 16; }

// Phase 1 of a stage: this wave's share of the tile.  al: the A operand, k-steps in pairs: float2 entry
// [(row tile * NKP + kp) * 64 + lane] = (A of k-step 2kp, A of k-step 2kp+1), NKP = (NKS+1)/2, so that the 64 lanes of
// a read touch 512 contiguous bytes; bl: entry [(column tile * NKS + ks) * 64 + lane].  Columns past 2M and rows
// past the last channel are not stored.
template <int NKS>
__device__ __forceinline__ void gen_phase_nks(int nch, int M, const float* __restrict__ al, const float* __restrict__ bl,
                                              float* __restrict__ tile, int wave, int lane) {
    constexpr int NKP = (NKS + 1) / 2;
    const int i = lane & 15, kk = lane >> 4;
    const int M2f = 2 * M;
    const int nct = (M2f + 15) >> 4, nrt = (nch + 15) >> 4, U = nct * nrt;
    int idx = (wave * U) >> 3;
    const int ue = ((wave + 1) * U) >> 3;
    if (idx >= ue) return;
    int ct = idx / nrt, rt = idx - ct * nrt;
    while (idx < ue) {
        const float* bp = bl + ct * (NKS * 64) + lane;
        float bv[NKS];
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) bv[ks] = bp[64 * ks];
        const int col = 16 * ct + i;
        const bool colok = col < M2f;
        const int rt_end = min(nrt, rt + (ue - idx));
        idx += rt_end - rt;
        for (; rt < rt_end; ++rt) {
            const float2* ap = reinterpret_cast<const float2*>(al) + rt * (NKP * 64) + lane;
            float a[2 * NKP];
#pragma unroll
            for (int kp = 0; kp < NKP; ++kp) {
                const float2 v = ap[64 * kp];
                a[2 * kp] = v.x;
                a[2 * kp + 1] = v.y;
            }
            f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) acc = mfma4(a[ks], bv[ks], acc);
            const int row = 16 * rt + 4 * kk;
            float* dst = tile + row * M2f + col;
            if (16 * rt + 16 <= nch) {               // wave-uniform: a full row tile
                if (colok) {
                    dst[0] = acc[0];
                    dst[M2f] = acc[1];
                    dst[2 * M2f] = acc[2];
                    dst[3 * M2f] = acc[3];
                }
            } else if (colok) {
#pragma unroll
                for (int v = 0; v < 4; ++v)
                    if (row + v < nch) dst[v * M2f] = acc[v];
            }
        }
        rt = 0;
        ++ct;
    }
}

__device__ __forceinline__ void gen_phase(const FusedTask& t, const float* __restrict__ al, const float* __restrict__ bl,
                                          float* __restrict__ tile, int wave, int lane) {
    const int nch = ft_nch(t), M = 2 * ft_l(t) + 1;
    switch (ft_nks(t)) {
        case 0:      // a degree without output channels: its product channels have no gradient
            for (int e = wave * 64 + lane; e < nch * 2 * M; e += kHybThreads) tile[e] = 0.f;
            break;
        case 1: gen_phase_nks<1>(nch, M, al, bl, tile, wave, lane); break;
        case 2: gen_phase_nks<2>(nch, M, al, bl, tile, wave, lane); break;
        case 3: gen_phase_nks<3>(nch, M, al, bl, tile, wave, lane); break;
        case 4: gen_phase_nks<4>(nch, M, al, bl, tile, wave, lane); break;
        case 5: gen_phase_nks<5>(nch, M, al, bl, tile, wave, lane); break;
        case 6: gen_phase_nks<6>(nch, M, al, bl, tile, wave, lane); break;
        case 7: gen_phase_nks<7>(nch, M, al, bl, tile, wave, lane); break;
        default: gen_phase_nks<8>(nch, M, al, bl, tile, wave, lane); break;
    }
}

// The loop over a unit's tasks, common to both roles; `work(task, table, l2 slab)` is phase 2.
//   carried: cur = task k, nxt = task k+1 (both in scalar registers), loaded one stage before they are needed
//   `diag` selects the stages the call runs: false = the leading ones of ordinary triples, true = the trailing ones
//   of diagonal triples (ft_c0 != 0; they form the last run of a unit).  A role that treats the two kinds with
//   different code calls the loop twice, so that each loop holds a single path (a branch inside the loop that
//   joins two matrix-core paths makes the compiler copy the accumulators at every stage).
struct FusedCursor { FusedTask cur, nxt; int k; };
__device__ __forceinline__ FusedCursor fused_cursor(const FusedTask* __restrict__ ft, int ntask) {
    return FusedCursor{ft[0], ft[min(1, ntask - 1)], 0};
}
template <bool SPLIT, typename Work>
__device__ __forceinline__ void fused_task_loop(const FusedCtx& c, const FusedTask* __restrict__ ft, int ntask,
                                                FusedCursor& cs, bool diag, Work work) {
    for (; cs.k < ntask && (!SPLIT || (ft_c0(cs.cur) != 0) == diag); ++cs.k) {
        const int k = cs.k;
        const FusedTask cur = cs.cur, nxt = cs.nxt;
        dma_wait();
        __syncthreads();       // the tile's operands have landed; nobody uses the tile, the table or the l2 slab
        const FusedTask nxt2 = ft[min(k + 2, ntask - 1)];        // needed at the next stage
        const bool more = k + 1 < ntask;
        // this stage's table and (at the start of a run) l2 slab are only read in phase 2: they arrive during phase 1
        dma16<kHybThreads>(c.CGP + cur.cgp_off, c.cg, cur.cgp_len >> 2, c.tid);
        if (ft_first(cur) || k == 0)
            dma16<kHybThreads>(c.Fp + cur.offF2p, c.f2, (ft_tau2(cur) * (2 * ft_l2(cur) + 2)) >> 1, c.tid);
        gen_phase(cur, c.al, c.bl, c.tile, c.wave, c.lane);
        dma_wait();
        lds_barrier();         // the tile is complete, table and slab have landed; the operand buffers are free
        if (more) {
            dma16<kHybThreads>(c.Ag + nxt.aoff, c.al, nxt.chunks & 0xffff, c.tid);
            dma16<kHybThreads>(c.Bg + nxt.boff, c.bl, nxt.chunks >> 16, c.tid);
        }
        work(cur, reinterpret_cast<const float*>(c.cg), reinterpret_cast<const float2*>(c.f2));
        cs.cur = nxt;
        cs.nxt = nxt2;
    }
}

// Waves of role A (slot 1 on the vector ALUs), as bwd_unit_loop_a.
template <int TI, int RW, int RM>
__device__ __forceinline__ void fused_loop_a(const FusedCtx& c, const BwdUnit& u, const FusedTask* __restrict__ ft,
                                             float2* __restrict__ dst) {
    float ax[kBwdMaxTI][2], ay[kBwdMaxTI][2], tx[kBwdMaxTI][2], ty[kBwdMaxTI][2];
#pragma unroll
    for (int i = 0; i < kBwdMaxTI; ++i) {
        ax[i][0] = ax[i][1] = ay[i][0] = ay[i][1] = 0.f;
        tx[i][0] = tx[i][1] = ty[i][0] = ty[i][1] = 0.f;
    }
    FusedCursor cs = fused_cursor(ft, u.task_end - u.task_begin);
    fused_task_loop<false>(c, ft, u.task_end - u.task_begin, cs, false, [&](const FusedTask& t, const float* cgp, const float2* f2) {
        // a diagonal triple's tile is symmetrised (see build_fused_link): this role reduces over the first 4 c0
        // channels only, the matrix waves over the others
        const int c0 = ft_c0(t);
        const BwdGeom q{ft_l(t), u.l1, ft_l2(t), u.rows, ft_tau2(t), c0 ? 4 * c0 : ft_tau2(t)};
        bwd_accum<1, TI, RW, RM>(q, cgp, reinterpret_cast<const float2*>(c.tile), f2, c.tid, ax, ay);
        if (ft_last(t)) {
#pragma unroll
            for (int i = 0; i < TI; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    tx[i][j] += ax[i][j];
                    ty[i][j] += ay[i][j];
                    ax[i][j] = ay[i][j] = 0.f;
                }
        }
    });
    bwd_flush<TI, RW>(u.rows, 2 * u.l1 + 1, c.tid, tx, ty, dst);
}

// Matrix-core waves (slot 2), as bwd_hybrid_loop_b.
template <int NK, bool KFULL>
__device__ __forceinline__ void fused_loop_b(const FusedCtx& c, const BwdUnit& u, const FusedTask* __restrict__ ft,
                                             int part, int split, float2* __restrict__ part2_b) {
    f32x4 dre[kHybMaxTiles], dim[kHybMaxTiles];
#pragma unroll
    for (int j = 0; j < kHybMaxTiles; ++j) dre[j] = dim[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const float inv_split = 1.0f / (float)split;
    const int ntask = u.task_end - u.task_begin;
    FusedCursor cs = fused_cursor(ft, ntask);
    // ordinary triples: the reduction over all rows; then the diagonal ones, whose first NK / 2 steps the vector
    // waves take (build_fused_link)
    fused_task_loop<true>(c, ft, ntask, cs, false, [&](const FusedTask& t, const float* cgp, const float2* f2) {
        const int l2 = ft_l2(t), tau2 = ft_tau2(t);
        const BwdGeom q{ft_l(t), u.l1, l2, u.rows, tau2, tau2};
        bwd_mm_task<NK, KFULL, 0>(q, cgp, reinterpret_cast<const float2*>(c.tile), c.f1, part, split, inv_split, c.lane, dre, dim);
        if (ft_last(t)) {
            const int M2 = 2 * l2 + 1;
            bwd_mm_store(dre, dim, tau2, M2, c.lane, part2_b + t.p2off + (size_t)part * tau2 * M2);
#pragma unroll
            for (int j = 0; j < kHybMaxTiles; ++j) dre[j] = dim[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
    });
    fused_task_loop<true>(c, ft, ntask, cs, true, [&](const FusedTask& t, const float* cgp, const float2* f2) {
        const int l2 = ft_l2(t), tau2 = ft_tau2(t);
        const BwdGeom q{ft_l(t), u.l1, l2, u.rows, tau2, tau2};
        bwd_mm_task<NK, KFULL, CGNET_DIAG_C0(NK)>(q, cgp, reinterpret_cast<const float2*>(c.tile), c.f1, part, split, inv_split, c.lane, dre, dim);
        if (ft_last(t)) {
            const int M2 = 2 * l2 + 1;
            bwd_mm_store(dre, dim, tau2, M2, c.lane, part2_b + t.p2off + (size_t)part * tau2 * M2);
#pragma unroll
            for (int j = 0; j < kHybMaxTiles; ++j) dre[j] = dim[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
        }
    });
}

// LDS map (bytes): [16 zero] f1 | f2 | table | B operand | A operand | [16 zero] tile [16 zero]
__host__ __device__ inline size_t bwd_fused_lds(int f1cap, int f2cap, int cgcap, int tcap, int bcap, int acap) {
    return 16 + (size_t)f1cap + (size_t)f2cap + (size_t)cgcap + (size_t)bcap + (size_t)acap + 16 + (size_t)tcap + 16;
}

__global__ void __launch_bounds__(kHybThreads, 6)     // 80 registers: three work-groups per compute unit where the LDS allows
cgbn_backward_fused_kernel(const float2* __restrict__ Fp, const float* __restrict__ Bg, const float* __restrict__ Ag,
                           const float* __restrict__ CGP, float2* __restrict__ part1, float2* __restrict__ part2,
                           const BwdUnit* __restrict__ units, const FusedTask* __restrict__ ftasks, int nF, int nFp,
                           int nBg, int P2, int f1cap, int f2cap, int cgcap, int tcap, int bcap, int acap, int B) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = unit_major(B);
    const BwdUnit u = units[up.unit];
    const int b = up.part;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M1 = 2 * u.l1 + 1;
    const bool roleA = wave < u.nA;                  // wave-uniform
    FusedCtx c;
    c.Fp = Fp + (size_t)b * nFp;
    c.Bg = Bg + (size_t)b * nBg;
    c.Ag = Ag;
    c.CGP = CGP;
    c.f1 = reinterpret_cast<float2*>(smem + 16);
    c.f2 = reinterpret_cast<char*>(smem) + 16 + f1cap;
    c.cg = c.f2 + f2cap;
    c.bl = reinterpret_cast<float*>(c.cg + cgcap);
    c.al = reinterpret_cast<float*>(reinterpret_cast<char*>(c.bl) + bcap);
    c.tile = reinterpret_cast<float*>(reinterpret_cast<char*>(c.al) + acap + 16);
    c.f2cap = f2cap; c.cgcap = cgcap;
    c.tid = tid; c.lane = tid & 63; c.wave = wave;
    {
        const int n16 = (int)(bwd_fused_lds(f1cap, f2cap, cgcap, tcap, bcap, acap) >> 4);
        float4* z = reinterpret_cast<float4*>(smem);
        for (int e = tid; e < n16; e += kHybThreads) z[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    __syncthreads();                                 // the clearing stores precede every copy
    const FusedTask* ft = ftasks + u.task_begin;
    const FusedTask t0 = ft[0];
    dma16<kHybThreads>(c.Fp + u.offF1p, c.f1, (u.rows * (M1 + 1)) >> 1, tid);
    dma16<kHybThreads>(c.Ag + t0.aoff, c.al, t0.chunks & 0xffff, tid);
    dma16<kHybThreads>(c.Bg + t0.boff, c.bl, t0.chunks >> 16, tid);
    // the first stage waits for these copies
    if (roleA) {
        float2* dst = u.p1off < 0 ? part1 + (size_t)b * nF + u.offF1 : part2 + (size_t)b * P2 + u.p1off;
#define CGNET_LOOP_A(TI_, RW_, RM_) fused_loop_a<TI_, RW_, RM_>(c, u, ft, dst)
        CGNET_BWD_SWITCH_A3(u.TI, u.RW, u.RM, CGNET_LOOP_A)
#undef CGNET_LOOP_A
    } else {
#define CGNET_LOOP_B(NK_, KF_) fused_loop_b<NK_, KF_>(c, u, ft, wave - u.nA, kHybWaves - u.nA, part2 + (size_t)b * P2)
        CGNET_HYB_ROLE_B(u.rows, CGNET_LOOP_B)
#undef CGNET_LOOP_B
    }
}

// The A operand of the fused kernel (layout: pack_w_gen_lane), one work-group of 64 threads per (task, row tile).
__global__ void __launch_bounds__(64)
pack_w_gen_kernel(const float2* __restrict__ W, const float* __restrict__ stds, float eps,
                  const GenTask* __restrict__ gens, const int* __restrict__ map, float* __restrict__ Ag) {
    pack_w_gen_lane(W, stds, eps, gens[map[2 * blockIdx.x]], map[2 * blockIdx.x + 1], threadIdx.x, Ag);
}

// The B operand of the fused kernel, per sample and degree: entry [(column tile * nks + ks) * 64 + lane] =
// B[k][col] for k = 4 * ks + lane / 16 = (to, re/im), col = 16 * column tile + lane % 16 = (m, re/im); k past 2 t_O
// and columns past 2M are zero.  map: per block (cumO, M, t_O, column tile | k-step << 8) of its degree.
__global__ void __launch_bounds__(64)
pack_go_gen_kernel(const float2* __restrict__ gO, const int* __restrict__ map, float* __restrict__ Bg, int nO, int nBg) {
    const int* mp = map + 4 * blockIdx.x;
    const int cumO = mp[0], M = mp[1], tO = mp[2], ks = mp[3] >> 8;
    const int ct = mp[3] & 255;
    const int lane = threadIdx.x, i = lane & 15, kk = lane >> 4;
    const int k = 4 * ks + kk, to = k >> 1, sel = k & 1;
    const int col = 16 * ct + i, m = col >> 1, r = col & 1;
    float v = 0.f;
    if (to < tO && m < M) {
        const float2 z = gO[(size_t)blockIdx.y * nO + cumO + to * M + m];
        v = (r == sel) ? (r ? -z.x : z.x) : z.y;
    }
    Bg[(size_t)blockIdx.y * nBg + (size_t)blockIdx.x * 64 + lane] = v;
}

// Builds the operands the unit kernel copies straight into LDS: fragments with one zero behind
// every row (blocks below nbF) and every triple's table between kTabLo / kTabHi zero rows
// (one block per triple).
__global__ void __launch_bounds__(256)
cg_backward_pad_kernel(const float2* __restrict__ F, const float* __restrict__ CG, float2* __restrict__ Fp,
                       float* __restrict__ CGP, const int* __restrict__ meta, int L, int nF, int nFp, int B,
                       int nbF) {
    __shared__ int s_tab[kMaxLookup];
    if ((int)blockIdx.x < nbF) pad_fragments_block(F, Fp, meta, L, nF, nFp, B, (int)blockIdx.x, s_tab);
    else pad_table_block(CG, CGP, meta + 2 * (L + 2) + kPadMetaInts * ((int)blockIdx.x - nbF));
}

// gF[b][e] = slot-1 part (if any unit owns the degree) + the slot-2 slabs of that degree, in list order
__global__ void __launch_bounds__(256)
cg_backward_combine_kernel(const float2* __restrict__ part1, const float2* __restrict__ part2,
                           float2* __restrict__ gF, const int* __restrict__ meta, int L, int nF, int P2, int B) {
    __shared__ int s_tab[kMaxLookup];
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int b = (int)(idx / nF), e = (int)(idx % nF);
    const int* cumF = meta;                 // L+2
    const int* own1 = meta + (L + 2);       // L+1
    const int* lbeg = own1 + (L + 1);       // L+2
    const int* loff = lbeg + (L + 2);
    const int lam = lookup_in_group(L + 1, e, [&](int k) { return cumF[k]; }, s_tab);
    if (idx >= (size_t)B * nF) return;
    const int rel = e - cumF[lam];
    float2 s = make_float2(0.f, 0.f);
    if (own1[lam]) s = part1[idx];
    const float2* p2 = part2 + (size_t)b * P2;
#pragma unroll 8
    for (int k = lbeg[lam]; k < lbeg[lam + 1]; ++k) {
        const float2 v = p2[loff[k] + rel];
        s.x += v.x;
        s.y += v.y;
    }
    gF[idx] = s;
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

__global__ void __launch_bounds__(256) fill_zero_f64_kernel(double* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.;
}

__global__ void __launch_bounds__(256) fill_zero_f32_kernel(float* p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

// ------------------------------------------------------------------------------------- host
// Partial statistics of cgnet_sparse_forward_stats_static: a fixed area every GPU the library runs
// on holds until the process ends.  In host code the array's name is only a handle; its device
// address is resolved once per device (resolve_static_scratch) and that pointer is what kernels get.
constexpr size_t kStaticScratchBytes = 16u << 20;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
static std::mutex g_scratch_mu;
static void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device (nullptr and an error message on failure).
void* resolve_static_scratch() {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        set_error("cannot identify the current device");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[device]) {
        void* ptr = nullptr;
        const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            set_error("hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[device] = ptr;
    }
    return g_scratch_ptr[device];
}

int bwd_groups_for(const cgnet_cg_plan* p, int B) {
    const int maxg = (int)p->bwd_group_begin.size() - 1;
    if (maxg <= 0) return 0;
    int want = (1024 + B - 1) / std::max(1, B);
    return std::max(1, std::min(maxg, want));
}

}  // namespace

int samples_per_group_for(int B, int ntasks) {
    // enough work-groups to fill 256 CUs a few times over, while each group amortises the
    // staging of its CG table over several samples
    int groups = std::max(1, std::min(B, (6144 + ntasks - 1) / std::max(1, ntasks)));
    return (B + groups - 1) / groups;
}
}  // namespace cgnet

using namespace cgnet;

static void free_plan(cgnet_cg_plan* plan) {
    if (!plan) return;
    if (plan->d_fwd_tasks) (void)hipFree(plan->d_fwd_tasks);
    if (plan->d_bwd_tasks) (void)hipFree(plan->d_bwd_tasks);
    if (plan->d_bwd_group_table) (void)hipFree(plan->d_bwd_group_table);
    if (plan->d_bwd_units) (void)hipFree(plan->d_bwd_units);
    if (plan->d_bwd_utasks) (void)hipFree(plan->d_bwd_utasks);
    if (plan->d_bwd_combine) (void)hipFree(plan->d_bwd_combine);
    if (plan->d_bwd_padmeta) (void)hipFree(plan->d_bwd_padmeta);
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

    auto build = [&](int tile_bytes, std::vector<CgTask>* out, int pad = 0, bool mm = false) -> int {
        for (int i = 0; i < nllls; ++i) {
            const int l = tl[i], l1 = tl1[i], l2 = tl2[i];
            const int tau1 = h_t_F[l1], tau2 = h_t_F[l2];
            if (tau1 == 0 || tau2 == 0) continue;
            const int M = 2 * l + 1;
            const long long row_bytes = 8LL * tau2 * (M + pad);
            int max_rows = (int)std::min<long long>(tau1, std::max<long long>(1, tile_bytes / row_bytes));
            max_rows = std::max(1, std::min(max_rows, kMaxTileChannels / tau2));
            if (mm) {
                // the whole work-group (tile, two pairs of fragment slabs, padded table) has to fit the LDS
                CgTask probe;
                probe.l = l; probe.l1 = l1; probe.l2 = l2; probe.tau1 = tau1; probe.tau2 = tau2;
                for (probe.rows = max_rows; probe.rows > 1 && fwd_task_lds_mm(probe) > kMaxLds; --probe.rows) {}
                max_rows = probe.rows;
            }
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
                // Register tile of the forward kernel: the one whose items (tiles x m) fill the waves they
                // occupy best, weighed by the instructions of one term of the inner loop
                // (4 TI TJ multiply-adds + 2 TI coefficient products + TI + TJ + 3 address / loop steps).
                double best_cost = -1;
                for (int ti = 1; ti <= std::min(4, t.rows); ++ti)
                    for (int tj = 1; tj <= std::min(4, tau2); ++tj) {
                        const int n1 = (t.rows + ti - 1) / ti, n2 = (tau2 + tj - 1) / tj;
                        const long long items = (long long)n1 * n2 * M;
                        double cost = (double)((items + 63) / 64) * (4 * ti * tj + 3 * ti + tj + 3);
                        // more items than threads: the per-item set-up is redone for every sample
                        if (items > kThreads) cost *= 1.25;
                        if (best_cost < 0 || cost < best_cost * (1 - 1e-9)) {
                            best_cost = cost;
                            t.nT1 = n1; t.nT2 = n2;
                        }
                    }
                t.TI = (t.rows + t.nT1 - 1) / t.nT1;
                t.TJ = (tau2 + t.nT2 - 1) / t.nT2;
                t.bTI[0] = t.bTI[1] = 1;
                t.bRW[0] = t.bRW[1] = 1;
                t.sym = 0;
                out->push_back(t);
            }
        }
        return 0;
    };
    // Product on the matrix cores when every channel count fills a good part of a 16 x 16 tile (CGNET_FWD_MM=0
    // keeps the vector-ALU kernel).  Its tasks then take all rows of a triple -- a row block of six of sixteen
    // rows, which the 32 KB limit gives at 41 values of m, fills the matrix tiles to 37 % -- up to kFwdMmTileBytes.
    p->fwd_mm = true;
    for (int l = 0; l < n1; ++l)
        if (h_t_F[l] != 0 && (h_t_F[l] < 8 || h_t_F[l] > 16)) p->fwd_mm = false;
    if (const char* e = getenv("CGNET_FWD_MM"); e && e[0] == '0') p->fwd_mm = false;
    build(p->fwd_mm ? kFwdMmTileBytes : kFwdTileBytes, &p->fwd_tasks, 0, p->fwd_mm);
    p->bwd_tasks.clear();
    build(kBwdTileBytes, &p->bwd_tasks, kPadLo + kPadHi);
    // Backward tiling.  Per slot a thread owns TI output channels x 2 m and RW lanes split the
    // reduced channels.  cost = passes over the work-group * sequential steps of a lane * TI;
    // the work-group size that wastes the fewest lane-steps over all tasks is kept.
    {
        const int cand[3] = {128, 192, 256};
        double best_total = -1;
        for (int ci = 0; ci < 3; ++ci) {
            const int wg = cand[ci];
            double total = 0;
            std::vector<CgTask> tmp = p->bwd_tasks;
            for (CgTask& t : tmp) {
                for (int slot = 0; slot < 2; ++slot) {
                    const int n_o = slot == 0 ? t.rows : t.tau2, n_r = slot == 0 ? t.tau2 : t.rows;
                    const int M_o = slot == 0 ? 2 * t.l1 + 1 : 2 * t.l2 + 1;
                    const int M_r = slot == 0 ? 2 * t.l2 + 1 : 2 * t.l1 + 1;
                    double best = -1;
                    for (int ti = 1; ti <= 4; ++ti)
                        for (int rw = 1; rw <= 16; rw *= 2) {
                            if (rw > 1 && rw / 2 >= n_r) continue;
                            const int items = ((n_o + ti - 1) / ti) * ((M_o + 1) / 2);
                            const int rows_blk = wg / rw;
                            const double passes = (items + rows_blk - 1) / rows_blk;
                            // steps of one lane; the row reduction costs about 2*ti*log2(rw) more
                            double c = passes * (((n_r + rw - 1) / rw) * (double)M_r * (ti + 0.75) + 1.5 * ti * rw);
                            if (best < 0 || c < best) { best = c; t.bTI[slot] = ti; t.bRW[slot] = rw; }
                        }
                    total += best * wg;
                }
            }
            if (best_total < 0 || total < best_total) {
                best_total = total;
                p->bwd_threads = wg;
                p->bwd_tasks = tmp;
            }
        }
    }
    // heaviest forward tasks first: a short tail when the grid drains
    std::stable_sort(p->fwd_tasks.begin(), p->fwd_tasks.end(), [](const CgTask& a, const CgTask& b) {
        return (long long)a.rows * a.tau2 * (2 * a.l + 1) * (2 * a.l2 + 1) >
               (long long)b.rows * b.tau2 * (2 * b.l + 1) * (2 * b.l2 + 1);
    });
    // One launch has one LDS size, and the largest task's would set the occupancy of all: the tasks are
    // grouped by the number of work-groups per compute unit their own LDS need allows (at most four, the
    // register limit), largest need first, and every class gets a launch of its own.
    const bool fwd_mm = p->fwd_mm;
    auto fwd_need = [fwd_mm](const CgTask& t) { return align_up(fwd_mm ? fwd_task_lds_mm(t) : fwd_task_lds(t), 16); };
    auto fwd_class = [&](const CgTask& t) { return (int)std::max<size_t>(1, std::min<size_t>(4, kMaxLds / fwd_need(t))); };
    std::stable_sort(p->fwd_tasks.begin(), p->fwd_tasks.end(),
                     [&](const CgTask& a, const CgTask& b) { return fwd_class(a) < fwd_class(b); });
    p->fwd_class_begin.clear();
    p->fwd_class_lds.clear();
    for (size_t k = 0; k < p->fwd_tasks.size(); ++k) {
        if (k == 0 || fwd_class(p->fwd_tasks[k]) != fwd_class(p->fwd_tasks[k - 1])) {
            p->fwd_class_begin.push_back((int)k);
            p->fwd_class_lds.push_back(0);
        }
        p->fwd_class_lds.back() = std::max(p->fwd_class_lds.back(), fwd_need(p->fwd_tasks[k]));
    }
    p->fwd_class_begin.push_back((int)p->fwd_tasks.size());
    size_t fl = 0, bl = 0;
    for (const CgTask& t : p->fwd_tasks) {
        fl = std::max(fl, fwd_need(t));
        CGNET_REQUIRE(2 * fwd_frag_lds(t) <= kMaxUnitLds, CGNET_ERR_UNSUPPORTED,
                      "fragment slabs of %zu bytes exceed the LDS staging window", 2 * fwd_frag_lds(t));
    }
    for (const CgTask& t : p->bwd_tasks) bl = std::max(bl, bwd_task_lds(t));
    p->fwd_lds = align_up(fl, 16);
    p->bwd_lds = align_up(bl, 16) + 8 * (size_t)p->nF;
    CGNET_REQUIRE(p->fwd_lds <= kMaxLds, CGNET_ERR_UNSUPPORTED,
                  "a single output row needs %zu bytes of LDS (limit %zu)", p->fwd_lds, kMaxLds);
    // The LDS-accumulator backward keeps a sample's whole input gradient in LDS.  Where that does not fit, the
    // backward depends on the unit kernels below; where they do not fit either, the plan serves the forward only and
    // cgnet_sparse_backward reports the shape as unsupported.
    p->bwd_general_ok = p->bwd_lds <= kMaxLds;

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

    // ---- register-resident backward: units = (l1, range of t1 rows), tasks ordered by (l2, l)
    std::vector<int> combine_meta, pad_meta;
    // First with slot 2 on the matrix cores where the shapes allow it: with the largest tiles that let four work-groups
    // share a compute unit's LDS (kHybLds4) unless that cuts a degree's tiles below four rows, then the same for three
    // groups (kHybLds3), failing that with two work-groups; then all on the vector ALUs.  Measured at tau = 16:
    // L=15, four groups with 5-row tiles 1.54 ms, three groups with 10-row tiles 1.57 ms; L=20 (B=16), four groups with
    // 2-row tiles 1.96 ms, three groups with 4-row tiles 1.44 ms.
    const int hyb_tiles_kb[] = {30, 28, 24, 20, 16, 12, 40, 36, 32, 28, 24, 20, 16, 12, 8, 4};
    const int n_hyb4 = 6;
    const int n_hyb = (int)(sizeof(hyb_tiles_kb) / sizeof(hyb_tiles_kb[0]));
    for (int attempt = 0; attempt < n_hyb + 2 && !p->bwd_fast; ++attempt) {
        bool ok = true;
        int P2 = 0;
        size_t lds_max = 0;
        // fragments with one zero behind every row; every triple's table between zero rows
        std::vector<int> cumFp(n1 + 1, 0), cgp_off(nllls + 1, 0);
        for (int l = 0; l < n1; ++l) cumFp[l + 1] = cumFp[l] + h_t_F[l] * (2 * l + 2);
        for (int i = 0; i < nllls; ++i) {
            const long long len = ((long long)(2 * tl[i] + 1 + kTabLo + kTabHi) * (2 * tl2[i] + 1) + 1 + 3) & ~3LL;
            if ((long long)cgp_off[i] + len > INT32_MAX) { ok = false; break; }
            cgp_off[i + 1] = cgp_off[i] + (int)len;
        }
        // Slot 2 on the matrix cores: needs every channel count to fit one 16-row tile (and to fill a
        // good part of it), the m2 axis kHybMaxTiles 16-column tiles.  CGNET_BWD_HYBRID=0 keeps all on the vector ALUs.
        bool hybrid = attempt <= n_hyb && n1 - 1 <= 8 * kHybMaxTiles - 1;
        for (int l = 0; l < n1; ++l)
            if (h_t_F[l] != 0 && (h_t_F[l] < 8 || h_t_F[l] > 16)) hybrid = false;
        if (const char* e = getenv("CGNET_BWD_HYBRID"); e && e[0] == '0') hybrid = false;
        bool use_rm = true;      // CGNET_BWD_MSPLIT=0: lanes of an item split only the reduced channels
        if (const char* e = getenv("CGNET_BWD_MSPLIT"); e && e[0] == '0') use_rm = false;
        if (attempt <= n_hyb && !hybrid) continue;
        // attempts 0 .. n_hyb4 - 1: four groups per compute unit; .. n_hyb - 1: three; attempt n_hyb: two groups, tiles
        // of kHybTileBytes
        const int hyb_groups = attempt < n_hyb4 ? 4 : attempt < n_hyb ? 3 : 2;
        // CGNET_BWD_MAX_GROUPS=3 (or 2): plans for four (three) work-groups per compute unit are not tried
        if (const char* e = getenv("CGNET_BWD_MAX_GROUPS"); e && hybrid && attempt <= n_hyb && hyb_groups > atoi(e)) continue;
        const long long tile_limit = !hybrid ? kBwdTileBytes : attempt < n_hyb ? hyb_tiles_kb[attempt] * 1024LL : kHybTileBytes;
        const size_t hyb_lds_limit = hyb_groups == 4 ? kHybLds4 : hyb_groups == 3 ? kHybLds3 : kMaxHybLds;
        const int hyb_max_ti = hyb_groups == 4 ? 2 : kHybMaxTI;
        int f1cap = 0, f2cap = 0, cgcap = 0, tcap = 0;
        std::vector<int> own1(n1, 0);
        std::vector<std::vector<int>> lam_offs(n1);
        std::vector<double> unit_cost, task_cost;
        for (int l1 = 0; l1 < n1 && ok; ++l1) {
            std::vector<int> tri;
            for (int i = 0; i < nllls; ++i)
                if (tl1[i] == l1 && h_t_F[l1] > 0 && h_t_F[tl2[i]] > 0) tri.push_back(i);
            if (tri.empty()) continue;
            own1[l1] = 1;
            std::stable_sort(tri.begin(), tri.end(), [&](int a, int b) {
                return tl2[a] != tl2[b] ? tl2[a] < tl2[b] : tl[a] < tl[b];
            });
            const int tau1 = h_t_F[l1], M1 = 2 * l1 + 1;
            const int nt = (int)tri.size();
            struct Choice { double total = -1; int rows = 0, nA = 0, TI = 0, RW = 0, RM = 1; std::vector<int> bTI, bRW; std::vector<double> tcost; };
            Choice best;
            int prev_rows = -1;
            for (int nchunks = 1; nchunks <= tau1; ++nchunks) {
                const int rows_c = (tau1 + nchunks - 1) / nchunks;
                if (rows_c == prev_rows) continue;
                prev_rows = rows_c;
                long long max_tile = 0;
                for (int i : tri) max_tile = std::max(max_tile, 8LL * rows_c * h_t_F[tl2[i]] * (2 * tl[i] + 1));
                if (max_tile > tile_limit && rows_c > 1) continue;
                if (hybrid && rows_c > kHybMaxRows) continue;
                const int real_chunks = (tau1 + rows_c - 1) / rows_c;
                for (int nA = hybrid ? 4 : 1; nA <= (hybrid ? 6 : 3); ++nA) {
                    const int lanesA = 64 * nA, lanesB = hybrid ? 0 : kThreads - lanesA;
                    // slot 2: best tiling per task (constant within a run of equal l2)
                    std::vector<double> costB(nt);
                    std::vector<int> bTI(nt), bRW(nt);
                    bool feasible = true;
                    for (int k = 0; k < nt && feasible; ++k) {
                        const int tau2 = h_t_F[tl2[tri[k]]], M2 = 2 * tl2[tri[k]] + 1;
                        double bc = -1;
                        if (hybrid) {
                            // a matrix instruction occupies its pipeline for eight vector-instruction slots
                            const int Mq = 2 * tl[tri[k]] + 1;
                            const int split = kHybWaves - nA;
                            bc = ((Mq + split - 1) / split) * (double)((M2 + 15) / 16) * (((rows_c + 3) / 4) * 32.0 + 18.0);
                            bTI[k] = 1; bRW[k] = 1;
                        }
                        for (int ti = 1; ti <= kBwdMaxTI && !hybrid; ++ti)
                            for (int rw = 1; rw <= 16; rw *= 2) {
                                if (rw > 1 && rw / 2 >= rows_c) continue;
                                const int items = ((tau2 + ti - 1) / ti) * ((M2 + 1) / 2);
                                if (items * rw > lanesB) continue;
                                const double c = ((rows_c + rw - 1) / rw) * (double)M1 * (8.0 * ti + 14.0);
                                if (bc < 0 || c < bc) { bc = c; bTI[k] = ti; bRW[k] = rw; }
                            }
                        if (bc < 0) feasible = false;
                        costB[k] = bc;
                    }
                    if (!feasible) continue;
                    int max_tau2 = 1;
                    for (int i : tri) max_tau2 = std::max(max_tau2, h_t_F[tl2[i]]);
                    for (int ti = 1; ti <= (hybrid ? hyb_max_ti : kBwdMaxTI); ++ti)
                        for (int rw = 1; rw <= 16; rw *= 2)
                            for (int rm = 1; rm <= 2; ++rm) {
                                // rm = 2: half of the lanes of an item take the second half of the reduced m range
                                if (rm == 2 && (rw < 4 || ti < 2 || !use_rm)) continue;
                                const int rc = rw / rm;
                                if (rc > 1 && rc / 2 >= max_tau2) continue;
                                const int items = ((rows_c + ti - 1) / ti) * ((M1 + 1) / 2);
                                if (items * rw > lanesA) continue;
                                double total = 0;
                                std::vector<double> tcost(nt);
                                for (int k = 0; k < nt; ++k) {
                                    const int tau2 = h_t_F[tl2[tri[k]]], M2 = 2 * tl2[tri[k]] + 1;
                                    const double scaleA = hybrid ? kHybSlot1Scale : 1.0;
                                    // steps of the busiest lane: its channels x its part of the m range (in step pairs)
                                    const double msteps = rm == 1 ? (double)M2 : 2.0 * ((M2 / 2 + 2) / 2) + 1.0;
                                    const double cA = scaleA * ((tau2 + rc - 1) / rc) * msteps * (8.0 * ti + 14.0);
                                    const double stage = 12.0 * rows_c * tau2 * (2 * tl[tri[k]] + 4) / kThreads + 200.0;
                                    tcost[k] = std::max(cA, costB[k]) + stage;
                                    total += tcost[k];
                                }
                                total *= real_chunks;
                                if (best.total < 0 || total < best.total) {
                                    best.total = total; best.rows = rows_c; best.nA = nA; best.TI = ti; best.RW = rw;
                                    best.RM = rm;
                                    best.bTI = bTI; best.bRW = bRW; best.tcost = tcost;
                                }
                            }
                }
            }
            if (best.total < 0) { ok = false; break; }
            // four groups per compute unit only while every degree keeps tiles of at least four rows
            if (hybrid && hyb_groups == 4 && best.rows < std::min(tau1, 4)) { ok = false; break; }
            for (int r0 = 0; r0 < tau1; r0 += best.rows) {
                BwdUnit u;
                u.l1 = l1;
                u.rows = std::min(best.rows, tau1 - r0);
                u.offF1 = p->cumF[l1] + r0 * M1;
                u.offF1p = cumFp[l1] + r0 * (M1 + 1);
                u.task_begin = (int)p->bwd_utasks.size();
                u.nA = best.nA; u.TI = best.TI; u.RW = best.RW; u.RM = best.RM;
                u.p1off = -1;
                f1cap = std::max(f1cap, (int)align_up((size_t)8 * u.rows * (M1 + 1), 16));
                for (int k = 0; k < nt; ++k) {
                    const int i = tri[k];
                    BwdUTask t;
                    t.l = tl[i]; t.l2 = tl2[i]; t.tau2 = h_t_F[tl2[i]];
                    const int M = 2 * t.l + 1, M2 = 2 * t.l2 + 1;
                    t.offFF = p->cumFF[t.l] + (p->t_off[i] + r0 * t.tau2) * M;
                    t.offF2 = p->cumF[t.l2];
                    t.offF2p = cumFp[t.l2];
                    t.cg_off = cgo[i];
                    t.cgp_off = cgp_off[i];
                    t.cgp_len = cgp_off[i + 1] - cgp_off[i];
                    t.first_of_l2 = (k == 0 || tl2[tri[k - 1]] != t.l2) ? 1 : 0;
                    t.last_of_l2 = (k + 1 == nt || tl2[tri[k + 1]] != t.l2) ? 1 : 0;
                    if (t.first_of_l2) {
                        // one slab per (unit, l2); the matrix-core waves write one each
                        t.p2off = P2;
                        for (int sp = 0; sp < (hybrid ? kHybWaves - best.nA : 1); ++sp) {
                            lam_offs[t.l2].push_back(P2);
                            P2 += t.tau2 * M2;
                        }
                    } else {
                        t.p2off = p->bwd_utasks.back().p2off;
                    }
                    t.TI = best.bTI[k]; t.RW = best.bRW[k];
                    p->bwd_utasks.push_back(t);
                    task_cost.push_back(best.tcost[k]);
                    const size_t tile_bytes = align_up((size_t)8 * u.rows * t.tau2 * M, 16);
                    if (tile_bytes > kMaxLds) { ok = false; break; }
                    f2cap = std::max(f2cap, (int)align_up((size_t)8 * t.tau2 * (M2 + 1), 16));
                    cgcap = std::max(cgcap, 4 * t.cgp_len);
                    tcap = std::max(tcap, (int)tile_bytes);
                }
                u.task_end = (int)p->bwd_utasks.size();
                lds_max = bwd_unit_lds(f1cap, f2cap, cgcap, tcap, hybrid ? 1 : 2);
                p->bwd_units.push_back(u);
            }
        }
        // A unit longer than its share of the machine would outlast all others: task lists are cut at
        // the boundaries between runs of equal l2 into pieces of at most 1/kBwdPieces of a sample's work.
        // The pieces after the first of a degree put their slot-1 result into slabs of the slot-2
        // partial area (the same cuts for all row ranges of the degree, so every slab is covered).
        if (ok) {
            double all = 0;
            for (double c : task_cost) all += c;
            int pieces = kBwdPieces;
            if (const char* e = getenv("CGNET_BWD_PIECES")) pieces = std::max(1, atoi(e));
            const double target = all / pieces;
            std::vector<BwdUnit> cut;
            std::vector<int> slab_of_piece;              // per degree: slab offsets of pieces 1, 2, ...
            int cur_l1 = -1;
            for (const BwdUnit& u : p->bwd_units) {
                const int M1 = 2 * u.l1 + 1, tau1 = h_t_F[u.l1];
                const int r0 = (u.offF1 - p->cumF[u.l1]) / M1;
                if (u.l1 != cur_l1) { cur_l1 = u.l1; slab_of_piece.clear(); }
                double piece_cost = 0;
                int start = u.task_begin, piece = 0;
                // all row ranges of a degree have the same task list and costs, hence the same cuts
                for (int k = u.task_begin; k < u.task_end; ++k) {
                    piece_cost += task_cost[k];
                    const bool last = k + 1 == u.task_end;
                    if (last || (p->bwd_utasks[k].last_of_l2 && piece_cost >= target)) {
                        BwdUnit v = u;
                        v.task_begin = start;
                        v.task_end = k + 1;
                        if (piece > 0) {
                            if ((int)slab_of_piece.size() < piece) {
                                slab_of_piece.push_back(P2);
                                lam_offs[u.l1].push_back(P2);
                                P2 += tau1 * M1;
                            }
                            v.p1off = slab_of_piece[piece - 1] + r0 * M1;
                        }
                        cut.push_back(v);
                        unit_cost.push_back(piece_cost);
                        start = k + 1;
                        piece_cost = 0;
                        ++piece;
                    }
                }
            }
            p->bwd_units.swap(cut);
        }
        // CGNET_BWD_GENERAL=1 forces the LDS-accumulator kernel (kept for shapes the unit scheme cannot hold)
        const char* force_general = getenv("CGNET_BWD_GENERAL");
        if (force_general && force_general[0] == '1') ok = false;
        if (ok && !p->bwd_units.empty() && lds_max <= (hybrid ? hyb_lds_limit : kMaxUnitLds)) {
            p->bwd_hybrid = hybrid;
            p->bwd_hyb_groups = hybrid ? hyb_groups : 0;
            // longest units first
            std::vector<int> order(p->bwd_units.size());
            for (size_t k = 0; k < order.size(); ++k) order[k] = (int)k;
            std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return unit_cost[a] > unit_cost[b]; });
            std::vector<BwdUnit> sorted;
            for (int k : order) sorted.push_back(p->bwd_units[k]);
            p->bwd_units.swap(sorted);
            p->bwd_fast = true;
            p->bwd_P2 = P2;
            p->bwd_nFp = cumFp[n1];
            p->bwd_cgp_len = cgp_off[nllls];
            p->bwd_f1cap = f1cap; p->bwd_f2cap = f2cap; p->bwd_cgcap = cgcap; p->bwd_tcap = tcap;
            pad_meta.insert(pad_meta.end(), p->cumF.begin(), p->cumF.end());           // L+2
            pad_meta.insert(pad_meta.end(), cumFp.begin(), cumFp.end());               // L+2
            for (int i = 0; i < nllls; ++i) {
                const int v[kPadMetaInts] = {cgo[i], cgp_off[i], cgp_off[i + 1] - cgp_off[i], 2 * tl[i] + 1, 2 * tl2[i] + 1, tl1[i]};
                pad_meta.insert(pad_meta.end(), v, v + kPadMetaInts);
            }
            if (const char* dbg = getenv("CGNET_DEBUG"); dbg && dbg[0] == '1') {
                fprintf(stderr, "[cgnet] backward units=%zu tasks=%zu P2=%d lds=%zu%s\n", p->bwd_units.size(),
                        p->bwd_utasks.size(), P2, lds_max, hybrid ? " (slot 2 on the matrix cores)" : "");
                for (const BwdUnit& u : p->bwd_units) {
                    const BwdUTask& t0 = p->bwd_utasks[u.task_begin];
                    const BwdUTask& t1 = p->bwd_utasks[u.task_end - 1];
                    fprintf(stderr, "[cgnet]   l1=%d rows=%d tasks=%d nA=%d A(TI=%d,RW=%d,RM=%d) B first(TI=%d,RW=%d) last(TI=%d,RW=%d)\n",
                            u.l1, u.rows, u.task_end - u.task_begin, u.nA, u.TI, u.RW, u.RM, t0.TI, t0.RW, t1.TI, t1.RW);
                }
            }
            p->bwd_fast_lds = align_up(lds_max, 16);
            combine_meta.insert(combine_meta.end(), p->cumF.begin(), p->cumF.end());   // L+2
            combine_meta.insert(combine_meta.end(), own1.begin(), own1.end());         // L+1
            int run = 0;
            for (int l = 0; l < n1; ++l) { combine_meta.push_back(run); run += (int)lam_offs[l].size(); }
            combine_meta.push_back(run);
            for (int l = 0; l < n1; ++l) combine_meta.insert(combine_meta.end(), lam_offs[l].begin(), lam_offs[l].end());
        } else {
            p->bwd_units.clear();
            p->bwd_utasks.clear();
        }
    }

    CGNET_HIP(hipGetDevice(&p->device));
    // set-up time: the statistics area of cgnet_sparse_forward_stats_static gets its address on this device
    // (a plan is usable without it: a failure here is reported by that entry point, which resolves the address again)
    if (!resolve_static_scratch()) clear_error();
    if (!p->fwd_tasks.empty()) {
        CGNET_HIP(hipMalloc((void**)&p->d_fwd_tasks, sizeof(CgTask) * p->fwd_tasks.size()));
        CGNET_HIP(hipMemcpy(p->d_fwd_tasks, p->fwd_tasks.data(), sizeof(CgTask) * p->fwd_tasks.size(), hipMemcpyHostToDevice));
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_tasks, sizeof(CgTask) * p->bwd_tasks.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_tasks, p->bwd_tasks.data(), sizeof(CgTask) * p->bwd_tasks.size(), hipMemcpyHostToDevice));
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_group_table, sizeof(int) * gtab.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_group_table, gtab.data(), sizeof(int) * gtab.size(), hipMemcpyHostToDevice));
    }
    if (p->bwd_fast) {
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_units, sizeof(BwdUnit) * p->bwd_units.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_units, p->bwd_units.data(), sizeof(BwdUnit) * p->bwd_units.size(), hipMemcpyHostToDevice));
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_utasks, sizeof(BwdUTask) * p->bwd_utasks.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_utasks, p->bwd_utasks.data(), sizeof(BwdUTask) * p->bwd_utasks.size(), hipMemcpyHostToDevice));
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_combine, sizeof(int) * combine_meta.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_combine, combine_meta.data(), sizeof(int) * combine_meta.size(), hipMemcpyHostToDevice));
        CGNET_HIP(hipMalloc((void**)&p->d_bwd_padmeta, sizeof(int) * pad_meta.size()));
        CGNET_HIP(hipMemcpy(p->d_bwd_padmeta, pad_meta.data(), sizeof(int) * pad_meta.size(), hipMemcpyHostToDevice));
        if (int rc = raise_dynamic_lds(!p->bwd_hybrid            ? (const void*)cg_backward_unit_kernel
                                       : p->bwd_hyb_groups == 4 ? (const void*)cg_backward_hybrid_kernel<true>
                                                                : (const void*)cg_backward_hybrid_kernel<false>,
                                       p->bwd_fast_lds))
            return rc;
    }
    if (int rc = raise_dynamic_lds(p->fwd_mm ? (const void*)cg_forward_mm_kernel : (const void*)cg_forward_kernel, p->fwd_lds)) return rc;
    if (p->bwd_general_ok)
        if (int rc = raise_dynamic_lds((const void*)cg_backward_kernel, p->bwd_lds)) return rc;
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

extern "C" size_t cgnet_cg_plan_forward_lds(const cgnet_cg_plan* plan) { return plan ? plan->fwd_lds : 0; }

extern "C" int cgnet_cg_plan_backward_groups(const cgnet_cg_plan* plan) {
    if (!plan) return 0;
    const size_t lds = cgnet_cg_plan_backward_lds(plan);
    const int by_lds = lds ? (int)std::min<size_t>(16, cgnet::kMaxLds / lds) : 16;
    // register budgets: the hybrid kernel 64 or 80 registers with eight waves per group, the unit kernel 128 with four
    const int by_regs = !plan->bwd_fast ? 8 : plan->bwd_hybrid ? std::max(2, std::min(4, plan->bwd_hyb_groups)) : 4;
    return std::max(1, std::min(by_lds, by_regs));
}

extern "C" size_t cgnet_cg_plan_backward_lds(const cgnet_cg_plan* plan) {
    if (!plan) return 0;
    return plan->bwd_fast ? plan->bwd_fast_lds : plan->bwd_lds;
}

extern "C" int cgnet_cg_plan_channels(const cgnet_cg_plan* plan, int* h_t_FF, int* h_t_offsets) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    if (h_t_FF) std::copy(plan->t_FF.begin(), plan->t_FF.end(), h_t_FF);
    if (h_t_offsets) std::copy(plan->t_off.begin(), plan->t_off.end(), h_t_offsets);
    return CGNET_OK;
}

int cgnet::cg_launch_forward(const cgnet_cg_plan* p, const float* d_F, float* d_FF, const float* d_CG, int B,
                          double* d_part, int spg, hipStream_t s, const CgTask* d_tasks, int nFF, int sumT) {
    if (!d_tasks) {
        d_tasks = p->d_fwd_tasks;
        nFF = p->nFF;
        sumT = p->sumT;
    }
    const int ntasks = (int)p->fwd_tasks.size();
    if (ntasks == 0 || B == 0) return CGNET_OK;
    const int ngroups = (B + spg - 1) / spg;
    CGNET_REQUIRE((long long)ntasks * ngroups < (1LL << 31), CGNET_ERR_UNSUPPORTED,
                  "%d tasks x %d sample groups exceed the grid limit", ntasks, ngroups);
    for (size_t k = 0; k + 1 < p->fwd_class_begin.size(); ++k) {
        const int t0 = p->fwd_class_begin[k], nt = p->fwd_class_begin[k + 1] - t0;
        if (p->fwd_mm) {
            CGNET_LAUNCH(cg_forward_mm_kernel, dim3((unsigned)(nt * ngroups)), dim3(kFwdMmThreads), p->fwd_class_lds[k], s,
                         (const float2*)d_F, (float2*)d_FF, d_CG, d_tasks + t0, p->nF, nFF, B, spg, d_part, sumT,
                         (int)p->fwd_class_lds[k]);
        } else {
            CGNET_LAUNCH(cg_forward_kernel, dim3((unsigned)(nt * ngroups)), dim3(kThreads), p->fwd_class_lds[k], s,
                         (const float2*)d_F, (float2*)d_FF, d_CG, d_tasks + t0, p->nF, nFF, B, spg, d_part, sumT);
        }
        CGNET_HIP(hipGetLastError());
    }
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
    return cg_launch_forward(plan, d_F, d_FF, d_CG, B, nullptr, spg, (hipStream_t)stream);
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
        // a fill kernel, not hipMemsetAsync: the call may be recorded into a graph
        const int n2 = 2 * plan->sumT;
        CGNET_LAUNCH(fill_zero_f64_kernel, dim3((n2 + 255) / 256), dim3(256), 0, s, d_sums, n2);
        CGNET_HIP(hipGetLastError());
        return CGNET_OK;
    }
    CGNET_REQUIRE(d_F && d_FF && d_CG, CGNET_ERR_ARG, "null device pointer");
    const size_t need = cgnet_sparse_forward_stats_workspace(plan, B);
    CGNET_REQUIRE(d_workspace && workspace_bytes >= need, CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    const int spg = samples_per_group_for(B, (int)plan->fwd_tasks.size());
    const int ngroups = (B + spg - 1) / spg;
    int rc = cg_launch_forward(plan, d_F, d_FF, d_CG, B, (double*)d_workspace, spg, s);
    if (rc != CGNET_OK) return rc;
    const int n2 = 2 * plan->sumT;
    CGNET_LAUNCH(stats_reduce_kernel, dim3((n2 + 255) / 256), dim3(256), 0, s,
                       (const double*)d_workspace, d_sums, n2, ngroups);
    CGNET_HIP(hipGetLastError());
    return CGNET_OK;
}

extern "C" size_t cgnet_sparse_forward_stats_static_limit(void) { return kStaticScratchBytes; }

extern "C" int cgnet_sparse_forward_stats_static(const cgnet_cg_plan* plan, const float* d_F, float* d_FF,
                                                 const float* d_CG, int B, double* d_sums, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (plan->sumT == 0) return CGNET_OK;
    CGNET_REQUIRE(d_sums, CGNET_ERR_ARG, "d_sums is NULL");
    hipStream_t s = (hipStream_t)stream;
    const int n2 = 2 * plan->sumT;
    if (B == 0 || plan->nFF == 0) {
        // a fill kernel, not a memset: the call may be recorded into a graph
        CGNET_LAUNCH(fill_zero_f64_kernel, dim3((n2 + 255) / 256), dim3(256), 0, s, d_sums, n2);
        CGNET_HIP(hipGetLastError());
        return CGNET_OK;
    }
    CGNET_REQUIRE(d_F && d_FF && d_CG, CGNET_ERR_ARG, "null device pointer");
    const size_t need = cgnet_sparse_forward_stats_workspace(plan, B);
    CGNET_REQUIRE(need <= kStaticScratchBytes, CGNET_ERR_UNSUPPORTED,
                  "the partial statistics of this call need %zu bytes, the static area holds %zu "
                  "(use cgnet_sparse_forward_stats with a caller workspace)", need, kStaticScratchBytes);
    void* area = resolve_static_scratch();   // resolved when the plan was created on this device; a lookup here
    if (!area) return CGNET_ERR_HIP;         // resolve_static_scratch has recorded the message
    const int spg = samples_per_group_for(B, (int)plan->fwd_tasks.size());
    const int ngroups = (B + spg - 1) / spg;
    // every partial sum [group][channel][2] of this call is written by the product kernel before the
    // reduction reads it, so what an earlier call left in the area needs no clearing
    int rc = cg_launch_forward(plan, d_F, d_FF, d_CG, B, (double*)area, spg, s);
    if (rc != CGNET_OK) return rc;
    CGNET_LAUNCH(stats_reduce_kernel, dim3((n2 + 255) / 256), dim3(256), 0, s, (const double*)area, d_sums, n2, ngroups);
    CGNET_HIP(hipGetLastError());
    return CGNET_OK;
}

extern "C" size_t cgnet_sparse_backward_workspace(const cgnet_cg_plan* plan, int B) {
    if (!plan || B <= 0) return 0;
    if (plan->bwd_fast)
        return align_up(sizeof(float) * 2 * (size_t)plan->nF * B, 256) +
               align_up(sizeof(float) * 2 * (size_t)plan->bwd_P2 * B, 256) +
               align_up(sizeof(float) * 2 * (size_t)plan->bwd_nFp * B, 256) +
               align_up(sizeof(float) * (size_t)plan->bwd_cgp_len, 256);
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
        // no triple contributes: the gradient is zero (a fill kernel, not hipMemsetAsync: the call may be recorded
        // into a graph)
        const size_t nf = 2 * (size_t)plan->nF * B;
        CGNET_LAUNCH(fill_zero_f32_kernel, dim3((unsigned)std::min<size_t>((nf + 255) / 256, 4096)), dim3(256), 0, s, d_gF, nf);
        CGNET_HIP(hipGetLastError());
        return CGNET_OK;
    }
    CGNET_REQUIRE(d_F && d_gFF && d_CG, CGNET_ERR_ARG, "null device pointer");
    const int ng = bwd_groups_for(plan, B);
    const size_t need = cgnet_sparse_backward_workspace(plan, B);
    CGNET_REQUIRE(need == 0 || (d_workspace && workspace_bytes >= need), CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    if (plan->bwd_fast) {
        float2* part1 = (float2*)d_workspace;
        float2* part2 = (float2*)((char*)part1 + align_up(sizeof(float) * 2 * (size_t)plan->nF * B, 256));
        float2* Fp = (float2*)((char*)part2 + align_up(sizeof(float) * 2 * (size_t)plan->bwd_P2 * B, 256));
        float* CGP = (float*)((char*)Fp + align_up(sizeof(float) * 2 * (size_t)plan->bwd_nFp * B, 256));
        CGNET_REQUIRE(((uintptr_t)d_workspace & 15) == 0, CGNET_ERR_ARG, "workspace must be 16-byte aligned");
        const size_t npad = (size_t)plan->bwd_nFp * B;
        const int nbF = (int)((npad + 255) / 256);
        CGNET_LAUNCH(cg_backward_pad_kernel, dim3((unsigned)(nbF + plan->nllls)), dim3(256), 0, s,
                     (const float2*)d_F, d_CG, Fp, CGP, plan->d_bwd_padmeta, plan->L, plan->nF, plan->bwd_nFp, B, nbF);
        CGNET_HIP(hipGetLastError());
        CGNET_REQUIRE((long long)B * (long long)plan->bwd_units.size() < (1LL << 31), CGNET_ERR_UNSUPPORTED,
                      "%d samples x %zu units exceed the grid limit", B, plan->bwd_units.size());
        if (plan->bwd_hybrid && plan->bwd_hyb_groups == 4) {
            CGNET_LAUNCH(cg_backward_hybrid_kernel<true>, dim3((unsigned)(B * plan->bwd_units.size())), dim3(kHybThreads),
                         plan->bwd_fast_lds, s, (const float2*)Fp, (const float2*)d_gFF, (const float*)CGP, part1, part2,
                         plan->d_bwd_units, plan->d_bwd_utasks, plan->nF, plan->bwd_nFp, plan->nFF, plan->bwd_P2,
                         plan->bwd_f1cap, plan->bwd_f2cap, plan->bwd_cgcap, plan->bwd_tcap, B);
        } else if (plan->bwd_hybrid) {
            CGNET_LAUNCH(cg_backward_hybrid_kernel<false>, dim3((unsigned)(B * plan->bwd_units.size())), dim3(kHybThreads),
                         plan->bwd_fast_lds, s, (const float2*)Fp, (const float2*)d_gFF, (const float*)CGP, part1, part2,
                         plan->d_bwd_units, plan->d_bwd_utasks, plan->nF, plan->bwd_nFp, plan->nFF, plan->bwd_P2,
                         plan->bwd_f1cap, plan->bwd_f2cap, plan->bwd_cgcap, plan->bwd_tcap, B);
        } else {
            CGNET_LAUNCH(cg_backward_unit_kernel, dim3((unsigned)(B * plan->bwd_units.size())), dim3(kThreads),
                         plan->bwd_fast_lds, s, (const float2*)Fp, (const float2*)d_gFF, (const float*)CGP, part1, part2,
                         plan->d_bwd_units, plan->d_bwd_utasks, plan->nF, plan->bwd_nFp, plan->nFF, plan->bwd_P2,
                         plan->bwd_f1cap, plan->bwd_f2cap, plan->bwd_cgcap, plan->bwd_tcap, B);
        }
        CGNET_HIP(hipGetLastError());
        const size_t n = (size_t)plan->nF * B;
        CGNET_LAUNCH(cg_backward_combine_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                     (const float2*)part1, (const float2*)part2, (float2*)d_gF, plan->d_bwd_combine, plan->L,
                     plan->nF, plan->bwd_P2, B);
        CGNET_HIP(hipGetLastError());
        return CGNET_OK;
    }
    CGNET_REQUIRE(plan->bwd_general_ok, CGNET_ERR_UNSUPPORTED,
                  "backward needs %zu bytes of LDS (limit %zu): too many input channels for this lmax; the plan serves "
                  "the forward only", plan->bwd_lds, kMaxLds);
    const int* d_gb = plan->d_bwd_group_table + plan->bwd_group_table_off[ng];
    float2* dst = ng > 1 ? (float2*)d_workspace : (float2*)d_gF;
    CGNET_LAUNCH(cg_backward_kernel, dim3(ng, B), dim3(plan->bwd_threads), plan->bwd_lds, s,
                       (const float2*)d_F, (const float2*)d_gFF, d_CG, dst, plan->d_bwd_tasks, d_gb,
                       plan->nF, plan->nFF, B);
    CGNET_HIP(hipGetLastError());
    if (ng > 1) {
        const size_t n = (size_t)plan->nF * B;
        CGNET_LAUNCH(partial_sum_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                           (const float2*)d_workspace, (float2*)d_gF, n, ng);
        CGNET_HIP(hipGetLastError());
    }
    return CGNET_OK;
}

// ---- fused layer backward: host side -----------------------------------------------------------
namespace cgnet {

void free_fused_link(FusedLink* link) {
    if (!link) return;
    void* ptrs[] = {link->d_gens, link->d_ftasks, link->d_packmap, link->d_bmap};
    for (void* q : ptrs)
        if (q) (void)hipFree(q);
    *link = FusedLink();
}

int build_fused_link(const cgnet_cg_plan* p, const cgnet_wmm_plan* w, FusedLink* link) {
    *link = FusedLink();
    CGNET_REQUIRE(wmm_plan_degrees(w) == p->L + 1, CGNET_ERR_ARG, "the two plans have different lmax");
    std::vector<WmmDegInfo> info(p->L + 1);
    for (int l = 0; l <= p->L; ++l) {
        if (int rc = wmm_plan_degree(w, l, &info[l])) return rc;
        CGNET_REQUIRE(info[l].K == p->t_FF[l], CGNET_ERR_ARG,
                      "degree %d: the mixing plan has %d mid channels, the product %d", l, info[l].K, p->t_FF[l]);
    }
    link->nO = info[p->L].cumO + info[p->L].tO * (2 * p->L + 1);
    CGNET_REQUIRE(p->bwd_fast && p->bwd_hybrid, CGNET_ERR_UNSUPPORTED,
                  "the fused backward needs the matrix-core unit backward (every channel count in 8..16, lmax <= 23)");
    CGNET_REQUIRE(wmm_gradff_operand_ok(w), CGNET_ERR_UNSUPPORTED, "the fused backward needs t_O <= 16 in every degree");
    // packed B operand of one sample: per degree nct x nks blocks of 64 floats
    std::vector<int> boff(p->L + 1, 0), bmap;
    int bop = 0, bcap = 16;
    for (int l = 0; l <= p->L; ++l) {
        const int M = 2 * l + 1, nct = (2 * M + 15) / 16, nks = info[l].tO > 0 ? (2 * info[l].tO + 3) / 4 : 0;
        boff[l] = bop;
        if (p->t_FF[l] == 0) continue;
        for (int ct = 0; ct < nct; ++ct)
            for (int ks = 0; ks < nks; ++ks) {
                const int v[4] = {info[l].cumO, M, info[l].tO, ct | (ks << 8)};
                bmap.insert(bmap.end(), v, v + 4);
            }
        bop += nct * nks * 64;
        bcap = std::max(bcap, nct * nks * 256);
    }
    bool fold = true;        // CGNET_DIAG_FOLD=0: diagonal triples take both slots like all others
    if (const char* e = getenv("CGNET_DIAG_FOLD"); e && e[0] == '0') fold = false;
    std::vector<GenTask> gens(p->bwd_utasks.size());
    std::vector<FusedTask> ft(p->bwd_utasks.size());
    std::vector<int> map;
    size_t aoff = 0;
    int acap = 16;
    for (const BwdUnit& u : p->bwd_units) {
        for (int k = u.task_begin; k < u.task_end; ++k) {
            const BwdUTask& t = p->bwd_utasks[k];
            const WmmDegInfo& d = info[t.l];
            const int M = 2 * t.l + 1, nct = (2 * M + 15) / 16;
            GenTask g{};
            g.aoff = (int)aoff;
            g.nks = d.tO > 0 ? (2 * d.tO + 3) / 4 : 0;
            g.tO = d.tO;
            g.chan0 = (t.offFF - p->cumFF[t.l]) / M;
            g.nch = u.rows * t.tau2;
            g.cumW = d.cumW;
            g.K = d.K;
            g.cumT = d.cumT;
            // Diagonal triple (l1 == l2) whose unit holds all rows: the tile g[t1][t2] and its mirror g[t2][t1] feed the
            // same gradient, slot2(g) = slot1((-1)^l g^T) (the table is (-1)^l-symmetric under m1 <-> m2), so the
            // weights are packed symmetrised, W'[to][(t1,t2)] = W[to][(t1,t2)]/div + (-1)^l W[to][(t2,t1)]/div', the tile
            // made from them is g + (-1)^l g^T, and one slot's worth of arithmetic on it gives both slots' sum: the
            // vector waves reduce over the first 4 c0 channels (slot-1 form), the matrix waves over the others (slot-2
            // form), instead of each over all.
            const int nk = (u.rows + 3) / 4;
            const bool diag = fold && t.l2 == u.l1 && u.rows == p->t_F[u.l1] && nk >= 2;   // the same for a whole run of equal l2
            const int c0 = diag ? CGNET_DIAG_C0(nk) : 0;
            g.sym = diag ? ((t.l & 1) ? -u.rows : u.rows) : 0;
            gens[k] = g;
            const int nrt = (g.nch + 15) / 16;
            for (int rt = 0; rt < nrt && g.nks > 0; ++rt) { map.push_back(k); map.push_back(rt); }
            FusedTask f{};
            f.geom = t.l | (t.l2 << 8) | (t.tau2 << 16) | (t.first_of_l2 << 24) | (t.last_of_l2 << 25) | (c0 << 26);
            f.offF2p = t.offF2p;
            f.cgp_off = t.cgp_off;
            f.cgp_len = t.cgp_len;
            f.p2off = t.p2off;
            f.aoff = g.aoff;
            f.shape = g.nks | (d.tO << 8) | (g.nch << 16);
            f.boff = boff[t.l];
            const int nkp = (g.nks + 1) / 2;
            f.chunks = (nrt * 32 * nkp) | ((nct * g.nks * 16) << 16);     // 16-byte pieces of the A block | of the B block
            ft[k] = f;
            aoff += (size_t)nrt * 128 * nkp;
            CGNET_REQUIRE(aoff < (1u << 30), CGNET_ERR_UNSUPPORTED, "packed weights of the fused backward exceed 2^30 floats");
            acap = std::max(acap, nrt * 512 * nkp);
        }
    }
    const size_t lds = bwd_fused_lds(p->bwd_f1cap, p->bwd_f2cap, p->bwd_cgcap, p->bwd_tcap, bcap, acap);
    CGNET_REQUIRE(lds <= kMaxHybLds, CGNET_ERR_UNSUPPORTED,
                  "the fused backward would need %zu bytes of LDS per work-group (limit %zu)", lds, kMaxHybLds);
    FusedLink tmp;
    auto upload = [](const void* src, size_t bytes, void** dst) -> int {
        if (bytes == 0) return CGNET_OK;
        CGNET_HIP(hipMalloc(dst, bytes));
        CGNET_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return CGNET_OK;
    };
    int rc = upload(gens.data(), sizeof(GenTask) * gens.size(), (void**)&tmp.d_gens);
    if (!rc) rc = upload(ft.data(), sizeof(FusedTask) * ft.size(), (void**)&tmp.d_ftasks);
    if (!rc) rc = upload(map.data(), sizeof(int) * map.size(), (void**)&tmp.d_packmap);
    if (!rc) rc = upload(bmap.data(), sizeof(int) * bmap.size(), (void**)&tmp.d_bmap);
    if (!rc) rc = raise_dynamic_lds((const void*)cgbn_backward_fused_kernel, lds);
    if (rc) {
        free_fused_link(&tmp);
        return rc;
    }
    tmp.npack = (int)(map.size() / 2);
    tmp.nbmap = (int)(bmap.size() / 4);
    tmp.operand_floats = aoff;
    tmp.bop_floats = bop;
    tmp.bcap = bcap;
    tmp.acap = acap;
    tmp.nO = link->nO;
    tmp.lds = lds;
    tmp.ok = true;
    *link = tmp;
    return CGNET_OK;
}

BwdAreas bwd_areas(const cgnet_cg_plan* p, int B) {
    BwdAreas a{};
    size_t o = 0;
    a.part1 = o; o += align_up(sizeof(float) * 2 * (size_t)p->nF * B, 256);
    a.part2 = o; o += align_up(sizeof(float) * 2 * (size_t)p->bwd_P2 * B, 256);
    a.Fp = o;    o += align_up(sizeof(float) * 2 * (size_t)p->bwd_nFp * B, 256);
    a.CGP = o;   o += align_up(sizeof(float) * (size_t)p->bwd_cgp_len, 256);
    a.total = o;
    return a;
}

int launch_backward_pad(const cgnet_cg_plan* plan, const float* d_F, const float* d_CG, float* d_Fp, float* d_CGP, int B,
                        hipStream_t s) {
    const size_t npad = (size_t)plan->bwd_nFp * B;
    const int nbF = (int)((npad + 255) / 256);
    CGNET_LAUNCH(cg_backward_pad_kernel, dim3((unsigned)(nbF + plan->nllls)), dim3(256), 0, s,
                 (const float2*)d_F, d_CG, (float2*)d_Fp, d_CGP, plan->d_bwd_padmeta, plan->L, plan->nF, plan->bwd_nFp, B, nbF);
    CGNET_HIP(hipGetLastError());
    return CGNET_OK;
}

int launch_pack_w_gen(const FusedLink& link, const float* d_W, const float* d_stds, float eps, float* d_Ag, hipStream_t s) {
    if (link.npack > 0) {
        CGNET_LAUNCH(pack_w_gen_kernel, dim3((unsigned)link.npack), dim3(64), 0, s, (const float2*)d_W, d_stds, eps,
                     link.d_gens, link.d_packmap, d_Ag);
        CGNET_HIP(hipGetLastError());
    }
    return CGNET_OK;
}

int launch_fused_backward(const cgnet_cg_plan* plan, const FusedLink& link, const float* d_gO, const float* d_Ag,
                          const float* d_Fp, const float* d_CGP, float* d_Bg, float* d_part1, float* d_part2,
                          float* d_gF, int B, hipStream_t s) {
    CGNET_REQUIRE(link.ok, CGNET_ERR_UNSUPPORTED, "the fused backward does not take this pair of plans");
    CGNET_REQUIRE(B <= 65535, CGNET_ERR_UNSUPPORTED, "B=%d above 65535", B);
    CGNET_REQUIRE((long long)B * (long long)plan->bwd_units.size() < (1LL << 31), CGNET_ERR_UNSUPPORTED,
                  "%d samples x %zu units exceed the grid limit", B, plan->bwd_units.size());
    if (link.nbmap > 0) {
        CGNET_LAUNCH(pack_go_gen_kernel, dim3((unsigned)link.nbmap, (unsigned)B), dim3(64), 0, s,
                     (const float2*)d_gO, link.d_bmap, d_Bg, link.nO, link.bop_floats);
        CGNET_HIP(hipGetLastError());
    }
    CGNET_LAUNCH(cgbn_backward_fused_kernel, dim3((unsigned)(B * plan->bwd_units.size())), dim3(kHybThreads), link.lds, s,
                 (const float2*)d_Fp, (const float*)d_Bg, d_Ag, d_CGP, (float2*)d_part1, (float2*)d_part2,
                 plan->d_bwd_units, link.d_ftasks, plan->nF, plan->bwd_nFp, link.bop_floats, plan->bwd_P2,
                 plan->bwd_f1cap, plan->bwd_f2cap, plan->bwd_cgcap, plan->bwd_tcap, link.bcap, link.acap, B);
    CGNET_HIP(hipGetLastError());
    const size_t n = (size_t)plan->nF * B;
    CGNET_LAUNCH(cg_backward_combine_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                 (const float2*)d_part1, (const float2*)d_part2, (float2*)d_gF, plan->d_bwd_combine, plan->L,
                 plan->nF, plan->bwd_P2, B);
    CGNET_HIP(hipGetLastError());
    return CGNET_OK;
}

}  // namespace cgnet

// ---- fused inference forward: host side -------------------------------------------------------------
namespace cgnet {

void free_fwd_link(FwdLink* link) {
    if (!link) return;
    void* ptrs[] = {link->d_mix, link->d_packmap, link->d_red, link->d_sel};
    for (void* q : ptrs)
        if (q) (void)hipFree(q);
    *link = FwdLink();
}

int build_fwd_link(const cgnet_cg_plan* p, const cgnet_wmm_plan* w, FwdLink* link) {
    *link = FwdLink();
    CGNET_REQUIRE(wmm_plan_degrees(w) == p->L + 1, CGNET_ERR_ARG, "the two plans have different lmax");
    std::vector<WmmDegInfo> info(p->L + 1);
    for (int l = 0; l <= p->L; ++l)
        if (int rc = wmm_plan_degree(w, l, &info[l])) return rc;
    CGNET_REQUIRE(p->fwd_mm, CGNET_ERR_UNSUPPORTED,
                  "the fused inference forward needs the matrix-core product (every channel count in 8..16)");
    CGNET_REQUIRE(p->L <= 15, CGNET_ERR_UNSUPPORTED, "the fused inference forward takes lmax <= 15 (two column tiles of 16 values of m)");
    for (int l = 0; l <= p->L; ++l)
        CGNET_REQUIRE(info[l].tO <= 16, CGNET_ERR_UNSUPPORTED, "the fused inference forward needs t_O <= 16 in every degree");
    const int nt = (int)p->fwd_tasks.size();
    std::vector<FwdMixTask> mix(nt);
    std::vector<int> map;
    std::vector<std::vector<std::pair<int, int>>> per_l(p->L + 1);       // (first channel, ooff) of every task of a degree
    size_t aoff = 0;
    int ooff = 0;
    for (int k = 0; k < nt; ++k) {
        const CgTask& t = p->fwd_tasks[k];
        const WmmDegInfo& d = info[t.l];
        const int nch = t.rows * t.tau2, M = 2 * t.l + 1;
        CGNET_REQUIRE(nch <= 4 * 64, CGNET_ERR_UNSUPPORTED, "a product tile of %d channels exceeds the mixing registers", nch);
        FwdMixTask g{};
        g.aoff = (int)aoff;
        g.nks = d.tO > 0 ? (nch + 3) / 4 : 0;
        g.tO = d.tO;
        g.ooff = ooff;
        g.cumW = d.cumW;
        g.K = d.K;
        g.c0 = t.chan0 - p->cumT[t.l];
        g.cumT = d.cumT;
        mix[k] = g;
        for (int ks = 0; ks < g.nks; ++ks) { map.push_back(k); map.push_back(ks); }
        aoff += (size_t)g.nks * 128;
        CGNET_REQUIRE(aoff < (1u << 30), CGNET_ERR_UNSUPPORTED, "packed weights of the fused forward exceed 2^30 floats");
        if (d.tO > 0) per_l[t.l].push_back(std::make_pair(g.c0, ooff));
        ooff += d.tO * M;
    }
    std::vector<int> red;
    for (int l = 0; l <= p->L; ++l) red.push_back(info[l].cumO);
    const int nO = info[p->L].cumO + info[p->L].tO * (2 * p->L + 1);
    red.push_back(nO);
    for (int l = 0; l <= p->L; ++l) red.push_back(info[l].tO);
    int run = 0;
    for (int l = 0; l <= p->L; ++l) { red.push_back(run); run += (int)per_l[l].size(); }
    red.push_back(run);
    for (int l = 0; l <= p->L; ++l) {
        std::sort(per_l[l].begin(), per_l[l].end());                      // channel order: the order the mixing kernel adds in
        for (const auto& e : per_l[l]) red.push_back(e.second);
    }
    FwdLink tmp;
    auto upload = [](const void* src, size_t bytes, void** dst) -> int {
        if (bytes == 0) return CGNET_OK;
        CGNET_HIP(hipMalloc(dst, bytes));
        CGNET_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return CGNET_OK;
    };
    int rc = upload(mix.data(), sizeof(FwdMixTask) * mix.size(), (void**)&tmp.d_mix);
    if (!rc) rc = upload(map.data(), sizeof(int) * map.size(), (void**)&tmp.d_packmap);
    if (!rc) rc = upload(red.data(), sizeof(int) * red.size(), (void**)&tmp.d_red);
    // one launch per (LDS class, number of column tiles of 16 values of m), over the class's tasks of that kind in the
    // class's order (by work)
    std::vector<int> sel;
    size_t lds_max[3] = {0, 0, 0};
    for (size_t k = 0; k + 1 < p->fwd_class_begin.size(); ++k)
        for (int T = 1; T <= 2; ++T) {
            FwdLaunch fl{};
            fl.T = T;
            fl.sel0 = (int)sel.size();
            for (int i = p->fwd_class_begin[k]; i < p->fwd_class_begin[k + 1]; ++i)
                if ((2 * p->fwd_tasks[i].l + 1 + 15) / 16 == T) sel.push_back(i);
            fl.n = (int)sel.size() - fl.sel0;
            fl.lds = p->fwd_class_lds[k] + mix_red_bytes(T);
            if (fl.n == 0) continue;
            lds_max[T] = std::max(lds_max[T], fl.lds);
            tmp.launches.push_back(fl);
        }
    if (!rc) rc = upload(sel.data(), sizeof(int) * sel.size(), (void**)&tmp.d_sel);
    if (!rc && std::max(lds_max[1], lds_max[2]) > kMaxLds) {
        set_error("the fused inference forward would need %zu bytes of LDS per work-group (limit %zu)",
                  std::max(lds_max[1], lds_max[2]), kMaxLds);
        rc = CGNET_ERR_UNSUPPORTED;
    }
    if (!rc && lds_max[1]) rc = raise_dynamic_lds((const void*)cgbn_forward_fused_kernel<1>, lds_max[1]);
    if (!rc && lds_max[2]) rc = raise_dynamic_lds((const void*)cgbn_forward_fused_kernel<2>, lds_max[2]);
    if (rc) {
        free_fwd_link(&tmp);
        return rc;
    }
    tmp.npack = (int)(map.size() / 2);
    tmp.a_floats = aoff;
    tmp.opart = ooff;
    tmp.nO = nO;
    tmp.L = p->L;
    tmp.ok = true;
    *link = tmp;
    return CGNET_OK;
}

// the tasks' packed weights: four (task, k-step) blocks of 64 lanes per work-group
__global__ void __launch_bounds__(256)
pack_w_mix_kernel(const float2* __restrict__ W, const float* __restrict__ stds, float eps, const CgTask* __restrict__ tasks,
                  const FwdMixTask* __restrict__ mix, const int* __restrict__ map, int npack, float* __restrict__ Af) {
    const int pair = (int)blockIdx.x * 4 + (int)(threadIdx.x >> 6);
    if (pair >= npack) return;
    const int k = map[2 * pair];
    pack_w_mix_lane(W, stds, eps, mix[k], tasks[k].rows * tasks[k].tau2, map[2 * pair + 1], threadIdx.x & 63, Af);
}

int launch_pack_w_mix(const cgnet_cg_plan* p, const FwdLink& link, const float* d_W, const float* d_stds, float eps, float* d_Af,
                      hipStream_t s) {
    if (link.npack > 0) {
        CGNET_LAUNCH(pack_w_mix_kernel, dim3((unsigned)((link.npack + 3) / 4)), dim3(256), 0, s, (const float2*)d_W, d_stds, eps,
                     p->d_fwd_tasks, link.d_mix, link.d_packmap, link.npack, d_Af);
        CGNET_HIP(hipGetLastError());
    }
    return CGNET_OK;
}

int launch_forward_fused(const cgnet_cg_plan* p, const FwdLink& link, const float* d_F, const float* d_CG, const float* d_Af,
                         float* d_Opart, float* d_O, int B, hipStream_t s) {
    CGNET_REQUIRE(link.ok, CGNET_ERR_UNSUPPORTED, "the fused inference forward does not take this pair of plans");
    const int ntasks = (int)p->fwd_tasks.size();
    const int spg = samples_per_group_for(B, ntasks);
    const int ngroups = (B + spg - 1) / spg;
    CGNET_REQUIRE((long long)ntasks * ngroups < (1LL << 31), CGNET_ERR_UNSUPPORTED,
                  "%d tasks x %d sample groups exceed the grid limit", ntasks, ngroups);
    for (const FwdLaunch& fl : link.launches) {
        if (fl.T == 1) {
            CGNET_LAUNCH(cgbn_forward_fused_kernel<1>, dim3((unsigned)(fl.n * ngroups)), dim3(kFwdMmThreads), fl.lds, s,
                         (const float2*)d_F, d_CG, p->d_fwd_tasks, link.d_mix, link.d_sel + fl.sel0, d_Af, (float2*)d_Opart,
                         p->nF, B, spg, link.opart, (int)fl.lds);
        } else {
            CGNET_LAUNCH(cgbn_forward_fused_kernel<2>, dim3((unsigned)(fl.n * ngroups)), dim3(kFwdMmThreads), fl.lds, s,
                         (const float2*)d_F, d_CG, p->d_fwd_tasks, link.d_mix, link.d_sel + fl.sel0, d_Af, (float2*)d_Opart,
                         p->nF, B, spg, link.opart, (int)fl.lds);
        }
        CGNET_HIP(hipGetLastError());
    }
    const size_t n = (size_t)link.nO * B;
    if (n > 0) {
        CGNET_LAUNCH(cgbn_forward_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (const float2*)d_Opart,
                     (float2*)d_O, link.d_red, link.L, link.nO, link.opart, B);
        CGNET_HIP(hipGetLastError());
    }
    return CGNET_OK;
}

}  // namespace cgnet
