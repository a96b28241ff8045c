// Fragment norm + per-degree complex channel mixing, forward and backward, for gfx950.
//
// The mixing of one degree l is a tall-skinny complex matrix product
//     O[b, to, m] = sum_c  W[to, c] / div[c] * FF[b, c, m]        (t_O x t_FF) . (t_FF x (2l+1))
// bounded by the one pass over FF.  It runs on the fp32 matrix cores as a real product with
// twice the rows:  P = [W_re; W_im] . X  where X is FF with (re, im) as adjacent real columns;
// then O_re = P_re-rows[re col] - P_im-rows[im col],  O_im = P_re-rows[im col] + P_im-rows[re col].
//
// v_mfma_f32_16x16x4_f32 operand layout (lane = 0..63): A[i][k] and B[k][j] sit in lane 16*k + i
// (resp. 16*k + j); D[4*(lane/16) + v][lane%16] is register v of the lane.  The k slots and the
// column slots of a tile can be assigned to memory freely as long as both operands agree, which
// is used here so that every lane reads whole complex numbers (8-byte loads):
//   forward : lane (k-slot kk, col-slot i) owns complex columns 2i and 2i+1 of a 32-column
//             chunk; their (re, im) parts feed four column tiles.
//   grad W  : the contraction runs over (b, m, re/im); lane (kk, i) reads complex entries
//             8*blk + 2*kk, +1 of channel row i and feeds four k-steps.
#include <algorithm>
#include <memory>
#include <vector>

#include "internal.h"

namespace cgnet {
namespace {

constexpr int kThreads = 256;
constexpr int kStatTileBytes = 32 * 1024;
constexpr int kStatGroups = 8;
constexpr int kGradWChunk = 32;     // samples whose weight-gradient sums one work-group forms, at most (the chunks of a
                                    // batch are made equal: 100 samples are four chunks of 25, not 32 + 32 + 32 + 4)
constexpr int kGradWFold = 1;       // samples per matrix-core chain inside a chunk

// --------------------------------------------------------------------------- statistics
// sums of |z| and |z|^2 over (b, m) per mid channel, from FF
__global__ void __launch_bounds__(kThreads)
fn_stats_kernel(const float2* __restrict__ FF, const WmmDeg* __restrict__ degs,
                const WmmChanUnit* __restrict__ units, int nFF, int B, int samples_per_group,
                double* __restrict__ part, int sumT) {
    extern __shared__ __align__(16) unsigned char smem[];
    float2* tile = reinterpret_cast<float2*>(smem);
    const UnitPart up = part_major((B + samples_per_group - 1) / samples_per_group);
    const WmmChanUnit u = units[up.unit];
    const WmmDeg d = degs[u.deg];
    const int n = u.nc * d.M;
    const int tid = threadIdx.x;
    double s1 = 0., s2 = 0.;
    const int b0 = up.part * samples_per_group, b1 = min(B, b0 + samples_per_group);
    for (int b = b0; b < b1; ++b) {
        const float2* src = FF + (size_t)b * nFF + d.cumFF + (size_t)u.c0 * d.M;
        for (int e = tid; e < n; e += kThreads) tile[e] = src[e];
        __syncthreads();
        if (tid < u.nc) {
            // both sums run over the same rounded |z| in double (no cancellation between
            // inconsistently rounded terms when the variance is formed)
            for (int mm = 0; mm < d.M; ++mm) {
                const float2 z = tile[tid * d.M + mm];
                const double r = (double)sqrtf(fmaf(z.x, z.x, z.y * z.y));
                s1 += r;
                s2 = fma(r, r, s2);
            }
        }
        __syncthreads();
    }
    if (tid < u.nc) {
        double* p = part + ((size_t)up.part * sumT + d.cumT + u.c0 + tid) * 2;
        p[0] = s1;
        p[1] = s2;
    }
}

__global__ void __launch_bounds__(256)
fn_sum_groups_kernel(const double* __restrict__ part, double* __restrict__ sums, int n2, int ngroups) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n2) return;
    double s = 0.;
    for (int g = 0; g < ngroups; ++g) s += part[(size_t)g * n2 + i];
    sums[i] = s;
}

// stds[c] <- stds[c] * cnt/(cnt+1) + std_batch[c] / (cnt+1)
__global__ void __launch_bounds__(256)
fn_update_std_kernel(const double* __restrict__ sums, float* __restrict__ stds,
                     const WmmDeg* __restrict__ degs, int ndeg, int sumT, int B, float cnt) {
    __shared__ int s_tab[kMaxLookup];
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int di = lookup_in_group(ndeg, c, [&](int k) { return degs[k].cumT; }, s_tab);
    if (c >= sumT) return;
    stds[c] = updated_std(stds[c], sums[2 * c], sums[2 * c + 1], (double)B * (double)degs[di].M, cnt);
}

// --------------------------------------------------------------------------- weight packing
// Forward operand (layout: pack_w_forward_thread): one thread writes the four floats of one lane.
__global__ void __launch_bounds__(256)
pack_w_forward_kernel(const float2* __restrict__ W, const float* __restrict__ stds, float eps,
                      const WmmDeg* __restrict__ degs, int ndeg, float* __restrict__ Wp, int total_blocks) {
    __shared__ int s_tab[kMaxLookup];
    pack_w_forward_thread(W, stds, eps, degs, ndeg, Wp, total_blocks, blockIdx.x * blockDim.x + threadIdx.x, s_tab);
}

// Backward operand: WT[cumW + c*tO + to] = conj(W[to][c]) / div[c]
__global__ void __launch_bounds__(256)
pack_w_backward_kernel(const float2* __restrict__ W, const float* __restrict__ stds, float eps,
                       const WmmDeg* __restrict__ degs, int ndeg, float2* __restrict__ WT, int nW) {
    __shared__ int s_tab[kMaxLookup];
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int di = lookup_in_group(ndeg, idx, [&](int k) { return degs[k].cumW; }, s_tab);
    if (idx >= nW) return;
    const WmmDeg d = degs[di];
    const int rel = idx - d.cumW;
    const int c = rel / d.tO, to = rel % d.tO;
    float2 w = W[d.cumW + (size_t)to * d.K + c];
    float r = 1.f;
    if (stds) r = fmaxf(eps, stds[d.cumT + c]);
    WT[idx] = make_float2(w.x / r, -w.y / r);
}

// --------------------------------------------------------------------------- forward (MFMA)
// Forward mixing.  Every wave works alone (no barrier in the kernel): it owns G whole samples
// of one degree (G*M complex columns in T tiles of 16) and a slice of the channels, and streams
// its samples' runs of kFwdKC channels (one contiguous run per sample) together with the
// packed weights of those channels straight from memory into a private ring of LDS stages,
// `depth` - 1 stages ahead of the arithmetic.  Loads complete in order, so "stage s has landed"
// is a vmcnt wait that leaves the younger stages in flight.
constexpr int kFwdKC = 8;        // channels per stage (two k-steps of 4)
constexpr int kFwdMaxT = 6;      // column tiles per wave (96 complex columns)
constexpr int kFwdDepth = 3;
constexpr int kFwdSlice = 256;   // channels per k-slice: short enough that the groups pack the CUs evenly

template <int T>
__device__ __forceinline__ void wmm_forward_wave(const float2* __restrict__ FF, const float* __restrict__ Wp,
                                                 float2* __restrict__ out, const WmmDeg& d, const WmmFwdUnit& u,
                                                 int B, int nFF, int nO, int b_first, unsigned char* ring, int depth,
                                                 int stage_bytes, int lane) {
    const int M = d.M;
    const int nb = min(d.G, B - b_first);
    const int i = lane & 15, kk = lane >> 4;
    const int run_cap = kFwdKC * M;                               // entries of one sample's run (64*M bytes)
    bool ok[T];
    int col_b[T], col_m[T], lofs[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int q = 16 * t + i;
        ok[t] = q < nb * M;
        col_b[t] = ok[t] ? q / M : 0;
        col_m[t] = ok[t] ? q - col_b[t] * M : 0;
        lofs[t] = col_b[t] * run_cap + kk * M + col_m[t];        // lanes past the last column read column 0
    }
    {
        // the ring starts out finite: entries a short last stage or a short last group of samples
        // never writes are multiplied by zero weights or land in columns nobody stores
        float4* z = reinterpret_cast<float4*>(ring);
        for (int e = lane; e < (depth * stage_bytes) >> 4; e += 64) z[e] = make_float4(0.f, 0.f, 0.f, 0.f);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the clearing stores precede the first copy into the ring
    }
    const int nk = u.k_end - u.k_begin;
    const int nfull = nk / kFwdKC, nstages = (nk + kFwdKC - 1) / kFwdKC;
    // A full stage is one list of 16-byte pieces, sample after sample (4*M pieces per run), that
    // lands contiguously behind the weights: piece c = lane + 64*r comes from a per-lane address
    // fixed for the whole slice plus the stage's offset.
    const int cpr = 4 * M, npieces = nb * cpr;
    const int nr = (npieces + 63) >> 6;                           // <= T copy instructions per stage
    const int ni = 1 + nr;                                        // copy instructions of a full stage
    const char* piece[T];
#pragma unroll
    for (int r = 0; r < T; ++r) {
        const int c = min(lane + 64 * r, npieces - 1);
        const int j = c / cpr, idx = c - j * cpr;
        piece[r] = reinterpret_cast<const char*>(FF + (size_t)(b_first + j) * nFF + d.cumFF + (size_t)u.k_begin * M) + 16 * idx;
    }
    const char* wpiece = reinterpret_cast<const char*>(Wp + (size_t)d.wp_base * 64 +
                                                       ((size_t)(u.k_begin >> 3) * d.nrc + u.rc) * 256) + 16 * lane;
    const size_t w_step = (size_t)d.nrc * 1024, f_step = (size_t)kFwdKC * M * 8;
    auto issue = [&](int s, int slot_idx) {
        unsigned char* slot = ring + (size_t)slot_idx * stage_bytes;
        __builtin_amdgcn_global_load_lds(wpiece + (size_t)s * w_step, (lds_void_ptr)slot, 16, 0, 0);
        if (s < nfull) {
#pragma unroll
            for (int r = 0; r < T; ++r)
                if (r < nr && lane + 64 * r < npieces)
                    __builtin_amdgcn_global_load_lds(piece[r] + (size_t)s * f_step, (lds_void_ptr)(slot + 1024 + 1024 * r), 16, 0, 0);
        } else {
            // the short last stage of a degree whose channel count is no multiple of kFwdKC
            const int k0 = u.k_begin + s * kFwdKC;
            const int n = (u.k_end - k0) * M;
            for (int j = 0; j < nb; ++j) {
                const float2* src = FF + (size_t)(b_first + j) * nFF + d.cumFF + (size_t)k0 * M;
                unsigned char* dst = slot + 1024 + (size_t)j * run_cap * 8;
                dma16<64>(src, dst, n >> 1, lane);
                if (n & 1) dma8(src + (n - 1), dst + 8 * (size_t)(n - 1), lane);
            }
        }
    };

    f32x4 acc[2][2 * T];
#pragma unroll
    for (int t = 0; t < 2 * T; ++t) {
        acc[0][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
        acc[1][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    }
    for (int s = 0; s < min(nstages, depth - 1); ++s) issue(s, s);
    int cur_slot = 0, next_slot = (depth - 1) % depth;            // ring positions of stage s and of stage s+depth-1
    for (int s = 0; s < nstages; ++s) {
        // stages s+1 .. s+depth-2 are in flight behind stage s
        const int youngest = min(s + depth - 2, nstages - 1);
        wait_vmcnt(youngest < nfull ? (youngest - s) * ni : 0);
        if (s + depth - 1 < nstages) issue(s + depth - 1, next_slot);
        const unsigned char* slot = ring + (size_t)cur_slot * stage_bytes;
        cur_slot = cur_slot + 1 == depth ? 0 : cur_slot + 1;
        next_slot = next_slot + 1 == depth ? 0 : next_slot + 1;
        const float4 a = reinterpret_cast<const float4*>(slot)[lane];   // (re, im rows) of k-step 0, of k-step 1
        const float2* cur = reinterpret_cast<const float2*>(slot + 1024);
        // channels past the end of the degree have zero weights
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            const float a0 = q ? a.z : a.x, a1 = q ? a.w : a.y;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const float2 v = cur[lofs[t] + 4 * q * M];
                acc[0][2 * t] = mfma4(a0, v.x, acc[0][2 * t]);
                acc[0][2 * t + 1] = mfma4(a0, v.y, acc[0][2 * t + 1]);
                acc[1][2 * t] = mfma4(a1, v.x, acc[1][2 * t]);
                acc[1][2 * t + 1] = mfma4(a1, v.y, acc[1][2 * t + 1]);
            }
        }
    }
    // complex outputs: the re / im columns of a complex column sit in the same lane
    float2* dst = out + (size_t)u.slice * B * nO;
#pragma unroll
    for (int t = 0; t < T; ++t) {
        if (!ok[t]) continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int to = u.rc * 16 + 4 * kk + v;
            if (to < d.tO) {
                const float re = acc[0][2 * t][v] - acc[1][2 * t + 1][v];
                const float im = acc[0][2 * t + 1][v] + acc[1][2 * t][v];
                dst[(size_t)(b_first + col_b[t]) * nO + d.cumO + to * M + col_m[t]] = make_float2(re, im);
            }
        }
    }
}

// TMAX = 3 serves the degrees with up to three column tiles per wave, TMAX = 6 the others (their
// accumulators need twice the registers).
template <int TMAX>
__global__ void __launch_bounds__(kThreads)
wmm_forward_kernel(const float2* __restrict__ FF, const float* __restrict__ Wp, float2* __restrict__ out,
                   const WmmDeg* __restrict__ degs, const WmmFwdUnit* __restrict__ units, int B, int nFF, int nO,
                   int stage_bytes, int depth, int nparts) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = part_major(nparts);
    const WmmFwdUnit u = units[up.unit];
    const WmmDeg d = degs[u.deg];
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave index, held in a scalar register
    const int b_first = (up.part * (int)(blockDim.x >> 6) + w) * d.G;   // a group is one wave or four
    if (b_first >= B) return;                                     // wave-uniform; the kernel has no barrier
    unsigned char* ring = smem + (size_t)w * depth * stage_bytes;
#define CGNET_FWD_T(T_) wmm_forward_wave<T_>(FF, Wp, out, d, u, B, nFF, nO, b_first, ring, depth, stage_bytes, lane)
    if (TMAX == 3) {
        switch (d.NC) {
            case 1: CGNET_FWD_T(1); break;
            case 2: CGNET_FWD_T(2); break;
            default: CGNET_FWD_T(3); break;
        }
    } else {
        switch (d.NC) {
            case 4: CGNET_FWD_T(4); break;
            case 5: CGNET_FWD_T(5); break;
            default: CGNET_FWD_T(6); break;
        }
    }
#undef CGNET_FWD_T
}

template __global__ void wmm_forward_kernel<3>(const float2*, const float*, float2*, const WmmDeg*, const WmmFwdUnit*, int,
                                               int, int, int, int, int);
template __global__ void wmm_forward_kernel<6>(const float2*, const float*, float2*, const WmmDeg*, const WmmFwdUnit*, int,
                                               int, int, int, int, int);

// O = sum over k-slices of the partial outputs, in slice order
__global__ void __launch_bounds__(256)
wmm_sum_slices_kernel(const float2* __restrict__ part, float2* __restrict__ O,
                      const int* __restrict__ cumO_S, int ndeg, int B, int nO) {
    __shared__ int s_tab[kMaxLookup];
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int e = (int)(idx % nO);
    const int di = lookup_in_group(ndeg, e, [&](int k) { return cumO_S[k]; }, s_tab);
    if (idx >= (size_t)B * nO) return;
    const int S = cumO_S[ndeg + 1 + di];
    float2 s = part[idx];
#pragma unroll 8
    for (int k = 1; k < S; ++k) {
        const float2 v = part[(size_t)k * B * nO + idx];
        s.x += v.x;
        s.y += v.y;
    }
    O[idx] = s;
}

// --------------------------------------------------------------------------- grad W (MFMA)
// NB blocks of eight m positions of one sample: all operands are read first, then the matrix
// instructions run back to back.  Positions past the end of the row read the last entry instead
// and get a zero gO operand; lanes without a channel or an output row read row 0 (their columns /
// rows of the accumulator are never stored).
template <int NB>
__device__ __forceinline__ void gradw_blocks(const float2* __restrict__ frow, const float2* __restrict__ grow,
                                             int blk0, int M, int kk, bool tok, f32x4& acc0, f32x4& acc1) {
    float2 f[NB][2], g[NB][2];
#pragma unroll
    for (int blk = 0; blk < NB; ++blk)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int p = (blk0 + blk) * 8 + kk * 2 + j;
            const int pc = min(p, M - 1);
            f[blk][j] = frow[pc];
            const float2 z = grow[pc];
            const bool on = tok && p < M;
            g[blk][j] = make_float2(on ? z.x : 0.f, on ? z.y : 0.f);
        }
#pragma unroll
    for (int blk = 0; blk < NB; ++blk) {
        const float2 f0 = f[blk][0], f1 = f[blk][1], g0 = g[blk][0], g1 = g[blk][1];
        acc0 = mfma4(g0.x, f0.x, acc0);
        acc0 = mfma4(g0.y, f0.y, acc0);
        acc0 = mfma4(g1.x, f1.x, acc0);
        acc0 = mfma4(g1.y, f1.y, acc0);
        acc1 = mfma4(g0.y, f0.x, acc1);
        acc1 = mfma4(-g0.x, f0.y, acc1);
        acc1 = mfma4(g1.y, f1.x, acc1);
        acc1 = mfma4(-g1.x, f1.y, acc1);
    }
}

// Raw sums  sum_{b in chunk, m} gO[b,to,m] * conj(FF[b,c,m])  of one chunk of samples into
// part[chunk][nW]; wmm_gradw_finish_kernel adds the chunks in order and divides by div[c].
// Per sample the group's FF rows (nc channels x M, one contiguous run) and the 16 gO rows are copied
// straight into LDS (LDS-direct loads, no registers), one sample ahead into the other half of a
// double buffer, one barrier per sample; each wave then reads its 16 channel rows in matrix-core
// operand order.
__global__ void __launch_bounds__(kThreads)
wmm_gradw_kernel(const float2* __restrict__ gO, const float2* __restrict__ FF, float2* __restrict__ part,
                 const WmmDeg* __restrict__ degs, const WmmChanUnit* __restrict__ units, int B,
                 int samples_per_chunk, int nFF, int nO, int nW, int ff_cap, int go_cap) {
    extern __shared__ __align__(16) unsigned char smem[];
    float2* ffbuf = reinterpret_cast<float2*>(smem);              // [2][ff_cap]
    float2* gobuf = ffbuf + 2 * ff_cap;                           // [2][go_cap]
    const UnitPart up = part_major((B + samples_per_chunk - 1) / samples_per_chunk);
    const WmmChanUnit u = units[up.unit];
    const WmmDeg d = degs[u.deg];
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int i = lane & 15, kk = lane >> 4;
    const int M = d.M;
    const bool wave_on = 16 * w < u.nc;
    const int c = u.c0 + 16 * w + i;
    const bool cok = wave_on && c < d.K && (16 * w + i) < u.nc;
    const int to_a = u.rc * 16 + i;
    const bool tok = to_a < d.tO;
    const int go_rows = min(16, d.tO - u.rc * 16);
    const int nblk = (M + 7) >> 3;
    const int n_ff = u.nc * M, n_go = go_rows * M;
    const int b_begin = up.part * samples_per_chunk;
    const int b_end = min(B, b_begin + samples_per_chunk);

    // one sample's FF rows of the unit (one contiguous run) and its gO rows, copied straight into LDS
    auto issue = [&](int b, int par) {
        const float2* fsrc = FF + (size_t)b * nFF + d.cumFF + (size_t)u.c0 * M;
        const float2* gsrc = gO + (size_t)b * nO + d.cumO + (size_t)u.rc * 16 * M;
        float2* fdst = ffbuf + par * ff_cap;
        float2* gdst = gobuf + par * go_cap;
        dma16<kThreads>(fsrc, fdst, n_ff >> 1, tid);
        if (n_ff & 1) dma8(fsrc + (n_ff - 1), fdst + (n_ff - 1), tid);
        dma16<kThreads>(gsrc, gdst, n_go >> 1, tid);
        if (n_go & 1) dma8(gsrc + (n_go - 1), gdst + (n_go - 1), tid);
    };
    if (b_begin < b_end) issue(b_begin, 0);
    // Blocked summation: the matrix-core chain runs over kGradWFold samples, then its sums are folded into
    // the totals -- a chain over the whole chunk (32 samples x 2M terms) loses several times the digits of the
    // blocked sums of a CPU matrix product.
    f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
    f32x4 tot0 = {0.f, 0.f, 0.f, 0.f}, tot1 = {0.f, 0.f, 0.f, 0.f};
    int buf = 0, since = 0;
    for (int b = b_begin; b < b_end; ++b, buf ^= 1) {
        const float2* ffl = ffbuf + buf * ff_cap;
        const float2* gol = gobuf + buf * go_cap;
        dma_wait();
        __syncthreads();           // sample b landed; nobody still reads the other buffer
        if (b + 1 < b_end) issue(b + 1, buf ^ 1);
        if (wave_on) {
            const float2* frow = ffl + (cok ? (16 * w + i) : 0) * M;
            const float2* grow = gol + (tok ? i : 0) * M;
            switch (nblk) {
                case 1: gradw_blocks<1>(frow, grow, 0, M, kk, tok, acc0, acc1); break;
                case 2: gradw_blocks<2>(frow, grow, 0, M, kk, tok, acc0, acc1); break;
                case 3: gradw_blocks<3>(frow, grow, 0, M, kk, tok, acc0, acc1); break;
                case 4: gradw_blocks<4>(frow, grow, 0, M, kk, tok, acc0, acc1); break;
                default:
                    for (int blk = 0; blk < nblk; blk += 3) {
                        if (blk + 3 <= nblk) gradw_blocks<3>(frow, grow, blk, M, kk, tok, acc0, acc1);
                        else if (blk + 2 == nblk) gradw_blocks<2>(frow, grow, blk, M, kk, tok, acc0, acc1);
                        else gradw_blocks<1>(frow, grow, blk, M, kk, tok, acc0, acc1);
                    }
                    break;
            }
            if (++since == kGradWFold) {
                since = 0;
                tot0 += acc0;
                tot1 += acc1;
                acc0 = acc1 = (f32x4){0.f, 0.f, 0.f, 0.f};
            }
        }
    }
    tot0 += acc0;
    tot1 += acc1;
    if (cok) {
        float2* dst = part + (size_t)up.part * nW;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int to = u.rc * 16 + 4 * kk + v;
            if (to < d.tO) dst[d.cumW + (size_t)to * d.K + c] = make_float2(tot0[v], tot1[v]);
        }
    }
}

__global__ void __launch_bounds__(256)
wmm_gradw_finish_kernel(const float2* __restrict__ part, const float* __restrict__ stds, float eps,
                        const WmmDeg* __restrict__ degs, int ndeg, float2* __restrict__ gW, int nW, int nchunks) {
    __shared__ int s_tab[kMaxLookup];
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int di = lookup_in_group(ndeg, idx, [&](int k) { return degs[k].cumW; }, s_tab);
    if (idx >= nW) return;
    float2 s = part[idx];
    for (int k = 1; k < nchunks; ++k) {
        const float2 v = part[(size_t)k * nW + idx];
        s.x += v.x;
        s.y += v.y;
    }
    if (stds) {
        const WmmDeg d = degs[di];
        const int c = (idx - d.cumW) % d.K;
        const float r = fmaxf(eps, stds[d.cumT + c]);
        s.x /= r;
        s.y /= r;
    }
    gW[idx] = s;
}

// --------------------------------------------------------------------------- grad FF
// gFF[b, c, m] = sum_to WT[c][to] * gO[b, to, m]   with WT = conj(W)/div packed channel-major
__global__ void __launch_bounds__(kThreads)
wmm_gradff_kernel(const float2* __restrict__ gO, const float2* __restrict__ WT, float2* __restrict__ gFF,
                  const WmmDeg* __restrict__ degs, const WmmChanUnit* __restrict__ units, int nFF, int nO, int B) {
    extern __shared__ __align__(16) unsigned char smem[];
    float2* go = reinterpret_cast<float2*>(smem);      // [tO][M]
    const UnitPart up = part_major(B);
    const WmmChanUnit u = units[up.unit];
    const WmmDeg d = degs[u.deg];
    const int b = up.part;
    const int M = d.M, tO = d.tO;
    const float2* src = gO + (size_t)b * nO + d.cumO;
    for (int e = threadIdx.x; e < tO * M; e += kThreads) go[e] = src[e];
    __syncthreads();
    const int n = u.nc * M;
    float2* dst = gFF + (size_t)b * nFF + d.cumFF + (size_t)u.c0 * M;
    for (int e = threadIdx.x; e < n; e += kThreads) {
        const int cl = e / M, m = e - cl * M;
        const float2* wt = WT + d.cumW + (size_t)(u.c0 + cl) * tO;
        float re = 0.f, im = 0.f;
        for (int to = 0; to < tO; ++to) {
            const float2 wv = wt[to];
            const float2 gv = go[to * M + m];
            re = fmaf(wv.x, gv.x, re);
            re = fmaf(-wv.y, gv.y, re);
            im = fmaf(wv.x, gv.y, im);
            im = fmaf(wv.y, gv.x, im);
        }
        dst[e] = make_float2(re, im);
    }
}

// ---- grad FF on the matrix cores -----------------------------------------------------------
// gFF[b, c, (m, re/im)] = sum over k = (to, re/im) of A[c][k] * Bop[k][(m, re/im)] with
//   A[c][(to,0)] = W_re[to][c]/div[c], A[c][(to,1)] = W_im[to][c]/div[c]        (packed once per call)
//   Bop[(to,0)][(m,0)] = gO_re, Bop[(to,1)][(m,0)] = gO_im, Bop[(to,0)][(m,1)] = gO_im, Bop[(to,1)][(m,1)] = -gO_re
// A wave keeps the A operand of its 16 channels in registers and walks over the samples of its
// group; a 16-channel x 16-column result tile is stored as four 64-byte row segments.
__global__ void __launch_bounds__(256)
pack_w_gradff_kernel(const float2* __restrict__ W, const float* __restrict__ stds, float eps,
                     const WmmDeg* __restrict__ degs, int ndeg, float* __restrict__ Ap, int total_blocks) {
    __shared__ int s_tab[kMaxLookup];
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;       // four weights of one row = two 16-byte stores
    const int blk = idx >> 3, half = (idx >> 2) & 1, i0 = (idx & 3) * 4;
    const int di = lookup_in_group(ndeg, blk, [&](int k) { return degs[k].ap_base; }, s_tab);
    if (blk >= total_blocks) return;
    const WmmDeg d = degs[di];
    const int rel = blk - d.ap_base;             // ctile * nks_b + ks
    const int ks = rel % d.nks_b, ctile = rel / d.nks_b;
    const int c0 = ctile * 16 + i0, to = 2 * ks + half;           // k = 4*ks + kk, to = k >> 1, kk = 2*half + sel
    float re[4] = {0.f, 0.f, 0.f, 0.f}, im[4] = {0.f, 0.f, 0.f, 0.f};
    if (to < d.tO) {
        const float2* wrow = W + d.cumW + (size_t)to * d.K;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + j;
            if (c < d.K) {
                const float2 w = wrow[c];
                const float r = stds ? fmaxf(eps, stds[d.cumT + c]) : 1.f;
                re[j] = stds ? w.x / r : w.x;
                im[j] = stds ? w.y / r : w.y;
            }
        }
    }
    float* dst = Ap + (size_t)blk * 64 + half * 32 + i0;
    *reinterpret_cast<float4*>(dst) = make_float4(re[0], re[1], re[2], re[3]);
    *reinterpret_cast<float4*>(dst + 16) = make_float4(im[0], im[1], im[2], im[3]);
}

// Gradient with respect to FF on the matrix cores (t_O <= 16): gFF[c, (m, re/im)] = sum_k A[c, k] * B[k, (m, re/im)]
// with k = (to, re/im).  A work-group is one wave (no barrier): it owns the up to 64 channels of its
// unit as tiles of 16, keeps their A operands in registers and walks over the samples of its group.
// The gO rows of the next sample arrive by LDS-direct loads while the current one is multiplied;
// one load of the rows serves all channel tiles.  Every 16 x 2M result tile goes through the wave's
// LDS image and leaves as one contiguous run of 16-byte stores, one tile behind the arithmetic.
// NT = column tiles worked on together; ONE: these are all column tiles of the degree, so the B
// operands are built once per sample and shared by the channel tiles.
constexpr int kGffSub = 4;     // channel tiles per wave
template <int NKS, int NT, bool ONE>
__device__ __forceinline__ void wmm_gradff_wave(const float2* __restrict__ gO, const float* __restrict__ Ap,
                                                float2* __restrict__ gFF, const WmmDeg& d, const WmmChanUnit& u, int B,
                                                int samples_per_group, int nFF, int nO, int out_bytes, int go_bytes,
                                                unsigned char* mine, int lane, int group) {
    float* ol = reinterpret_cast<float*>(mine);                              // [16][2M]
    unsigned char* gobuf = mine + out_bytes;                                  // [2][go_bytes]
    const int i = lane & 15, kk = lane >> 4;
    const int M = d.M, tO = d.tO;
    constexpr int nks = NKS;
    const int nsub = (u.nc + 15) >> 4;
    float a[kGffSub][NKS];
#pragma unroll
    for (int sub = 0; sub < kGffSub; ++sub)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
            a[sub][ks] = sub < nsub ? Ap[((size_t)d.ap_base + (size_t)((u.c0 >> 4) + sub) * nks + ks) * 64 + lane] : 0.f;
    // k = 4*ks + kk  ->  to = 2*ks + (kk >> 1), re/im = kk & 1;  column 16*ct + i -> m = 8*ct + (i >> 1), re/im = i & 1
    const int to_lane = kk >> 1, sel = kk & 1, r = i & 1;
    const float cx = (r == sel) ? (r ? -1.f : 1.f) : 0.f, cy = (r == sel) ? 0.f : 1.f;   // B = cx * re + cy * im
    const int nct = (2 * M + 15) >> 4;
    const int n_go = tO * M;                      // complex entries of the gO rows
    const int b_begin = group * samples_per_group, b_end = min(B, b_begin + samples_per_group);
    if (b_begin >= b_end) return;
    {
        // rows past t_O are read (times zero weights): they must hold finite values
        float4* z = reinterpret_cast<float4*>(gobuf);
        for (int e = lane; e < (2 * go_bytes) >> 4; e += 64) z[e] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    auto issue = [&](int b, int par) {
        const float2* src = gO + (size_t)b * nO + d.cumO;
        unsigned char* dst = gobuf + (size_t)par * go_bytes;
        dma16<64>(src, dst, n_go >> 1, lane);
        if (n_go & 1) dma8(src + (n_go - 1), dst + 8 * (size_t)(n_go - 1), lane);
    };
    auto rows_of = [&](int sub) { return min(16, u.nc - 16 * sub); };
    auto store_tile = [&](int b, int sub) {
        const size_t off = (size_t)b * nFF + d.cumFF + (size_t)(u.c0 + 16 * sub) * M;
        const int n_out = rows_of(sub) * M;
        float2* dst = gFF + off;
        const float2* src = reinterpret_cast<const float2*>(ol);
        const int head = (int)(off & 1);          // unaligned first entry
        if (head && lane == 0) dst[0] = src[0];
        const int n4 = (n_out - head) >> 1;
        for (int idx = lane; idx < n4; idx += 64) {
            const float2 z0 = src[head + 2 * idx], z1 = src[head + 2 * idx + 1];
            stream_store16(dst + head + 2 * idx, z0.x, z0.y, z1.x, z1.y);
        }
        if (((n_out - head) & 1) && lane == 0) dst[n_out - 1] = src[n_out - 1];
    };
    // lower bound of the store instructions of one tile (the loop of store_tile, without head and tail)
    auto stores_of = [&](int sub) { return (((rows_of(sub) * M - 1) >> 1) + 63) >> 6; };
    // Vector memory operations complete in the order issued.  The copy of sample b is started at the
    // beginning of sample b-1 and followed there by the stores of the last tile of sample b-2 and of
    // all tiles but the last of sample b-1: waiting until no more than that many operations are
    // outstanding is enough for the copy and leaves those stores in flight.
    int later_stores = 0;
    for (int sub = 0; sub + 1 < nsub; ++sub) later_stores += stores_of(sub);
    const int last_stores = stores_of(nsub - 1);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the clearing stores precede the first copy
    issue(b_begin, 0);
    const int row0 = 4 * kk;                      // D rows of this lane inside a tile
    int par = 0;
    for (int b = b_begin; b < b_end; ++b, par ^= 1) {
        wait_vmcnt(b == b_begin ? 0 : later_stores + (b - 2 >= b_begin ? last_stores : 0));   // gO rows of sample b landed
        if (b + 1 < b_end) issue(b + 1, par ^ 1);
        const float2* g = reinterpret_cast<const float2*>(gobuf + (size_t)par * go_bytes);
        float bv[NKS][NT];
        auto build_b = [&](int ct0) {
            int mofs[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) mofs[t] = min(8 * (ct0 + t) + (i >> 1), M - 1);   // clamped: extra columns are not stored
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const int to = min(2 * ks + to_lane, tO - 1);                 // clamped: rows past t_O carry zero weights
#pragma unroll
                for (int t = 0; t < NT; ++t) {
                    const float2 z = g[to * M + mofs[t]];
                    bv[ks][t] = fmaf(z.x, cx, z.y * cy);
                }
            }
        };
        if (ONE) build_b(0);
#pragma unroll
        for (int sub = 0; sub < kGffSub; ++sub) {
            if (sub < nsub) {
                // the tile before this one leaves (its LDS image is read before it is overwritten below)
                if (sub > 0) store_tile(b, sub - 1);
                else if (b > b_begin) store_tile(b - 1, nsub - 1);
                for (int ct0 = 0; ct0 < nct; ct0 += NT) {
                    if (!ONE) build_b(ct0);
                    f32x4 acc[NT];
#pragma unroll
                    for (int t = 0; t < NT; ++t) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
                        for (int t = 0; t < NT; ++t) acc[t] = mfma4(a[sub][ks], bv[ks][t], acc[t]);
#pragma unroll
                    for (int t = 0; t < NT; ++t) {
                        const int col = (ct0 + t) * 16 + i;
                        if (col < 2 * M) {
#pragma unroll
                            for (int v = 0; v < 4; ++v) ol[(size_t)(row0 + v) * 2 * M + col] = acc[t][v];
                        }
                    }
                    if (ONE) break;
                }
            }
        }
    }
    store_tile(b_end - 1, nsub - 1);
}

__global__ void __launch_bounds__(64)
wmm_gradff_mfma_kernel(const float2* __restrict__ gO, const float* __restrict__ Ap, float2* __restrict__ gFF,
                       const WmmDeg* __restrict__ degs, const WmmChanUnit* __restrict__ units, int B,
                       int samples_per_group, int nFF, int nO, int out_bytes, int go_bytes) {
    extern __shared__ __align__(16) unsigned char smem[];
    const UnitPart up = part_major((B + samples_per_group - 1) / samples_per_group);
    const WmmChanUnit u = units[up.unit];
    const WmmDeg d = degs[u.deg];
    const int lane = threadIdx.x;
#define CGNET_GFF_ARGS gO, Ap, gFF, d, u, B, samples_per_group, nFF, nO, out_bytes, go_bytes, smem, lane, up.part
#define CGNET_GFF(N_)                                                                     \
    case N_:                                                                              \
        if (nct == 1) wmm_gradff_wave<N_, 1, true>(CGNET_GFF_ARGS);                       \
        else if (nct == 2) wmm_gradff_wave<N_, 2, true>(CGNET_GFF_ARGS);                  \
        else if (nct == 3) wmm_gradff_wave<N_, 3, true>(CGNET_GFF_ARGS);                  \
        else wmm_gradff_wave<N_, 3, false>(CGNET_GFF_ARGS);                               \
        break;
    const int nct = (2 * d.M + 15) >> 4;
    switch (d.nks_b) {
        CGNET_GFF(1) CGNET_GFF(2) CGNET_GFF(3) CGNET_GFF(4) CGNET_GFF(5) CGNET_GFF(6) CGNET_GFF(7)
        default:
            if (nct == 1) wmm_gradff_wave<8, 1, true>(CGNET_GFF_ARGS);
            else if (nct == 2) wmm_gradff_wave<8, 2, true>(CGNET_GFF_ARGS);
            else if (nct == 3) wmm_gradff_wave<8, 3, true>(CGNET_GFF_ARGS);
            else wmm_gradff_wave<8, 3, false>(CGNET_GFF_ARGS);
            break;
    }
#undef CGNET_GFF_ARGS
#undef CGNET_GFF
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* p, size_t n) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0.f;
}

int stat_groups_for(int B) { return std::max(1, std::min(B, kStatGroups)); }

struct FwdWorkspace {
    size_t sums, part, wp, opart, total;
};

FwdWorkspace fwd_workspace(const cgnet_wmm_plan* p, int B) {
    FwdWorkspace w;
    size_t o = 0;
    w.sums = o;
    o += align_up(sizeof(double) * 2 * (size_t)p->sumT, 256);
    w.part = o;
    o += align_up(sizeof(double) * 2 * (size_t)p->sumT * stat_groups_for(B), 256);
    w.wp = o;
    o += align_up(sizeof(float) * 64 * (size_t)p->wp_blocks, 256);
    w.opart = o;
    if (p->maxS > 1) o += align_up(sizeof(float) * 2 * (size_t)p->nO * B * p->maxS, 256);
    w.total = o;
    return w;
}

}  // namespace
}  // namespace cgnet

using namespace cgnet;

static void free_plan(cgnet_wmm_plan* plan) {
    if (!plan) return;
    void* ptrs[] = {plan->d_degs, plan->d_fwd_units, plan->d_gw_units, plan->d_gw_units_rc0, plan->d_gff_units, plan->d_gff_zero_units,
                    plan->d_stat_units, plan->d_cumO};
    for (void* q : ptrs)
        if (q) (void)hipFree(q);
    delete plan;
}

// Number of work-groups of a one-dimensional (unit, part) grid; 0 when the product exceeds the grid limit.
static unsigned grid_1d(size_t nunits, size_t nparts) {
    const unsigned long long n = (unsigned long long)nunits * nparts;
    return n < (1ULL << 31) ? (unsigned)n : 0u;
}

extern "C" int cgnet_wmm_plan_create(cgnet_wmm_plan** plan, int L, const int* h_t_FF, const int* h_t_O) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    *plan = nullptr;
    CGNET_REQUIRE(L >= 0 && L <= kMaxL, CGNET_ERR_UNSUPPORTED, "lmax=%d outside [0, %d]", L, kMaxL);
    CGNET_REQUIRE(h_t_FF && h_t_O, CGNET_ERR_ARG, "null pointer argument");
    cgnet_wmm_plan* p = new cgnet_wmm_plan();
    std::unique_ptr<cgnet_wmm_plan, void (*)(cgnet_wmm_plan*)> guard(p, free_plan);
    p->L = L;
    long long cFF = 0, cO = 0, cW = 0, cT = 0;
    int wp = 0;
    for (int l = 0; l <= L; ++l) {
        const int K = h_t_FF[l], tO = h_t_O[l], M = 2 * l + 1;
        CGNET_REQUIRE(K >= 0 && tO >= 0, CGNET_ERR_ARG, "negative channel count at degree %d", l);
        CGNET_REQUIRE(tO <= kMaxTau, CGNET_ERR_UNSUPPORTED, "t_O[%d]=%d above %d", l, tO, kMaxTau);
        WmmDeg d;
        d.l = l; d.M = M; d.K = K; d.tO = tO;
        d.cumFF = (int)cFF; d.cumO = (int)cO; d.cumW = (int)cW; d.cumT = (int)cT;
        d.nrc = std::max(1, (tO + 15) / 16);
        d.wp_base = wp;
        // forward: a wave owns G samples = G*M complex columns in NC tiles of 16 columns
        int bestG = 1, bestNC = (M + 15) / 16;
        {
            double best = -1;
            for (int nc = 1; nc <= 3; ++nc) {
                const int g = (16 * nc) / M;
                if (g < 1) continue;
                const double eff = (double)g * M / (16.0 * nc);
                if (eff > best + 1e-9) { best = eff; bestG = g; bestNC = nc; }
            }
        }
        d.G = bestG;
        d.NC = bestNC;
        // k-slices of about kFwdSlice channels (multiples of 8)
        d.S = std::max(1, (K + kFwdSlice - 1) / kFwdSlice);
        d.nks_b = std::max(1, (2 * tO + 3) / 4);
        d.ap_base = p->ap_blocks;
        p->ap_blocks += ((K + 15) / 16) * d.nks_b;
        if (tO > 16) p->gff_mfma = false;
        p->degs.push_back(d);
        cFF += (long long)K * M;
        cO += (long long)tO * M;
        cW += (long long)K * tO;
        cT += K;
        wp += ((K + 7) / 8) * d.nrc * 4;
        CGNET_REQUIRE(cFF < (1LL << 30) && cW < (1LL << 30), CGNET_ERR_UNSUPPORTED, "sizes above 2^30 complex entries");
    }
    p->nFF = (int)cFF; p->nO = (int)cO; p->nW = (int)cW; p->sumT = (int)cT;
    p->wp_blocks = wp;
    const int ndeg = (int)p->degs.size();
    for (int di = 0; di < ndeg; ++di) {
        const WmmDeg& d = p->degs[di];
        if (d.K == 0 || d.tO == 0) continue;
        CGNET_REQUIRE(d.NC <= kFwdMaxT, CGNET_ERR_UNSUPPORTED, "degree %d has more than 96 columns per sample", d.l);
        p->maxS = std::max(p->maxS, d.S);
        p->maxG = std::max(p->maxG, d.G);
        p->fwd_stage_cap = std::max(p->fwd_stage_cap, 1024 + d.G * kFwdKC * d.M * 8);   // bytes: weights + runs
        const int steps = (d.K + 7) / 8;
        const int per = ((steps + d.S - 1) / d.S) * 8;
        for (int rc = 0; rc < d.nrc; ++rc)
            for (int s = 0; s < d.S; ++s) {
                WmmFwdUnit u{di, rc, s, std::min(d.K, s * per), std::min(d.K, (s + 1) * per)};
                p->fwd_units.push_back(u);
            }
        int gw_nc = 64;
        // both stages of the unit's FF rows and of the 16 gO rows fit 64 KB of LDS
        while (gw_nc > 16 && 16 * ((size_t)gw_nc * d.M + 2 + 16 * (size_t)d.M + 2) > 64 * 1024) gw_nc /= 2;
        for (int rc = 0; rc < d.nrc; ++rc)
            for (int c0 = 0; c0 < d.K; c0 += gw_nc)
                p->gw_units.push_back(WmmChanUnit{di, rc, c0, std::min(gw_nc, d.K - c0)});
        p->gff_out_cap = std::max(p->gff_out_cap, (int)align_up((size_t)16 * d.M * 8, 16));                       // bytes per wave
        p->gff_go_cap = std::max(p->gff_go_cap, (int)align_up((size_t)std::min(d.tO, 16) * d.M * 8 + 16, 16));   // bytes per wave and buffer
        p->gw_ff_cap = std::max(p->gw_ff_cap, (int)align_up((size_t)gw_nc * d.M + 2, 2));
        p->gw_go_cap = std::max(p->gw_go_cap, (int)align_up((size_t)16 * d.M + 2, 2));
    }
    for (int di = 0; di < ndeg; ++di) {
        const WmmDeg& d = p->degs[di];
        if (d.K == 0) continue;
        const int per_stat = std::max(1, std::min(kThreads, kStatTileBytes / (8 * d.M)));
        for (int c0 = 0; c0 < d.K; c0 += per_stat)
            p->stat_units.push_back(WmmChanUnit{di, 0, c0, std::min(per_stat, d.K - c0)});
        p->stat_lds = std::max(p->stat_lds, (size_t)8 * per_stat * d.M);
        const int per_gff = std::max(1, 4096 / d.M);
        for (int c0 = 0; c0 < d.K; c0 += per_gff) {
            p->gff_units.push_back(WmmChanUnit{di, 0, c0, std::min(per_gff, d.K - c0)});
            if (d.tO == 0) p->gff_zero_units.push_back(p->gff_units.back());
        }
        p->gff_lds = std::max(p->gff_lds, (size_t)8 * d.tO * d.M);
    }
    // the matrix-core gradient kernel keeps a tile and two operand buffers per wave inside 64 KB of LDS
    if ((size_t)p->gff_out_cap + 2 * (size_t)p->gff_go_cap > 64 * 1024) p->gff_mfma = false;
    CGNET_REQUIRE(p->gff_lds <= 64 * 1024, CGNET_ERR_UNSUPPORTED, "t_O*(2l+1) too large for the gradient kernel");
    // heavier forward units first
    std::stable_sort(p->fwd_units.begin(), p->fwd_units.end(), [&](const WmmFwdUnit& a, const WmmFwdUnit& b) {
        return (long long)(a.k_end - a.k_begin) * p->degs[a.deg].M > (long long)(b.k_end - b.k_begin) * p->degs[b.deg].M;
    });
    std::stable_sort(p->gw_units.begin(), p->gw_units.end(), [&](const WmmChanUnit& a, const WmmChanUnit& b) {
        return p->degs[a.deg].M > p->degs[b.deg].M;
    });

    std::vector<int> cumO_S(2 * ndeg + 1);
    for (int di = 0; di < ndeg; ++di) cumO_S[di] = p->degs[di].cumO;
    cumO_S[ndeg] = p->nO;
    for (int di = 0; di < ndeg; ++di) cumO_S[ndeg + 1 + di] = (p->degs[di].K == 0 || p->degs[di].tO == 0) ? 0 : p->degs[di].S;

    auto upload = [&](const void* src, size_t bytes, void** dst) -> int {
        if (bytes == 0) return CGNET_OK;
        CGNET_HIP(hipMalloc(dst, bytes));
        CGNET_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return CGNET_OK;
    };
    int rc;
    if ((rc = upload(p->degs.data(), sizeof(WmmDeg) * ndeg, (void**)&p->d_degs))) return rc;
    {
        // longest units first, so that the last groups to start are short ones
        auto work = [&](const WmmFwdUnit& u) {
            const WmmDeg& d = p->degs[u.deg];
            return (long long)(u.k_end - u.k_begin) * d.M * d.G;
        };
        std::stable_sort(p->fwd_units.begin(), p->fwd_units.end(),
                         [&](const WmmFwdUnit& a, const WmmFwdUnit& b) { return work(a) > work(b); });
        auto mid = std::stable_partition(p->fwd_units.begin(), p->fwd_units.end(),
                                         [&](const WmmFwdUnit& u) { return p->degs[u.deg].NC <= 3; });
        p->fwd_units_small = (int)(mid - p->fwd_units.begin());
    }
    if ((rc = upload(p->fwd_units.data(), sizeof(WmmFwdUnit) * p->fwd_units.size(), (void**)&p->d_fwd_units))) return rc;
    if ((rc = upload(p->gw_units.data(), sizeof(WmmChanUnit) * p->gw_units.size(), (void**)&p->d_gw_units))) return rc;
    for (const WmmChanUnit& u : p->gw_units)
        if (u.rc == 0) p->gw_units_rc0.push_back(u);
    if ((rc = upload(p->gw_units_rc0.data(), sizeof(WmmChanUnit) * p->gw_units_rc0.size(), (void**)&p->d_gw_units_rc0))) return rc;
    if ((rc = upload(p->gff_units.data(), sizeof(WmmChanUnit) * p->gff_units.size(), (void**)&p->d_gff_units))) return rc;
    if ((rc = upload(p->gff_zero_units.data(), sizeof(WmmChanUnit) * p->gff_zero_units.size(), (void**)&p->d_gff_zero_units))) return rc;
    if ((rc = upload(p->stat_units.data(), sizeof(WmmChanUnit) * p->stat_units.size(), (void**)&p->d_stat_units))) return rc;
    if ((rc = upload(cumO_S.data(), sizeof(int) * cumO_S.size(), (void**)&p->d_cumO))) return rc;
    *plan = guard.release();
    return CGNET_OK;
}

extern "C" int cgnet_wmm_plan_destroy(cgnet_wmm_plan* plan) {
    clear_error();
    free_plan(plan);
    return CGNET_OK;
}

extern "C" size_t cgnet_wmm_plan_gradw_lds(const cgnet_wmm_plan* plan) {
    if (!plan) return 0;
    return sizeof(float2) * 2 * ((size_t)plan->gw_ff_cap + plan->gw_go_cap);
}

extern "C" int cgnet_wmm_plan_sizes(const cgnet_wmm_plan* plan, int sizes[4]) {
    clear_error();
    CGNET_REQUIRE(plan && sizes, CGNET_ERR_ARG, "null pointer argument");
    sizes[0] = plan->nFF;
    sizes[1] = plan->nO;
    sizes[2] = plan->nW;
    sizes[3] = plan->sumT;
    return CGNET_OK;
}

extern "C" size_t cgnet_FN_WMM_forward_workspace(const cgnet_wmm_plan* plan, int B) {
    if (!plan || B <= 0) return 0;
    return fwd_workspace(plan, B).total;
}

extern "C" int cgnet_FN_WMM_forward(const cgnet_wmm_plan* plan, const float* d_FF, float* d_O, const float* d_W,
                                    int B, float* d_stds, float cnt, float eps, int flags, const double* d_sums,
                                    void* d_workspace, size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (B == 0) return CGNET_OK;
    const bool bn = flags & CGNET_FN_BATCHNORM, upd = bn && (flags & CGNET_FN_UPDATE_STD);
    CGNET_REQUIRE(!bn || d_stds, CGNET_ERR_ARG, "batch-norm flag set but d_stds is NULL");
    CGNET_REQUIRE(plan->nO == 0 || d_O, CGNET_ERR_ARG, "d_O is NULL");
    CGNET_REQUIRE(plan->nFF == 0 || d_FF, CGNET_ERR_ARG, "d_FF is NULL");
    CGNET_REQUIRE(plan->nW == 0 || d_W, CGNET_ERR_ARG, "d_W is NULL");
    const FwdWorkspace ws = fwd_workspace(plan, B);
    CGNET_REQUIRE(d_workspace && workspace_bytes >= ws.total, CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, ws.total);
    hipStream_t s = (hipStream_t)stream;
    char* base = (char*)d_workspace;
    const int ndeg = (int)plan->degs.size();

    if (upd && plan->sumT > 0) {
        const double* sums = d_sums;
        if (!sums) {
            const int ng = stat_groups_for(B);
            const int spg = (B + ng - 1) / ng;
            const int ngroups = (B + spg - 1) / spg;
            CGNET_LAUNCH(fn_stats_kernel, dim3(grid_1d(plan->stat_units.size(), ngroups)), dim3(kThreads),
                               plan->stat_lds, s, (const float2*)d_FF, plan->d_degs, plan->d_stat_units, plan->nFF,
                               B, spg, (double*)(base + ws.part), plan->sumT);
            CGNET_HIP(hipGetLastError());
            const int n2 = 2 * plan->sumT;
            CGNET_LAUNCH(fn_sum_groups_kernel, dim3((n2 + 255) / 256), dim3(256), 0, s,
                               (const double*)(base + ws.part), (double*)(base + ws.sums), n2, ngroups);
            CGNET_HIP(hipGetLastError());
            sums = (const double*)(base + ws.sums);
        }
        CGNET_LAUNCH(fn_update_std_kernel, dim3((plan->sumT + 255) / 256), dim3(256), 0, s, sums, d_stds,
                           plan->d_degs, ndeg, plan->sumT, B, cnt);
        CGNET_HIP(hipGetLastError());
    }
    if (plan->nO == 0) return CGNET_OK;
    float* Wp = (float*)(base + ws.wp);
    if (!plan->fwd_units.empty()) {
        const int total = plan->wp_blocks * 16;   // one thread per four packed floats
        CGNET_LAUNCH(pack_w_forward_kernel, dim3((total + 255) / 256), dim3(256), 0, s, (const float2*)d_W,
                           bn ? d_stds : nullptr, eps, plan->d_degs, ndeg, Wp, plan->wp_blocks);
        CGNET_HIP(hipGetLastError());
    }
    return wmm_forward_packed(plan, d_FF, d_O, Wp, B, base + ws.opart, s);
}

namespace cgnet {
size_t wmm_forward_wp_bytes(const cgnet_wmm_plan* plan) { return sizeof(float) * 64 * (size_t)plan->wp_blocks; }
size_t wmm_forward_opart_bytes(const cgnet_wmm_plan* plan, int B) {
    return plan->maxS > 1 ? sizeof(float) * 2 * (size_t)plan->nO * B * plan->maxS : 0;
}

// The mixing itself, with the weights already packed (pack_w_forward_thread): O = sum over channel slices.
int wmm_forward_packed(const cgnet_wmm_plan* plan, const float* d_FF, float* d_O, const float* Wp, int B,
                       void* d_opart, hipStream_t s) {
    const int ndeg = (int)plan->degs.size();
    if (plan->nO == 0 || B == 0) return CGNET_OK;
    if (plan->fwd_units.empty()) {   // degrees with outputs but no mid channels produce zeros
        const size_t n = (size_t)2 * plan->nO * B;
        CGNET_LAUNCH(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_O, n);
        CGNET_HIP(hipGetLastError());
        return CGNET_OK;
    }
    // degrees with t_O > 0 but no mid channels are never written by the product kernel
    bool holes = false;
    for (const WmmDeg& d : plan->degs) holes |= (d.tO > 0 && d.K == 0);
    float2* out = plan->maxS > 1 ? (float2*)d_opart : (float2*)d_O;
    if (holes) {
        const size_t n = (size_t)2 * plan->nO * B * (plan->maxS > 1 ? plan->maxS : 1);
        CGNET_LAUNCH(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, (float*)out, n);
        CGNET_HIP(hipGetLastError());
    }
    // Work-groups of one wave: the waves do not cooperate, and a group that is one wave leaves no LDS idle beside a
    // short last group of samples and lets the grid drain wave by wave (CGNET_WMM_FWD_WPG=4: four waves a group).
    static const int wpg = [] { const char* e = getenv("CGNET_WMM_FWD_WPG"); return e && atoi(e) == 4 ? 4 : 1; }();
    int ygroups = 1;
    for (const WmmDeg& d : plan->degs)
        if (d.K > 0 && d.tO > 0) ygroups = std::max(ygroups, (B + wpg * d.G - 1) / (wpg * d.G));
    CGNET_REQUIRE(ygroups <= 65535, CGNET_ERR_UNSUPPORTED, "B=%d too large", B);
    // the LDS-direct copies address the first 64 KB of a group's LDS
    static const int want_depth = [] { const char* e = getenv("CGNET_WMM_FWD_DEPTH"); return e ? atoi(e) : kFwdDepth; }();
    const int depth = (int)std::min<size_t>(want_depth, (64 * 1024) / (wpg * (size_t)plan->fwd_stage_cap));
    CGNET_REQUIRE(depth >= 2, CGNET_ERR_UNSUPPORTED, "forward stage of %d bytes does not fit the LDS ring", plan->fwd_stage_cap);
    const size_t lds = wpg * (size_t)depth * plan->fwd_stage_cap;
    if (plan->fwd_units_small > 0) {
        CGNET_LAUNCH(wmm_forward_kernel<3>, dim3(grid_1d(plan->fwd_units_small, ygroups)), dim3(64 * wpg), lds, s,
                     (const float2*)d_FF, Wp, out, plan->d_degs, plan->d_fwd_units, B, plan->nFF, plan->nO,
                     plan->fwd_stage_cap, depth, ygroups);
        CGNET_HIP(hipGetLastError());
    }
    if ((int)plan->fwd_units.size() > plan->fwd_units_small) {
        CGNET_LAUNCH(wmm_forward_kernel<6>, dim3(grid_1d(plan->fwd_units.size() - plan->fwd_units_small, ygroups)),
                     dim3(64 * wpg), lds, s, (const float2*)d_FF, Wp, out, plan->d_degs,
                     plan->d_fwd_units + plan->fwd_units_small, B, plan->nFF, plan->nO, plan->fwd_stage_cap, depth,
                     ygroups);
        CGNET_HIP(hipGetLastError());
    }
    if (plan->maxS > 1) {
        const size_t n = (size_t)plan->nO * B;
        CGNET_LAUNCH(wmm_sum_slices_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                           (const float2*)out, (float2*)d_O, plan->d_cumO, ndeg, B, plan->nO);
        CGNET_HIP(hipGetLastError());
    }
    return CGNET_OK;
}
}  // namespace cgnet

namespace cgnet {
bool wmm_gradff_operand_ok(const cgnet_wmm_plan* plan) { return plan && plan->gff_mfma; }
int wmm_plan_degrees(const cgnet_wmm_plan* plan) { return (int)plan->degs.size(); }
int wmm_plan_degree(const cgnet_wmm_plan* plan, int l, WmmDegInfo* info) {
    if (!plan || l < 0 || l >= (int)plan->degs.size() || !info) return CGNET_ERR_ARG;
    const WmmDeg& d = plan->degs[l];
    *info = WmmDegInfo{d.K, d.tO, d.cumO, d.cumW, d.cumT};
    return CGNET_OK;
}
}  // namespace cgnet

static int gradw_chunks(int B) { return (B + kGradWChunk - 1) / kGradWChunk; }

namespace cgnet {
size_t wmm_gradw_part_bytes(const cgnet_wmm_plan* plan, int B) {
    return sizeof(float) * 2 * (size_t)plan->nW * gradw_chunks(B);
}
int wmm_gradw_raw(const cgnet_wmm_plan* plan, const float* d_gO, const float* d_FF, float* d_part, int B, int* nchunks_out,
                  hipStream_t s) {
    // equal chunks of at most kGradWChunk samples; the kernel derives the number of chunks from their size
    const int spc = (B + gradw_chunks(B) - 1) / gradw_chunks(B);
    const int nchunks = (B + spc - 1) / spc;             // <= gradw_chunks(B), what the partial area holds
    const size_t lds = sizeof(float2) * 2 * ((size_t)plan->gw_ff_cap + plan->gw_go_cap);
    CGNET_LAUNCH(wmm_gradw_kernel, dim3(grid_1d(plan->gw_units.size(), nchunks)), dim3(kThreads), lds, s,
                 (const float2*)d_gO, (const float2*)d_FF, (float2*)d_part, plan->d_degs, plan->d_gw_units, B, spc,
                 plan->nFF, plan->nO, plan->nW, plan->gw_ff_cap, plan->gw_go_cap);
    CGNET_HIP(hipGetLastError());
    *nchunks_out = nchunks;
    return CGNET_OK;
}
}  // namespace cgnet
static size_t gff_operand_bytes(const cgnet_wmm_plan* plan) {
    return plan->gff_mfma ? sizeof(float) * 64 * (size_t)plan->ap_blocks : sizeof(float) * 2 * (size_t)plan->nW;
}

extern "C" size_t cgnet_FN_WMM_backward_workspace(const cgnet_wmm_plan* plan, int B) {
    if (!plan || B <= 0) return 0;
    // [operand of the FF-gradient kernel] [raw weight-gradient sums per chunk of samples]
    return align_up(gff_operand_bytes(plan), 256) +
           align_up(sizeof(float) * 2 * (size_t)plan->nW * gradw_chunks(B), 256);
}

extern "C" int cgnet_FN_WMM_backward(const cgnet_wmm_plan* plan, const float* d_gO, float* d_gFF, float* d_gW,
                                     const float* d_FF, const float* d_W, int B, const float* d_stds, float eps,
                                     int flags, void* d_workspace, size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    const bool bn = flags & CGNET_FN_BATCHNORM;
    CGNET_REQUIRE(!bn || d_stds, CGNET_ERR_ARG, "batch-norm flag set but d_stds is NULL");
    CGNET_REQUIRE(((uintptr_t)d_gO & 15) == 0 && ((uintptr_t)d_FF & 15) == 0 && ((uintptr_t)d_gFF & 15) == 0,
                  CGNET_ERR_ARG, "d_gO, d_FF and d_gFF must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    const int ndeg = (int)plan->degs.size();
    const size_t need = cgnet_FN_WMM_backward_workspace(plan, B);
    CGNET_REQUIRE(B == 0 || (d_workspace && workspace_bytes >= need), CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, need);
    float2* WT = (float2*)d_workspace;
    float2* gw_part = (float2*)((char*)d_workspace + align_up(gff_operand_bytes(plan), 256));
    if (d_gW && plan->nW > 0) {
        if (B == 0 || plan->nO == 0) {
            const size_t n = (size_t)2 * plan->nW;
            CGNET_LAUNCH(fill_zero_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d_gW, n);
            CGNET_HIP(hipGetLastError());
        } else {
            CGNET_REQUIRE(d_gO && d_FF, CGNET_ERR_ARG, "null device pointer");
            int nchunks = 0;
            if (int rc = wmm_gradw_raw(plan, d_gO, d_FF, (float*)gw_part, B, &nchunks, s)) return rc;
            CGNET_LAUNCH(wmm_gradw_finish_kernel, dim3((plan->nW + 255) / 256), dim3(256), 0, s,
                               (const float2*)gw_part, bn ? d_stds : nullptr, eps, plan->d_degs, ndeg,
                               (float2*)d_gW, plan->nW, nchunks);
            CGNET_HIP(hipGetLastError());
        }
    }
    if (d_gFF && plan->nFF > 0 && B > 0) {
        CGNET_REQUIRE(B <= 65535, CGNET_ERR_UNSUPPORTED, "B=%d above 65535", B);
        CGNET_REQUIRE(d_W, CGNET_ERR_ARG, "d_W is NULL");
        CGNET_REQUIRE(plan->nO == 0 || d_gO, CGNET_ERR_ARG, "d_gO is NULL");
        if (plan->gff_mfma && plan->nW > 0 && plan->nO > 0) {
            float* Ap = (float*)d_workspace;
            const int total = plan->ap_blocks * 8;    // one thread per four weights
            CGNET_LAUNCH(pack_w_gradff_kernel, dim3((total + 255) / 256), dim3(256), 0, s, (const float2*)d_W,
                         bn ? d_stds : nullptr, eps, plan->d_degs, ndeg, Ap, plan->ap_blocks);
            CGNET_HIP(hipGetLastError());
            const int groups = std::max(1, std::min(B, 8));
            const int spg = (B + groups - 1) / groups;
            const int out_bytes = plan->gff_out_cap, go_bytes = plan->gff_go_cap;   // per wave
            const size_t lds = (size_t)out_bytes + 2 * (size_t)go_bytes;
            CGNET_LAUNCH(wmm_gradff_mfma_kernel, dim3(grid_1d(plan->gw_units_rc0.size(), (B + spg - 1) / spg)),
                         dim3(64), lds, s, (const float2*)d_gO, (const float*)Ap, (float2*)d_gFF, plan->d_degs,
                         plan->d_gw_units_rc0, B, spg, plan->nFF, plan->nO, out_bytes, go_bytes);
            CGNET_HIP(hipGetLastError());
            if (!plan->gff_zero_units.empty()) {
                // degrees that produce no output channels: the general kernel writes their zeros
                CGNET_LAUNCH(wmm_gradff_kernel, dim3(grid_1d(plan->gff_zero_units.size(), B)), dim3(kThreads),
                             plan->gff_lds, s, (const float2*)d_gO, (const float2*)nullptr, (float2*)d_gFF,
                             plan->d_degs, plan->d_gff_zero_units, plan->nFF, plan->nO, B);
                CGNET_HIP(hipGetLastError());
            }
        } else {
            if (plan->nW > 0) {
                CGNET_LAUNCH(pack_w_backward_kernel, dim3((plan->nW + 255) / 256), dim3(256), 0, s,
                             (const float2*)d_W, bn ? d_stds : nullptr, eps, plan->d_degs, ndeg, WT, plan->nW);
                CGNET_HIP(hipGetLastError());
            }
            CGNET_LAUNCH(wmm_gradff_kernel, dim3(grid_1d(plan->gff_units.size(), B)), dim3(kThreads),
                         plan->gff_lds, s, (const float2*)d_gO, (const float2*)WT, (float2*)d_gFF, plan->d_degs,
                         plan->d_gff_units, plan->nFF, plan->nO, B);
            CGNET_HIP(hipGetLastError());
        }
    }
    return CGNET_OK;
}
