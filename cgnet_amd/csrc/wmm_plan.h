// Types of the fragment-norm + weight-mixing plan shared by the translation units of libcgnet_hip.
#pragma once
#include <vector>

#include "common.h"

namespace cgnet {


struct WmmDeg {
    int l, M;          // degree, 2l+1
    int K, tO;         // mid channels, output channels
    int cumFF, cumO;   // complex offsets of the degree inside a sample's FF / O
    int cumW;          // complex offset of the degree's weights
    int cumT;          // first mid channel of the degree among all mid channels
    int nrc;           // row chunks of 16 output channels
    int wp_base;       // first 64-float block of the degree in the packed weights
    int G, NC;         // forward: samples per work-group, 32-column chunks per wave
    int S;             // forward: number of k-slices
    int nks_b;         // gradient wrt FF: k-steps of 4 over the 2*tO real rows (re, im interleaved)
    int ap_base;       // first 64-float block of the degree in the packed conj(W)/div operand
};

struct WmmFwdUnit { int deg, rc, slice, k_begin, k_end; };
struct WmmChanUnit { int deg, rc, c0, nc; };   // a chunk of mid channels of one degree

}  // namespace cgnet

struct cgnet_wmm_plan {
    int L = 0;
    int nFF = 0, nO = 0, nW = 0, sumT = 0;
    int wp_blocks = 0;     // 64-float blocks of the packed forward weights
    int ap_blocks = 0;     // 64-float blocks of the packed operand of the FF-gradient kernel
    bool gff_mfma = true;  // every degree has t_O <= 16 (the operand then fits eight registers)
    int gw_ff_cap = 2, gw_go_cap = 2;   // LDS capacities (complex entries) of one stage of the weight-gradient kernel
    int fwd_stage_cap = 16;             // LDS bytes of one stage of one wave of the forward kernel
    int gff_out_cap = 16, gff_go_cap = 16; // LDS bytes per wave of the FF-gradient kernel: result tile / one gO buffer
    int maxS = 1, maxG = 1;
    std::vector<cgnet::WmmDeg> degs;
    std::vector<cgnet::WmmFwdUnit> fwd_units;   // units of degrees with NC <= 3 first
    int fwd_units_small = 0;
    std::vector<cgnet::WmmChanUnit> gw_units, gw_units_rc0, gff_units, gff_zero_units, stat_units;
    std::vector<int> cumO_all, cumFF_all;   // L+2 entries, for element -> degree lookups
    cgnet::WmmDeg* d_degs = nullptr;
    cgnet::WmmFwdUnit* d_fwd_units = nullptr;
    cgnet::WmmChanUnit* d_gw_units = nullptr;
    cgnet::WmmChanUnit* d_gw_units_rc0 = nullptr;   // one entry per 64-channel chunk (row chunk 0 only)
    cgnet::WmmChanUnit* d_gff_units = nullptr;
    cgnet::WmmChanUnit* d_gff_zero_units = nullptr;   // channels of degrees without outputs: their gradient is zero
    cgnet::WmmChanUnit* d_stat_units = nullptr;
    int* d_cumO = nullptr;      // per deg index: cumO, and S, interleaved: [ndeg+1] cumO then [ndeg] S
    size_t stat_lds = 0, gff_lds = 0;
};


namespace cgnet {

// Running fragment-norm value after this batch: population std of |z| over the N = B(2l+1) entries of the channel
// from the sums of |z| and |z|^2, folded into the moving average exactly as the reference does
// (cudaCG_FNWMM.cu:58-74).
__device__ __forceinline__ float updated_std(float old, double s1, double s2, double N, float cnt) {
    const double mean = s1 / N;
    const double var = s2 / N - mean * mean;
    const double sd = var > 0. ? sqrt(var) : 0.;
    float m = old;
    m *= cnt / (cnt + 1.f);
    return (float)((double)m + sd / (double)(cnt + 1.f));
}

// Packed forward weights: for every degree, block of 8 channels kb and row chunk rc: 256 floats, lane-major,
// four per lane = (k-step 0 | 1) x (W_re | W_im) of W[rc*16+row][kb*8 + 4*step + kk] / div with
// lane = 16*kk + row.  Thread `idx` writes the four floats of one lane (two weights, one 16-byte store).  Every thread
// of the group must call (one barrier inside).
// With a channel map the plan `degs` counts compact mid channels while W and stds keep the layout of `full`: compact
// channel c of a degree stands for the channel cmap[cumT + c].x (index over all degrees of the full layout) and, where
// cmap[..].y >= 0, also for that mirror channel, whose product entries are (-1)^l times the first one's; its weight
// is then the sum of the two normalised weights.
__device__ __forceinline__ void pack_w_forward_thread(const float2* __restrict__ W, const float* __restrict__ stds,
                                                      float eps, const WmmDeg* __restrict__ degs, int ndeg,
                                                      float* __restrict__ Wp, int total_blocks, int idx, int* s_tab,
                                                      const WmmDeg* __restrict__ full = nullptr,
                                                      const int2* __restrict__ cmap = nullptr) {
    const int blk = idx >> 4;                                     // 64-float block of the packed array
    const int di = lookup_in_group(ndeg, blk, [&](int k) { return degs[k].wp_base; }, s_tab);
    if (blk >= total_blocks) return;
    const WmmDeg d = degs[di];
    const int rel = idx - d.wp_base * 16;
    const int lane = rel & 63, grp = rel >> 6;
    const int rc = grp % d.nrc, kb = grp / d.nrc;
    const int row = lane & 15, kk = lane >> 4;
    const int to = rc * 16 + row;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (to < d.tO) {
        const int c0 = kb * 8 + kk, c1 = c0 + 4;
        if (cmap) {
            const WmmDeg f = full[di];
            const float2* wrow = W + f.cumW + (size_t)to * f.K;             // the row; cmap holds channels over all degrees
            const float sgn = (d.l & 1) ? -1.f : 1.f;
            auto folded = [&](int c) {
                float2 w = make_float2(0.f, 0.f);
                if (c < d.K) {
                    const int2 m = cmap[d.cumT + c];
                    w = wrow[m.x - f.cumT];
                    if (stds) {
                        const float r = fmaxf(eps, stds[m.x]);
                        w.x /= r;
                        w.y /= r;
                    }
                    if (m.y >= 0) {
                        float2 u = wrow[m.y - f.cumT];
                        if (stds) {
                            const float r = fmaxf(eps, stds[m.y]);
                            u.x /= r;
                            u.y /= r;
                        }
                        w.x += sgn * u.x;
                        w.y += sgn * u.y;
                    }
                }
                return w;
            };
            const float2 w0 = folded(c0), w1 = folded(c1);
            v = make_float4(w0.x, w0.y, w1.x, w1.y);
        } else {
            const float2* wrow = W + d.cumW + (size_t)to * d.K;
            float2 w0 = make_float2(0.f, 0.f), w1 = w0;
            float r0 = 1.f, r1 = 1.f;
            if (c0 < d.K) {
                w0 = wrow[c0];
                if (stds) r0 = fmaxf(eps, stds[d.cumT + c0]);
            }
            if (c1 < d.K) {
                w1 = wrow[c1];
                if (stds) r1 = fmaxf(eps, stds[d.cumT + c1]);
            }
            v = stds ? make_float4(w0.x / r0, w0.y / r0, w1.x / r1, w1.y / r1) : make_float4(w0.x, w0.y, w1.x, w1.y);
        }
    }
    reinterpret_cast<float4*>(Wp)[idx] = v;
}

}  // namespace cgnet
