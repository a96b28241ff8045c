// One CGNet layer (CG product -> fragment norm -> weight mixing) as a unit: the link between a product plan and
// the mixing plan that consumes its output, a forward that prepares in one launch everything the later kernels
// read (packed weights of the mixing, and for the backward the packed weights of the fused kernel, the padded
// fragments and the padded tables), and the entry point of the one-kernel layer backward.
#include <algorithm>
#include <cstring>
#include <memory>

#include "internal.h"

namespace cgnet {
// Compact product tensor of a layer whose FF never leaves it.  For a diagonal triple (l1 = l2) the reference keeps
// both orderings of a channel pair, and FF[(t2, t1)] = (-1)^l FF[(t1, t2)]: the compact layout holds only the
// channels (t1 <= t2, t2) of such a triple, column after column, everything else as in the reference's layout.  The mixing
// then runs over the compact channels with the two weights of a pair added up (pack_w_forward_thread), the weight
// gradient of a pair is one compact entry given to both, and a compact channel's statistics update both stds.
struct CompactLink {
    bool ok = false;
    int nFF = 0, sumT = 0;               // complex entries / channels of one sample's compact FF
    cgnet_wmm_plan* wmm = nullptr;       // mixing plan over the compact channels (owned)
    CgTask* d_tasks = nullptr;           // the product plan's forward tasks, same order, with compact offsets
    int2* d_cmap = nullptr;              // per compact channel: channel of the full layout (over all degrees), mirror or -1
    int* d_f2c = nullptr;                // per full channel: compact channel (over all degrees), bit 31 = takes the sign (-1)^l
};
}  // namespace cgnet

struct cgnet_layer_plan {
    const cgnet_cg_plan* cg = nullptr;
    const cgnet_wmm_plan* wmm = nullptr;
    cgnet::FusedLink link;
    char reason[512] = "";       // why the fused backward does not take this layer ("" if it does)
    cgnet::FwdLink fwd;
    char fwd_reason[512] = "";   // why the fused inference forward does not take it
    cgnet::CompactLink compact;
};

namespace cgnet {
namespace {

// Running fragment-norm values from the per-group partial sums of the product kernel: the groups are added in
// order (as stats_reduce_kernel does), then the moving average is updated (as fn_update_std_kernel does).
__global__ void __launch_bounds__(64)
fn_finish_kernel(const double* __restrict__ part, int ngroups, float* __restrict__ stds,
                 const WmmDeg* __restrict__ degs, int ndeg, int sumT, int B, float cnt) {
    __shared__ int s_tab[kMaxLookup];
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int di = lookup_in_group(ndeg, c, [&](int k) { return degs[k].cumT; }, s_tab);
    if (c >= sumT) return;
    double s1 = 0., s2 = 0.;
    const double2* p = reinterpret_cast<const double2*>(part) + c;
    int g = 0;
    for (; g + 4 <= ngroups; g += 4) {               // four loads in flight, added in group order
        const double2 v0 = p[(size_t)g * sumT], v1 = p[(size_t)(g + 1) * sumT];
        const double2 v2 = p[(size_t)(g + 2) * sumT], v3 = p[(size_t)(g + 3) * sumT];
        s1 += v0.x; s2 += v0.y;
        s1 += v1.x; s2 += v1.y;
        s1 += v2.x; s2 += v2.y;
        s1 += v3.x; s2 += v3.y;
    }
    for (; g < ngroups; ++g) {
        const double2 v = p[(size_t)g * sumT];
        s1 += v.x;
        s2 += v.y;
    }
    stds[c] = updated_std(stds[c], s1, s2, (double)B * (double)degs[di].M, cnt);
}

// The same for a compact product tensor: the sums belong to compact channels, the stds keep the reference's layout;
// a compact channel that stands for a pair updates both entries (each from its own old value).
__global__ void __launch_bounds__(64)
fn_finish_compact_kernel(const double* __restrict__ part, int ngroups, float* __restrict__ stds,
                         const WmmDeg* __restrict__ degs, int ndeg, int sumT, int B, float cnt,
                         const int2* __restrict__ cmap) {
    __shared__ int s_tab[kMaxLookup];
    const int c = blockIdx.x * blockDim.x + threadIdx.x;
    const int di = lookup_in_group(ndeg, c, [&](int k) { return degs[k].cumT; }, s_tab);
    if (c >= sumT) return;
    double s1 = 0., s2 = 0.;
    const double2* p = reinterpret_cast<const double2*>(part) + c;
    int g = 0;
    for (; g + 4 <= ngroups; g += 4) {
        const double2 v0 = p[(size_t)g * sumT], v1 = p[(size_t)(g + 1) * sumT];
        const double2 v2 = p[(size_t)(g + 2) * sumT], v3 = p[(size_t)(g + 3) * sumT];
        s1 += v0.x; s2 += v0.y;
        s1 += v1.x; s2 += v1.y;
        s1 += v2.x; s2 += v2.y;
        s1 += v3.x; s2 += v3.y;
    }
    for (; g < ngroups; ++g) {
        const double2 v = p[(size_t)g * sumT];
        s1 += v.x;
        s2 += v.y;
    }
    const int2 m = cmap[c];
    const double N = (double)B * (double)degs[di].M;
    stds[m.x] = updated_std(stds[m.x], s1, s2, N, cnt);
    if (m.y >= 0) stds[m.y] = updated_std(stds[m.y], s1, s2, N, cnt);
}

// Weight gradient in the reference's layout from the raw sums over compact channels: the chunks of samples are added
// in order, a mirror channel takes the sign (-1)^l, every channel is divided by its own std.
__global__ void __launch_bounds__(256)
gradw_unfold_kernel(const float2* __restrict__ part, int nchunks, int nWc, const float* __restrict__ stds, float eps,
                    const WmmDeg* __restrict__ full, const WmmDeg* __restrict__ comp, int ndeg,
                    const int* __restrict__ f2c, float2* __restrict__ gW, int nW) {
    __shared__ int s_tab[kMaxLookup];
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    const int di = lookup_in_group(ndeg, idx, [&](int k) { return full[k].cumW; }, s_tab);
    if (idx >= nW) return;
    const WmmDeg f = full[di], d = comp[di];
    const int to = (idx - f.cumW) / f.K, c = (idx - f.cumW) - to * f.K;
    const int e = f2c[f.cumT + c];
    const int cc = (e & 0x7fffffff) - d.cumT;                     // compact channel inside the degree
    const size_t src = (size_t)d.cumW + (size_t)to * d.K + cc;
    float2 s = part[src];
    for (int k = 1; k < nchunks; ++k) {
        const float2 v = part[(size_t)k * nWc + src];
        s.x += v.x;
        s.y += v.y;
    }
    if (e < 0 && (f.l & 1)) {
        s.x = -s.x;
        s.y = -s.y;
    }
    if (stds) {
        const float r = fmaxf(eps, stds[f.cumT + c]);
        s.x /= r;
        s.y /= r;
    }
    gW[idx] = s;
}

// Everything the kernels after the statistics read that depends only on W, the (updated) stds, F and the table, in
// one launch; the work-groups are dealt out by role:
//   [0, nb_fwd)      packed weights of the mixing forward               (pack_w_forward_thread; `degs` is the plan the
//                    mixing runs with: the layer's, or the compact one together with degs_full and cmap)
//   [.., + nb_gen)   packed weights of the fused backward, four (task, row tile) pairs each   (pack_w_gen_lane)
//   [.., + nbF)      fragments with a zero behind every row             (pad_fragments_block)
//   [.., + ntab)     every triple's table between zero rows             (pad_table_block)
//   [.., + nb_std)   a copy of the stds (the running values move on with the next batch; the backward of this one
//                    needs those it was normalised with)
__global__ void __launch_bounds__(256)
layer_prepare_kernel(const float2* __restrict__ W, const float* __restrict__ stds, float eps,
                     const WmmDeg* __restrict__ degs, int ndeg, float* __restrict__ Wp, int wp_blocks, int nb_fwd,
                     const WmmDeg* __restrict__ degs_full, const int2* __restrict__ cmap,
                     const GenTask* __restrict__ gens, const int* __restrict__ packmap, int npack, float* __restrict__ Ag,
                     int nb_gen, const float2* __restrict__ F, const float* __restrict__ CG, float2* __restrict__ Fp,
                     float* __restrict__ CGP, const int* __restrict__ padmeta, int L, int nF, int nFp, int B, int nbF,
                     int ntab, float* __restrict__ stds_copy, int sumT) {
    __shared__ int s_tab[kMaxLookup];
    int blk = (int)blockIdx.x;
    if (blk < nb_fwd) {
        pack_w_forward_thread(W, stds, eps, degs, ndeg, Wp, wp_blocks, blk * 256 + (int)threadIdx.x, s_tab, degs_full, cmap);
        return;
    }
    blk -= nb_fwd;
    if (blk < nb_gen) {
        const int pair = blk * 4 + (int)(threadIdx.x >> 6);
        if (pair < npack) pack_w_gen_lane(W, stds, eps, gens[packmap[2 * pair]], packmap[2 * pair + 1], threadIdx.x & 63, Ag);
        return;
    }
    blk -= nb_gen;
    if (blk < nbF) {
        pad_fragments_block(F, Fp, padmeta, L, nF, nFp, B, blk, s_tab);
        return;
    }
    blk -= nbF;
    if (blk < ntab) {
        pad_table_block(CG, CGP, padmeta + 2 * (L + 2) + kPadMetaInts * blk);
        return;
    }
    blk -= ntab;
    const int c = blk * 256 + (int)threadIdx.x;
    if (c < sumT) stds_copy[c] = stds[c];
}

struct SavedAreas { size_t stds, Ag, Fp, CGP, total; };
SavedAreas saved_areas(const cgnet_layer_plan* lp, int B) {
    SavedAreas a{};
    if (!lp->link.ok || B <= 0) return a;
    size_t o = 0;
    a.stds = o; o += align_up(sizeof(float) * (size_t)lp->cg->sumT, 256);   // the stds this batch was normalised with
    a.Ag = o;   o += align_up(sizeof(float) * lp->link.operand_floats, 256);
    a.Fp = o;   o += align_up(sizeof(float) * 2 * (size_t)lp->cg->bwd_nFp * B, 256);
    a.CGP = o;  o += align_up(sizeof(float) * (size_t)lp->cg->bwd_cgp_len, 256);
    a.total = o;
    return a;
}

struct FwdAreas { size_t part, wp, opart, total; int spg, ngroups; };
FwdAreas forward_areas(const cgnet_layer_plan* lp, int B) {
    FwdAreas a{};
    a.spg = samples_per_group_for(B, (int)lp->cg->fwd_tasks.size());
    a.ngroups = (B + a.spg - 1) / a.spg;
    // sized for either layout of the product tensor
    size_t wp = wmm_forward_wp_bytes(lp->wmm), opart = wmm_forward_opart_bytes(lp->wmm, B);
    if (lp->compact.ok) {
        wp = std::max(wp, wmm_forward_wp_bytes(lp->compact.wmm));
        opart = std::max(opart, wmm_forward_opart_bytes(lp->compact.wmm, B));
    }
    size_t o = 0;
    a.part = o;  o += align_up(sizeof(double) * 2 * (size_t)lp->cg->sumT * a.ngroups, 256);
    a.wp = o;    o += align_up(wp, 256);
    a.opart = o; o += align_up(opart, 256);
    a.total = o;
    return a;
}

void free_compact_link(CompactLink* c) {
    if (c->wmm) (void)cgnet_wmm_plan_destroy(c->wmm);
    void* ptrs[] = {c->d_tasks, c->d_cmap, c->d_f2c};
    for (void* q : ptrs)
        if (q) (void)hipFree(q);
    *c = CompactLink();
}

// The compact layout exists where the product runs on the matrix cores and at least one diagonal triple is a single
// forward task (all rows); CGNET_COMPACT_FF=0 switches it off.
int build_compact_link(const cgnet_cg_plan* cg, const cgnet_wmm_plan* wmm, CompactLink* out) {
    *out = CompactLink();
    if (!cg->fwd_mm || cg->nFF == 0) return CGNET_OK;
    if (const char* e = getenv("CGNET_COMPACT_FF"); e && e[0] == '0') return CGNET_OK;
    const int nt = (int)cg->fwd_tasks.size(), L = cg->L;
    std::vector<int> order(nt);
    for (int k = 0; k < nt; ++k) order[k] = k;
    std::sort(order.begin(), order.end(), [&](int a, int b) { return cg->fwd_tasks[a].chan0 < cg->fwd_tasks[b].chan0; });
    std::vector<CgTask> ct = cg->fwd_tasks;
    std::vector<int> tFFc(L + 1, 0), coff(nt, 0);
    int nsym = 0;
    for (int k : order) {
        CgTask& t = ct[k];
        t.sym = (t.l1 == t.l2 && t.t1_begin == 0 && t.rows == t.tau1 && t.tau1 == t.tau2 && t.rows >= 2) ? 1 : 0;
        nsym += t.sym;
        coff[k] = tFFc[t.l];
        tFFc[t.l] += t.sym ? t.rows * (t.rows + 1) / 2 : t.rows * t.tau2;
    }
    if (nsym == 0) return CGNET_OK;
    std::vector<int> cumTc(L + 2, 0), cumFFc(L + 2, 0), tO(L + 1, 0);
    for (int l = 0; l <= L; ++l) {
        cumTc[l + 1] = cumTc[l] + tFFc[l];
        cumFFc[l + 1] = cumFFc[l] + tFFc[l] * (2 * l + 1);
        tO[l] = wmm->degs[l].tO;
    }
    std::vector<int2> cmap(cumTc[L + 1]);
    std::vector<int> f2c(cg->sumT, -1);
    for (int k = 0; k < nt; ++k) {
        CgTask& t = ct[k];
        const int full0 = cg->fwd_tasks[k].chan0, M = 2 * t.l + 1, tau = t.tau2;
        t.chan0 = cumTc[t.l] + coff[k];
        t.offFF = cumFFc[t.l] + coff[k] * M;
        if (t.sym) {
            for (int r = 0; r < tau; ++r)
                for (int c = r; c < tau; ++c) {
                    const int cc = t.chan0 + c * (c + 1) / 2 + r;          // column after column (CgTask::sym)
                    cmap[cc] = make_int2(full0 + r * tau + c, c != r ? full0 + c * tau + r : -1);
                    f2c[full0 + r * tau + c] = cc;
                    if (c != r) f2c[full0 + c * tau + r] = cc | (int)0x80000000;
                }
        } else {
            for (int ch = 0; ch < t.rows * tau; ++ch) {
                cmap[t.chan0 + ch] = make_int2(full0 + ch, -1);
                f2c[full0 + ch] = t.chan0 + ch;
            }
        }
    }
    for (int c = 0; c < cg->sumT; ++c)
        CGNET_REQUIRE(f2c[c] != -1, CGNET_ERR_ARG, "channel %d of the product has no forward task", c);
    CompactLink tmp;
    int rc = cgnet_wmm_plan_create(&tmp.wmm, L, tFFc.data(), tO.data());
    auto upload = [](const void* src, size_t bytes, void** dst) -> int {
        CGNET_HIP(hipMalloc(dst, bytes));
        CGNET_HIP(hipMemcpy(*dst, src, bytes, hipMemcpyHostToDevice));
        return CGNET_OK;
    };
    if (!rc) rc = upload(ct.data(), sizeof(CgTask) * ct.size(), (void**)&tmp.d_tasks);
    if (!rc) rc = upload(cmap.data(), sizeof(int2) * cmap.size(), (void**)&tmp.d_cmap);
    if (!rc) rc = upload(f2c.data(), sizeof(int) * f2c.size(), (void**)&tmp.d_f2c);
    if (rc) {
        free_compact_link(&tmp);
        return rc;
    }
    tmp.nFF = cumFFc[L + 1];
    tmp.sumT = cumTc[L + 1];
    tmp.ok = true;
    *out = tmp;
    return CGNET_OK;
}

struct BwdFusedAreas { BwdAreas own; size_t Ag, Bg, total; };
BwdFusedAreas backward_areas(const cgnet_layer_plan* lp, int B) {
    BwdFusedAreas a{};
    a.own = bwd_areas(lp->cg, B);
    size_t o = a.own.total;
    a.Ag = o; o += align_up(sizeof(float) * lp->link.operand_floats, 256);
    a.Bg = o; o += align_up(sizeof(float) * (size_t)lp->link.bop_floats * B, 256);
    a.total = o;
    return a;
}

}  // namespace
}  // namespace cgnet

using namespace cgnet;

extern "C" int cgnet_layer_plan_create(cgnet_layer_plan** plan, const cgnet_cg_plan* cg_plan,
                                       const cgnet_wmm_plan* wmm_plan) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    *plan = nullptr;
    CGNET_REQUIRE(cg_plan && wmm_plan, CGNET_ERR_ARG, "null plan");
    CGNET_REQUIRE(wmm_plan->L == cg_plan->L, CGNET_ERR_ARG, "the two plans have different lmax (%d, %d)", cg_plan->L,
                  wmm_plan->L);
    for (int l = 0; l <= cg_plan->L; ++l)
        CGNET_REQUIRE(wmm_plan->degs[l].K == cg_plan->t_FF[l], CGNET_ERR_ARG,
                      "degree %d: the mixing plan has %d mid channels, the product %d", l, wmm_plan->degs[l].K,
                      cg_plan->t_FF[l]);
    std::unique_ptr<cgnet_layer_plan> p(new cgnet_layer_plan());
    p->cg = cg_plan;
    p->wmm = wmm_plan;
    const int rc = build_fused_link(cg_plan, wmm_plan, &p->link);
    if (rc == CGNET_ERR_UNSUPPORTED) {
        // the layer still runs, with the two-kernel backward
        std::strncpy(p->reason, cgnet_last_error(), sizeof(p->reason) - 1);
        clear_error();
    } else if (rc != CGNET_OK) {
        return rc;
    }
    const int rc2 = build_fwd_link(cg_plan, wmm_plan, &p->fwd);
    if (rc2 == CGNET_ERR_UNSUPPORTED) {
        std::strncpy(p->fwd_reason, cgnet_last_error(), sizeof(p->fwd_reason) - 1);
        clear_error();
    } else if (rc2 != CGNET_OK) {
        free_fused_link(&p->link);
        return rc2;
    }
    // the compact product tensor serves the route whose backward never reads FF as a whole: the one-kernel backward
    if (p->link.ok) {
        const int rc3 = build_compact_link(cg_plan, wmm_plan, &p->compact);
        if (rc3 != CGNET_OK) {
            free_fwd_link(&p->fwd);
            free_fused_link(&p->link);
            return rc3;
        }
    }
    *plan = p.release();
    return CGNET_OK;
}

extern "C" int cgnet_layer_plan_destroy(cgnet_layer_plan* plan) {
    clear_error();
    if (!plan) return CGNET_OK;
    free_compact_link(&plan->compact);
    free_fwd_link(&plan->fwd);
    free_fused_link(&plan->link);
    delete plan;
    return CGNET_OK;
}

extern "C" int cgnet_CGBN_backward_fused_supported(const cgnet_layer_plan* plan) {
    return plan && plan->link.ok ? 1 : 0;
}

extern "C" const char* cgnet_CGBN_backward_fused_reason(const cgnet_layer_plan* plan) {
    return plan ? plan->reason : "no plan";
}

extern "C" size_t cgnet_CGBN_saved_bytes(const cgnet_layer_plan* plan, int B) {
    return plan ? saved_areas(plan, B).total : 0;
}

extern "C" size_t cgnet_CGBN_saved_stds_bytes(const cgnet_layer_plan* plan, int B) {
    if (!plan || !plan->link.ok || B <= 0) return 0;
    return sizeof(float) * (size_t)plan->cg->sumT;          // the copy sits at the start of the area
}

extern "C" size_t cgnet_CGBN_forward_workspace(const cgnet_layer_plan* plan, int B) {
    if (!plan || B <= 0) return 0;
    return forward_areas(plan, B).total;
}

extern "C" int cgnet_CGBN_forward(const cgnet_layer_plan* plan, const float* d_F, float* d_FF, float* d_O,
                                  const float* d_W, const float* d_CG, int B, float* d_stds, float cnt, float eps,
                                  int flags, void* d_saved, size_t saved_bytes, void* d_workspace,
                                  size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (B == 0) return CGNET_OK;
    const cgnet_cg_plan* cg = plan->cg;
    const cgnet_wmm_plan* wmm = plan->wmm;
    const bool bn = flags & CGNET_FN_BATCHNORM, upd = bn && (flags & CGNET_FN_UPDATE_STD);
    const bool compact = (flags & CGNET_LAYER_COMPACT_FF) != 0;
    CGNET_REQUIRE(!compact || plan->compact.ok, CGNET_ERR_UNSUPPORTED, "this layer has no compact product tensor");
    if (compact) wmm = plan->compact.wmm;                  // the mixing runs over the compact channels
    CGNET_REQUIRE(!bn || d_stds, CGNET_ERR_ARG, "batch-norm flag set but d_stds is NULL");
    CGNET_REQUIRE(cg->nF == 0 || d_F, CGNET_ERR_ARG, "d_F is NULL");
    CGNET_REQUIRE(cg->nFF == 0 || (d_FF && d_CG), CGNET_ERR_ARG, "d_FF or d_CG is NULL");
    CGNET_REQUIRE(wmm->nO == 0 || d_O, CGNET_ERR_ARG, "d_O is NULL");
    CGNET_REQUIRE(wmm->nW == 0 || d_W, CGNET_ERR_ARG, "d_W is NULL");
    const FwdAreas fa = forward_areas(plan, B);
    CGNET_REQUIRE(d_workspace && workspace_bytes >= fa.total, CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, fa.total);
    const SavedAreas sa = saved_areas(plan, B);
    const bool save = d_saved != nullptr && sa.total > 0;
    CGNET_REQUIRE(!save || saved_bytes >= sa.total, CGNET_ERR_WORKSPACE,
                  "saved-operand area of %zu bytes given, %zu needed", saved_bytes, sa.total);
    CGNET_REQUIRE(!save || ((uintptr_t)d_saved & 15) == 0, CGNET_ERR_ARG, "the saved-operand area must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)d_workspace;
    const int ndeg = (int)wmm->degs.size();

    // product, with the per-group partial statistics when the running stds are to be updated
    const bool stats = upd && cg->sumT > 0 && cg->nFF > 0;
    if (cg->nFF > 0) {
        double* part = stats ? (double*)(ws + fa.part) : nullptr;
        const int rc = compact ? cg_launch_forward(cg, d_F, d_FF, d_CG, B, part, fa.spg, s, plan->compact.d_tasks,
                                                   plan->compact.nFF, plan->compact.sumT)
                               : cg_launch_forward(cg, d_F, d_FF, d_CG, B, part, fa.spg, s);
        if (rc) return rc;
    }
    if (stats && compact) {
        const int n = plan->compact.sumT;
        CGNET_LAUNCH(fn_finish_compact_kernel, dim3((n + 63) / 64), dim3(64), 0, s, (const double*)(ws + fa.part),
                     fa.ngroups, d_stds, wmm->d_degs, ndeg, n, B, cnt, plan->compact.d_cmap);
        CGNET_HIP(hipGetLastError());
    } else if (stats) {
        CGNET_LAUNCH(fn_finish_kernel, dim3((cg->sumT + 63) / 64), dim3(64), 0, s, (const double*)(ws + fa.part),
                     fa.ngroups, d_stds, wmm->d_degs, ndeg, cg->sumT, B, cnt);
        CGNET_HIP(hipGetLastError());
    }
    // the operands of the mixing forward and (when asked for) of the backward
    float* Wp = (float*)(ws + fa.wp);
    const bool pack_fwd = wmm->nO > 0 && !wmm->fwd_units.empty();
    const int nb_fwd = pack_fwd ? (wmm->wp_blocks * 16 + 255) / 256 : 0;
    const int nb_gen = save ? (plan->link.npack + 3) / 4 : 0;
    const int nbF = save ? (int)(((size_t)cg->bwd_nFp * B + 255) / 256) : 0;
    const int ntab = save ? cg->nllls : 0;
    const int nb_std = save && bn ? (cg->sumT + 255) / 256 : 0;
    if (nb_fwd + nb_gen + nbF + ntab + nb_std > 0) {
        char* sv = (char*)d_saved;
        CGNET_LAUNCH(layer_prepare_kernel, dim3((unsigned)(nb_fwd + nb_gen + nbF + ntab + nb_std)), dim3(256), 0, s,
                     (const float2*)d_W, bn ? d_stds : nullptr, eps, wmm->d_degs, ndeg, Wp, wmm->wp_blocks, nb_fwd,
                     compact ? plan->wmm->d_degs : nullptr, compact ? plan->compact.d_cmap : nullptr, plan->link.d_gens, plan->link.d_packmap, plan->link.npack, save ? (float*)(sv + sa.Ag) : nullptr,
                     nb_gen, (const float2*)d_F, d_CG, save ? (float2*)(sv + sa.Fp) : nullptr,
                     save ? (float*)(sv + sa.CGP) : nullptr, cg->d_bwd_padmeta, cg->L, cg->nF, cg->bwd_nFp, B, nbF, ntab,
                     save ? (float*)(sv + sa.stds) : nullptr, cg->sumT);
        CGNET_HIP(hipGetLastError());
    }
    return wmm_forward_packed(wmm, d_FF, d_O, Wp, B, ws + fa.opart, s);
}

extern "C" size_t cgnet_CGBN_backward_fused_workspace(const cgnet_layer_plan* plan, int B) {
    if (!plan || B <= 0 || !plan->link.ok) return 0;
    return backward_areas(plan, B).total;
}

extern "C" int cgnet_CGBN_backward_fused(const cgnet_layer_plan* plan, const float* d_F, float* d_gF, const float* d_gO,
                                         const float* d_W, const float* d_CG, int B, const float* d_stds, float eps,
                                         int flags, const void* d_saved, size_t saved_bytes, void* d_workspace,
                                         size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    const cgnet_cg_plan* cg = plan->cg;
    if (B == 0 || cg->nF == 0) return CGNET_OK;
    CGNET_REQUIRE(plan->link.ok, CGNET_ERR_UNSUPPORTED, "%s", plan->reason);
    const bool bn = flags & CGNET_FN_BATCHNORM;
    CGNET_REQUIRE(d_gF && d_gO, CGNET_ERR_ARG, "null device pointer");
    const BwdFusedAreas ba = backward_areas(plan, B);
    CGNET_REQUIRE(d_workspace && workspace_bytes >= ba.total, CGNET_ERR_WORKSPACE,
                  "workspace of %zu bytes given, %zu needed", workspace_bytes, ba.total);
    CGNET_REQUIRE(((uintptr_t)d_workspace & 15) == 0, CGNET_ERR_ARG, "workspace must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    char* ws = (char*)d_workspace;
    const float *Ag, *Fp, *CGP;
    if (d_saved) {
        const SavedAreas sa = saved_areas(plan, B);
        CGNET_REQUIRE(saved_bytes >= sa.total, CGNET_ERR_WORKSPACE, "saved-operand area of %zu bytes given, %zu needed",
                      saved_bytes, sa.total);
        CGNET_REQUIRE(((uintptr_t)d_saved & 15) == 0, CGNET_ERR_ARG, "the saved-operand area must be 16-byte aligned");
        const char* sv = (const char*)d_saved;
        Ag = (const float*)(sv + sa.Ag);
        Fp = (const float*)(sv + sa.Fp);
        CGP = (const float*)(sv + sa.CGP);
    } else {
        CGNET_REQUIRE(!bn || d_stds, CGNET_ERR_ARG, "batch-norm flag set but d_stds is NULL");
        CGNET_REQUIRE(d_F && d_W && d_CG, CGNET_ERR_ARG, "null device pointer");
        if (int rc = launch_pack_w_gen(plan->link, d_W, bn ? d_stds : nullptr, eps, (float*)(ws + ba.Ag), s)) return rc;
        if (int rc = launch_backward_pad(cg, d_F, d_CG, (float*)(ws + ba.own.Fp), (float*)(ws + ba.own.CGP), B, s)) return rc;
        Ag = (const float*)(ws + ba.Ag);
        Fp = (const float*)(ws + ba.own.Fp);
        CGP = (const float*)(ws + ba.own.CGP);
    }
    return launch_fused_backward(cg, plan->link, d_gO, Ag, Fp, CGP, (float*)(ws + ba.Bg), (float*)(ws + ba.own.part1),
                                 (float*)(ws + ba.own.part2), d_gF, B, s);
}

// ---- compact product tensor: sizes, weight gradient --------------------------------------------------
extern "C" int cgnet_CGBN_compact_supported(const cgnet_layer_plan* plan) { return plan && plan->compact.ok ? 1 : 0; }

extern "C" size_t cgnet_CGBN_internal_nFF(const cgnet_layer_plan* plan, int flags) {
    if (!plan) return 0;
    return (flags & CGNET_LAYER_COMPACT_FF) && plan->compact.ok ? (size_t)plan->compact.nFF : (size_t)plan->cg->nFF;
}

extern "C" size_t cgnet_CGBN_backward_gradw_workspace(const cgnet_layer_plan* plan, int B, int flags) {
    if (!plan || B <= 0) return 0;
    if ((flags & CGNET_LAYER_COMPACT_FF) && plan->compact.ok) return align_up(wmm_gradw_part_bytes(plan->compact.wmm, B), 256);
    return cgnet_FN_WMM_backward_workspace(plan->wmm, B);
}

extern "C" int cgnet_CGBN_backward_gradw(const cgnet_layer_plan* plan, const float* d_gO, const float* d_FF, float* d_gW,
                                         int B, const float* d_stds, float eps, int flags, void* d_workspace,
                                         size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (!(flags & CGNET_LAYER_COMPACT_FF))
        return cgnet_FN_WMM_backward(plan->wmm, d_gO, nullptr, d_gW, d_FF, nullptr, B, d_stds, eps,
                                     flags & (CGNET_FN_BATCHNORM | CGNET_FN_UPDATE_STD), d_workspace, workspace_bytes, stream);
    CGNET_REQUIRE(plan->compact.ok, CGNET_ERR_UNSUPPORTED, "this layer has no compact product tensor");
    const cgnet_wmm_plan* wc = plan->compact.wmm;
    const cgnet_wmm_plan* wf = plan->wmm;
    if (wf->nW == 0) return CGNET_OK;
    CGNET_REQUIRE(d_gW, CGNET_ERR_ARG, "d_gW is NULL");
    const bool bn = flags & CGNET_FN_BATCHNORM;
    CGNET_REQUIRE(!bn || d_stds, CGNET_ERR_ARG, "batch-norm flag set but d_stds is NULL");
    hipStream_t s = (hipStream_t)stream;
    if (B == 0 || wf->nO == 0)                             // all zeros, whatever the layout of FF
        return cgnet_FN_WMM_backward(wf, d_gO, nullptr, d_gW, d_FF, nullptr, B, d_stds, eps, flags & CGNET_FN_BATCHNORM,
                                     d_workspace, workspace_bytes, stream);
    CGNET_REQUIRE(d_gO && d_FF, CGNET_ERR_ARG, "null device pointer");
    CGNET_REQUIRE(((uintptr_t)d_gO & 15) == 0 && ((uintptr_t)d_FF & 15) == 0, CGNET_ERR_ARG,
                  "d_gO and d_FF must be 16-byte aligned");
    const size_t need = cgnet_CGBN_backward_gradw_workspace(plan, B, flags);
    CGNET_REQUIRE(d_workspace && workspace_bytes >= need, CGNET_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed",
                  workspace_bytes, need);
    int nchunks = 0;
    if (int rc = wmm_gradw_raw(wc, d_gO, d_FF, (float*)d_workspace, B, &nchunks, s)) return rc;
    CGNET_LAUNCH(gradw_unfold_kernel, dim3((wf->nW + 255) / 256), dim3(256), 0, s, (const float2*)d_workspace, nchunks,
                 wc->nW, bn ? d_stds : nullptr, eps, wf->d_degs, wc->d_degs, (int)wf->degs.size(), plan->compact.d_f2c,
                 (float2*)d_gW, wf->nW);
    CGNET_HIP(hipGetLastError());
    return CGNET_OK;
}

// ---- inference forward without FF ---------------------------------------------------------------------
extern "C" int cgnet_CGBN_forward_inference_supported(const cgnet_layer_plan* plan) { return plan && plan->fwd.ok ? 1 : 0; }

extern "C" const char* cgnet_CGBN_forward_inference_reason(const cgnet_layer_plan* plan) {
    return plan ? plan->fwd_reason : "no plan";
}

extern "C" size_t cgnet_CGBN_forward_inference_workspace(const cgnet_layer_plan* plan, int B) {
    if (!plan || !plan->fwd.ok || B <= 0) return 0;
    return align_up(sizeof(float) * plan->fwd.a_floats, 256) + align_up(sizeof(float) * 2 * (size_t)plan->fwd.opart * B, 256);
}

extern "C" int cgnet_CGBN_forward_inference(const cgnet_layer_plan* plan, const float* d_F, float* d_O, const float* d_W,
                                            const float* d_CG, int B, const float* d_stds, float eps, int flags,
                                            void* d_workspace, size_t workspace_bytes, void* stream) {
    clear_error();
    CGNET_REQUIRE(plan, CGNET_ERR_ARG, "plan is NULL");
    CGNET_REQUIRE(B >= 0, CGNET_ERR_ARG, "B=%d is negative", B);
    if (B == 0 || plan->wmm->nO == 0) return CGNET_OK;
    CGNET_REQUIRE(plan->fwd.ok, CGNET_ERR_UNSUPPORTED, "%s", plan->fwd_reason);
    const bool bn = flags & CGNET_FN_BATCHNORM;
    CGNET_REQUIRE(!(flags & CGNET_FN_UPDATE_STD), CGNET_ERR_ARG,
                  "the inference forward cannot update the running stds (they depend on the whole batch's product)");
    CGNET_REQUIRE(!bn || d_stds, CGNET_ERR_ARG, "batch-norm flag set but d_stds is NULL");
    CGNET_REQUIRE(d_O && (plan->cg->nF == 0 || d_F) && (plan->wmm->nW == 0 || d_W) && (plan->cg->nFF == 0 || d_CG), CGNET_ERR_ARG,
                  "null device pointer");
    const size_t need = cgnet_CGBN_forward_inference_workspace(plan, B);
    CGNET_REQUIRE(d_workspace && workspace_bytes >= need, CGNET_ERR_WORKSPACE, "workspace of %zu bytes given, %zu needed",
                  workspace_bytes, need);
    CGNET_REQUIRE(((uintptr_t)d_workspace & 15) == 0, CGNET_ERR_ARG, "workspace must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    float* Af = (float*)d_workspace;
    float* Opart = (float*)((char*)d_workspace + align_up(sizeof(float) * plan->fwd.a_floats, 256));
    if (int rc = launch_pack_w_mix(plan->cg, plan->fwd, d_W, bn ? d_stds : nullptr, eps, Af, s)) return rc;
    return launch_forward_fused(plan->cg, plan->fwd, d_F, d_CG, Af, Opart, d_O, B, s);
}
