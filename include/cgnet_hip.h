/*
 * cgnet_hip.h -- C ABI of libcgnet_hip.so: the Clebsch-Gordan layer hot path on MI355X (gfx950).
 *
 * Every entry point takes plain pointers and sizes.  Device pointers are marked d_, host
 * pointers h_.  `stream` is a hipStream_t passed as void* (NULL = the default stream); work
 * is enqueued on it and the call returns without synchronising the device.  Return value:
 * CGNET_OK or a negative CGNET_ERR_* code; cgnet_last_error() then holds a message for the
 * calling thread.  The caller owns every buffer, outputs included (as in the reference, where
 * the Python side allocates outputs and the native side fills them in place).
 *
 * Each function names the reference interface it stands in for.  File:line citations are
 * relative to the reference checkout (zlin7/CGNet).  The reference binds these operations
 * through the pybind11 module `CG_cuda_ops` (CGNet/cudaCG/cudaCG_all.cpp:207-215); that
 * module passes int32 device tensors for the per-degree metadata, which forces the kernels to
 * re-derive the layout on every call.  Here the metadata is handed over once, from host
 * arrays, into a plan object; the per-call functions then take only data pointers.
 *
 * Tensor layouts (all float32, complex numbers interleaved (re, im)):
 *   "straight" fragments  F  [B][nF ][2], nF  = sum_l t_F [l](2l+1); inside degree l: [t][m]
 *   CG product            FF [B][nFF][2], nFF = sum_l t_FF[l](2l+1)
 *   layer output          O  [B][nO ][2], nO  = sum_l t_O [l](2l+1)
 *   weights               W  [nW][2], nW = sum_l t_O[l]*t_FF[l]; degree l is a row-major
 *                            (t_O[l], t_FF[l]) complex matrix
 *   CG table              CG [cg_len]; triple i owns (2l+1)(2l2+1) floats at CG_offsets[i],
 *                            entry [m+l][m2+l2] = <l1 m-m2 l2 m2 | l m>, 0 where |m-m2| > l1
 */
#ifndef CGNET_HIP_H
#define CGNET_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CGNET_OK               0
#define CGNET_ERR_ARG         (-1)   /* null pointer, negative size, inconsistent metadata */
#define CGNET_ERR_HIP         (-2)   /* a HIP runtime call failed */
#define CGNET_ERR_WORKSPACE   (-3)   /* workspace missing or smaller than *_workspace() */
#define CGNET_ERR_UNSUPPORTED (-4)   /* size beyond what the kernels are built for */

/* fragment-norm flags of FN_WMM_forward / FN_WMM_backward (CGNet/CG_layers.py:22-33) */
#define CGNET_FN_BATCHNORM   0x1     /* divide each mid channel by max(eps, std) */
#define CGNET_FN_UPDATE_STD  0x2     /* fold this batch into the running stds before use */

typedef struct cgnet_cg_plan  cgnet_cg_plan;
typedef struct cgnet_wmm_plan cgnet_wmm_plan;

/* Message describing the last error on the calling thread ("" if none). */
const char* cgnet_last_error(void);

/* ABI revision of this header. */
int cgnet_abi_version(void);

/* Largest supported lmax.  Replaces CG_cuda_ops.sparse_maxL (cudaCG_all.cpp:130-132). */
int cgnet_sparse_maxL(void);

/* Fill the flat Clebsch-Gordan table on the device (double-precision Racah sum, stored as
 * float).  Replaces CG_cuda_ops.sparse_precomputeCG (cudaCG_all.cpp:114-127; kernel
 * cudaCG_sparse.cu:68-92, host :304-317).  h_llls[i] = (l*(L+1)+l1)*(L+1)+l2 with l1 >= l2;
 * h_CG_offsets has nllls+1 entries.  Every entry of the table is written (zeros included). */
int cgnet_sparse_precomputeCG(float* d_CG, int L, const int* h_llls, int nllls,
                              const int* h_CG_offsets, void* stream);

/* ---- Clebsch-Gordan product ------------------------------------------------------------ */

/* Build the plan of one CG product: h_t_F[L+1] input channels per degree, h_llls[nllls] kept
 * triples in the order that fixes the output channel order.  h_t_offsets (nllls entries,
 * channel offset of each triple inside its output degree) and h_CG_offsets (nllls+1) may be
 * NULL, in which case they are the running sums the reference computes at
 * CGNet/CG_layers.py:253-262 and CGNet/CGutils.py:179-187.  Stands in for the int32 device
 * tensors t_F, cumu_tm_F, t_FF, cumu_tm_FF, llls, l_l1_to_lllidx_offsets, t_offsets,
 * CG_offsets that the reference passes on every call (cudaCG_all.cpp:39-51). */
int cgnet_cg_plan_create(cgnet_cg_plan** plan, int L, const int* h_t_F, const int* h_llls, int nllls,
                         const int* h_t_offsets, const int* h_CG_offsets);
int cgnet_cg_plan_destroy(cgnet_cg_plan* plan);
/* sizes[0..4] = nF, nFF, sum_l t_FF[l], cg_len, nllls */
int cgnet_cg_plan_sizes(const cgnet_cg_plan* plan, int sizes[5]);
/* h_t_FF[L+1], h_t_offsets[nllls]; either may be NULL */
int cgnet_cg_plan_channels(const cgnet_cg_plan* plan, int* h_t_FF, int* h_t_offsets);
/* LDS bytes one work-group of the product's backward kernel holds (0 without a plan).  No counterpart in the
 * reference: a scheduling hint for callers that run another kernel on a second stream beside the backward
 * (a compute unit has 160 KB; what two such groups leave decides whether the other kernel fits beside them). */
size_t cgnet_cg_plan_backward_lds(const cgnet_cg_plan* plan);
/* The same for the forward kernel (its largest launch class).  No counterpart in the reference. */
size_t cgnet_cg_plan_forward_lds(const cgnet_cg_plan* plan);
/* Work-groups of the backward kernel that share a compute unit (its LDS need and register budget decide); with
 * cgnet_cg_plan_backward_lds the LDS the backward occupies.  No counterpart in the reference. */
int cgnet_cg_plan_backward_groups(const cgnet_cg_plan* plan);

/* FF = CG product of F with itself over the plan's triples:
 *   FF[b, l, t_off + t1*t_F[l2] + t2, m] = sum_{m1+m2=m} CG * F[b,l1,t1,m1] * F[b,l2,t2,m2].
 * Replaces CG_cuda_ops.sparse_forward (cudaCG_all.cpp:39-71; kernel cudaCG_sparse.cu:96-184).
 * Every element of d_FF is written; it need not be zeroed. */
int cgnet_sparse_forward(const cgnet_cg_plan* plan, const float* d_F, float* d_FF,
                         const float* d_CG, int B, void* stream);

/* Same product that also returns, per mid channel c, sum_{b,m} |FF| and sum_{b,m} |FF|^2 in
 * d_sums[2*c], d_sums[2*c+1] (double), so that the fragment-norm statistics need no second
 * pass over FF.  No counterpart in the reference (its statistics kernel
 * cudaCG_FNWMM.cu:29-79 re-reads FF); the result feeds cgnet_FN_WMM_forward(d_sums=...). */
size_t cgnet_sparse_forward_stats_workspace(const cgnet_cg_plan* plan, int B);
int cgnet_sparse_forward_stats(const cgnet_cg_plan* plan, const float* d_F, float* d_FF,
                               const float* d_CG, int B, double* d_sums,
                               void* d_workspace, size_t workspace_bytes, void* stream);

/* cgnet_sparse_forward_stats for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the same product and the same sums,
 * bit for bit, but the partial sums live in a fixed area of cgnet_sparse_forward_stats_static_limit()
 * bytes (16 MiB) inside the library instead of a caller workspace, and the call allocates nothing.
 * It has no counterpart in the reference.  A call whose partial sums need more (16 * sum_l t_FF[l] *
 * sample groups bytes, i.e. cgnet_sparse_forward_stats_workspace) returns CGNET_ERR_UNSUPPORTED.
 * All calls on one GPU share that area: calls that overlap on one GPU (two streams, two threads)
 * race; calls on one stream are ordered and safe. */
size_t cgnet_sparse_forward_stats_static_limit(void);
int cgnet_sparse_forward_stats_static(const cgnet_cg_plan* plan, const float* d_F, float* d_FF,
                                      const float* d_CG, int B, double* d_sums, void* stream);

/* Gradient of the product with respect to F given d_gFF = dLoss/dFF:
 *   gF[b,l1,t1,m1] = sum CG * gFF[b,l,t,m1+m2] * conj(F[b,l2,t2,m2])  + the same with the
 *   roles of the two slots exchanged (a diagonal triple l1 == l2 contributes through both).
 * Replaces CG_cuda_ops.sparse_backward (cudaCG_all.cpp:73-108; kernel cudaCG_sparse.cu:186-298).
 * Deterministic.  Every element of d_gF is written. */
size_t cgnet_sparse_backward_workspace(const cgnet_cg_plan* plan, int B);
int cgnet_sparse_backward(const cgnet_cg_plan* plan, const float* d_F, float* d_gF,
                          const float* d_gFF, const float* d_CG, int B,
                          void* d_workspace, size_t workspace_bytes, void* stream);

/* ---- fragment norm + per-degree complex weight mixing -------------------------------- */

/* Plan for mixing h_t_FF[l] mid channels into h_t_O[l] output channels, l = 0..L.  Stands in
 * for the device tensors t_FF, cumu_tm_FF, t_O, cumu_tm_O, cumu_tt_W (cudaCG_all.cpp:137-146). */
int cgnet_wmm_plan_create(cgnet_wmm_plan** plan, int L, const int* h_t_FF, const int* h_t_O);
int cgnet_wmm_plan_destroy(cgnet_wmm_plan* plan);
/* sizes[0..3] = nFF, nO, nW, sum_l t_FF[l] */
int cgnet_wmm_plan_sizes(const cgnet_wmm_plan* plan, int sizes[4]);
/* LDS bytes one work-group of the weight-gradient kernel holds (0 without a plan); a scheduling hint like
 * cgnet_cg_plan_backward_lds, no counterpart in the reference. */
size_t cgnet_wmm_plan_gradw_lds(const cgnet_wmm_plan* plan);

/* O[b,l,to,m] = sum_c W[l,to,c] * FF[b,l,c,m] / max(eps, stds[c])   (no division without
 * CGNET_FN_BATCHNORM).  With CGNET_FN_UPDATE_STD the running stds are first updated in place:
 *   s = population std over (b, m) of |FF[b,l,c,m]|;  stds[c] = stds[c]*cnt/(cnt+1) + s/(cnt+1)
 * and the updated value normalises this very batch.  d_sums, if not NULL, holds the per-channel
 * sums produced by cgnet_sparse_forward_stats and replaces the statistics pass over FF.
 * Replaces CG_cuda_ops.FN_WMM_forward (cudaCG_all.cpp:137-165; kernels cudaCG_FNWMM.cu:29-123,
 * host :215-245).  d_stds may be NULL when CGNET_FN_BATCHNORM is not set. */
size_t cgnet_FN_WMM_forward_workspace(const cgnet_wmm_plan* plan, int B);
int cgnet_FN_WMM_forward(const cgnet_wmm_plan* plan, const float* d_FF, float* d_O, const float* d_W,
                         int B, float* d_stds, float cnt, float eps, int flags, const double* d_sums,
                         void* d_workspace, size_t workspace_bytes, void* stream);

/* gW[l,to,c]   = sum_{b,m} gO[b,l,to,m] * conj(FF[b,l,c,m]) / max(eps, stds[c])
 * gFF[b,l,c,m] = (sum_to conj(W[l,to,c]) * gO[b,l,to,m]) / max(eps, stds[c])
 * with the stds treated as constants.  Replaces CG_cuda_ops.FN_WMM_backward
 * (cudaCG_all.cpp:172-205; kernels cudaCG_FNWMM.cu:126-211, host :250-282).  Unlike the
 * reference (float atomics over the batch) the gW reduction is deterministic.  Every element
 * of d_gFF and d_gW is written.  Either of d_gFF / d_gW may be NULL to skip that output. */
size_t cgnet_FN_WMM_backward_workspace(const cgnet_wmm_plan* plan, int B);
int cgnet_FN_WMM_backward(const cgnet_wmm_plan* plan, const float* d_gO, float* d_gFF, float* d_gW,
                          const float* d_FF, const float* d_W, int B, const float* d_stds,
                          float eps, int flags,
                          void* d_workspace, size_t workspace_bytes, void* stream);

/* ---- the layer as a unit (no counterpart in the reference) ------------------------------------------ */

/* One CGNet layer, F -> CG product -> fragment norm + weight mixing -> O (CGBN_cuda.forward, CGNet/CG_layers.py:313-318),
 * as a unit.  The reference chains two autograd Functions that meet at the materialised tensors FF and grad_FF
 * (CG_layers.py:14-72,168-203); inside the layer neither is visible to the user, which these entry points use:
 * the forward prepares in one launch every operand the later kernels read, and the backward can go from gO to gF
 * in one kernel without grad_FF in memory.
 *
 * A layer plan links a product plan with the mixing plan that consumes its output (t_FF must agree).  It keeps
 * pointers to both, which must outlive it, and a little device memory of its own (allocated here, at creation, on
 * the current device; never changed afterwards, so concurrent calls need no lock and no per-call entry point
 * allocates). */
typedef struct cgnet_layer_plan cgnet_layer_plan;
int cgnet_layer_plan_create(cgnet_layer_plan** plan, const cgnet_cg_plan* cg_plan, const cgnet_wmm_plan* wmm_plan);
int cgnet_layer_plan_destroy(cgnet_layer_plan* plan);

/* 1 if cgnet_CGBN_backward_fused takes this layer (every input channel count in 8..16, lmax <= 23, t_O <= 16,
 * LDS within limits), else 0; cgnet_CGBN_backward_fused_reason then names what is missing. */
int cgnet_CGBN_backward_fused_supported(const cgnet_layer_plan* plan);
const char* cgnet_CGBN_backward_fused_reason(const cgnet_layer_plan* plan);

/* O = layer(F): cgnet_sparse_forward_stats (statistics only with CGNET_FN_UPDATE_STD) followed by
 * cgnet_FN_WMM_forward(d_sums = ...), same arithmetic and same results bit for bit, in fewer launches: the
 * statistics are reduced and the running stds updated in one kernel, and one further kernel packs the weights of
 * the mixing and -- when d_saved is given -- the three operands cgnet_CGBN_backward_fused would otherwise build
 * itself (packed W / max(eps, stds) per task, F with a zero behind every row, the tables between zero rows), all of
 * which depend only on what the forward already holds.  d_FF (B x nFF complex) is written as by
 * cgnet_sparse_forward: the weight gradient needs it.  d_saved: cgnet_CGBN_saved_bytes(plan, B) bytes, 16-byte
 * aligned, or NULL (inference; also when the fused backward is not supported, where the size is 0).
 * d_stds / cnt / eps / flags as in cgnet_FN_WMM_forward. */
size_t cgnet_CGBN_saved_bytes(const cgnet_layer_plan* plan, int B);
/* With CGNET_FN_BATCHNORM the area starts with a copy of the stds this batch was normalised with (float,
 * cgnet_CGBN_saved_stds_bytes(plan, B) bytes = 4 * sum_l t_FF[l]; 0 when nothing is saved): the running values
 * move on with the next batch, and the weight gradient of this one (cgnet_FN_WMM_backward, d_stds) needs these. */
size_t cgnet_CGBN_saved_stds_bytes(const cgnet_layer_plan* plan, int B);
size_t cgnet_CGBN_forward_workspace(const cgnet_layer_plan* plan, int B);
int cgnet_CGBN_forward(const cgnet_layer_plan* plan, const float* d_F, float* d_FF, float* d_O, const float* d_W,
                       const float* d_CG, int B, float* d_stds, float cnt, float eps, int flags,
                       void* d_saved, size_t saved_bytes, void* d_workspace, size_t workspace_bytes, void* stream);

/* gF = dLoss/dF of the layer from d_gO = dLoss/dO, i.e. what cgnet_FN_WMM_backward(d_gFF = ...) followed by
 * cgnet_sparse_backward(d_gFF) returns in d_gF, without the intermediate gradient gFF (B x nFF complex) ever
 * existing in memory: every tile of it is formed in LDS on the matrix cores from gO and W / div right where the
 * product's backward consumes it.  The weight gradient still comes from cgnet_FN_WMM_backward (d_gFF = NULL).
 * With d_saved (the area cgnet_CGBN_forward filled for the same F, W, stds, table and B) d_F, d_W, d_CG and d_stds
 * are not read and may be NULL; with d_saved = NULL the call builds those operands itself (two more launches).
 * d_stds / eps / flags as in cgnet_FN_WMM_backward (the stds the forward pass used, treated as constants).
 * Returns CGNET_ERR_UNSUPPORTED where cgnet_CGBN_backward_fused_supported is 0.  Allocates nothing. */
size_t cgnet_CGBN_backward_fused_workspace(const cgnet_layer_plan* plan, int B);
int cgnet_CGBN_backward_fused(const cgnet_layer_plan* plan, const float* d_F, float* d_gF, const float* d_gO,
                              const float* d_W, const float* d_CG, int B, const float* d_stds, float eps, int flags,
                              const void* d_saved, size_t saved_bytes,
                              void* d_workspace, size_t workspace_bytes, void* stream);

/* O = layer(F) for inference, without the product tensor FF (B x nFF complex) ever existing in memory: every tile
 * of it is mixed with its slice of W / max(eps, stds) on the matrix cores while it lies in LDS, and what leaves the
 * product kernel is a partial output per kept triple (t_O x (2l+1) values for a tile of t_F[l1] t_F[l2] x (2l+1)); a second
 * kernel adds the partial outputs of a degree in channel order.  Same result as cgnet_CGBN_forward up to the order of
 * the additions.  The running stds cannot be updated on this route (CGNET_FN_UPDATE_STD is refused): normalising a
 * batch with its own statistics needs the whole batch's product first.  It serves CGBN_cuda in evaluation mode
 * (CGNet/CG_layers.py:313-318 with self.training false) and layers without fragment norm, when no gradient is
 * wanted.  Supported where the product runs on the matrix cores (every input channel count in 8..16), lmax <= 15
 * and t_O <= 16; cgnet_CGBN_forward_inference_supported / _reason as for the fused backward.  Allocates nothing. */
int cgnet_CGBN_forward_inference_supported(const cgnet_layer_plan* plan);
const char* cgnet_CGBN_forward_inference_reason(const cgnet_layer_plan* plan);
size_t cgnet_CGBN_forward_inference_workspace(const cgnet_layer_plan* plan, int B);
int cgnet_CGBN_forward_inference(const cgnet_layer_plan* plan, const float* d_F, float* d_O, const float* d_W,
                                 const float* d_CG, int B, const float* d_stds, float eps, int flags,
                                 void* d_workspace, size_t workspace_bytes, void* stream);

/* Compact product tensor.  For a triple with l1 = l2 the reference keeps both orderings (t1, t2), (t2, t1) of every
 * channel pair (CGNet/CG_layers.py:253-262), and FF[(t2, t1)] = (-1)^l FF[(t1, t2)]: 8 % of FF at L=11, tau=12 is
 * redundant.  Inside the layer FF is invisible to the user, so with CGNET_LAYER_COMPACT_FF in `flags`
 * cgnet_CGBN_forward writes only the channels (t1 <= t2, t2) of such triples (cgnet_CGBN_internal_nFF(plan, flags)
 * complex entries per sample instead of nFF), mixes them with the two weights of a pair added up, and updates the
 * stds of both channels of a pair from the pair's one set of sums.  O, the stds and the saved operands are the same
 * as without the flag up to rounding.  A compact FF serves exactly two consumers: cgnet_CGBN_backward_gradw (below)
 * and nothing else -- cgnet_FN_WMM_backward and cgnet_sparse_backward expect the reference's layout -- so the flag
 * belongs with the one-kernel backward, which reads no FF.  cgnet_CGBN_compact_supported: 1 where the one-kernel
 * backward is supported, the product runs on the matrix cores and some diagonal triple is a single forward task.
 * gW of the layer (what cgnet_FN_WMM_backward(d_gFF = NULL) returns in d_gW) from gO and the FF that
 * cgnet_CGBN_forward wrote with the same `flags` (without the compact flag this IS cgnet_FN_WMM_backward).
 * d_stds: the stds the batch was normalised with (reference layout).  Allocates nothing. */
#define CGNET_LAYER_COMPACT_FF 0x4
int cgnet_CGBN_compact_supported(const cgnet_layer_plan* plan);
size_t cgnet_CGBN_internal_nFF(const cgnet_layer_plan* plan, int flags);
size_t cgnet_CGBN_backward_gradw_workspace(const cgnet_layer_plan* plan, int B, int flags);
int cgnet_CGBN_backward_gradw(const cgnet_layer_plan* plan, const float* d_gO, const float* d_FF, float* d_gW, int B,
                              const float* d_stds, float eps, int flags, void* d_workspace, size_t workspace_bytes,
                              void* stream);

/* ---- measurement hooks (no counterpart in the reference, which times nothing) ------------ */

/* With timing enabled every kernel launch of this library is bracketed by two HIP events
 * recorded on the launch stream.  After the caller has synchronised those streams,
 * cgnet_profile_collect() folds the finished pairs into per-kernel totals and returns the
 * number of distinct kernels; cgnet_profile_get(i, ...) reads entry i (name, summed
 * milliseconds, launches).  cgnet_profile_enable returns the previous setting.
 * cgnet_profile_select("kernel") restricts the bracketing to launches of that one kernel
 * (recording events costs a few microseconds per launch, which a timed region that only wants
 * one kernel's duration need not pay for the others); NULL or "" selects every kernel again. */
int cgnet_profile_enable(int on);
int cgnet_profile_select(const char* kernel_name);
int cgnet_profile_reset(void);
int cgnet_profile_collect(void);
int cgnet_profile_get(int index, char* name, int name_capacity, double* total_ms, int* launches);

#ifdef __cplusplus
}
#endif
#endif /* CGNET_HIP_H */
