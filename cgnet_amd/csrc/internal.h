// Host-side functions the translation units of libcgnet_hip call in each other (not part of the C ABI).
#pragma once
#include "common.h"
#include "cg_plan.h"
#include "wmm_plan.h"

namespace cgnet {

// ---- fnwmm.hip
size_t wmm_forward_wp_bytes(const cgnet_wmm_plan* plan);              // packed forward weights
size_t wmm_forward_opart_bytes(const cgnet_wmm_plan* plan, int B);    // partial outputs of the channel slices
// O = W' FF with the weights already packed (pack_w_forward_thread); d_opart: wmm_forward_opart_bytes bytes
int wmm_forward_packed(const cgnet_wmm_plan* plan, const float* d_FF, float* d_O, const float* d_Wp, int B,
                       void* d_opart, hipStream_t s);

// raw weight-gradient sums  sum_{b in chunk, m} gO conj(FF)  per chunk of samples: d_part[chunk][nW] complex
// (wmm_gradw_part_bytes bytes); *nchunks = chunks written.  The caller adds them and divides by the stds.
size_t wmm_gradw_part_bytes(const cgnet_wmm_plan* plan, int B);
int wmm_gradw_raw(const cgnet_wmm_plan* plan, const float* d_gO, const float* d_FF, float* d_part, int B, int* nchunks,
                  hipStream_t s);

// ---- cg_product.hip
int samples_per_group_for(int B, int ntasks);
// the product kernels of one call; d_part != nullptr: also the per-group partial statistics [group][sumT][2]
// d_tasks: another table of the plan's forward tasks, in the same order, whose tiles lie elsewhere in the product
// tensor (nFF complex entries and sumT channels per sample); nullptr = the plan's own
int cg_launch_forward(const cgnet_cg_plan* p, const float* d_F, float* d_FF, const float* d_CG, int B, double* d_part,
                      int spg, hipStream_t s, const CgTask* d_tasks = nullptr, int nFF = 0, int sumT = 0);
// Per-task metadata of the fused layer backward for this pair of plans, on the current device.  link->ok says
// whether the fused kernel takes the pair; when it does not, the return code is CGNET_ERR_UNSUPPORTED and
// cgnet_last_error() names the reason.
int build_fused_link(const cgnet_cg_plan* p, const cgnet_wmm_plan* w, FusedLink* link);
void free_fused_link(FusedLink* link);
// bytes of the unit backward's own areas (partials, padded fragments, padded tables) = cgnet_sparse_backward_workspace
struct BwdAreas { size_t part1, part2, Fp, CGP, total; };
BwdAreas bwd_areas(const cgnet_cg_plan* p, int B);
// padded fragments and tables (the operands the unit kernels copy into LDS)
int launch_backward_pad(const cgnet_cg_plan* p, const float* d_F, const float* d_CG, float* d_Fp, float* d_CGP, int B,
                        hipStream_t s);
// packed A operand (conj-free weights / div, per task) of the fused backward
int launch_pack_w_gen(const FusedLink& link, const float* d_W, const float* d_stds, float eps, float* d_Ag, hipStream_t s);
// gO packing + fused kernel + combine; the A operand, padded fragments and tables are given
int launch_fused_backward(const cgnet_cg_plan* p, const FusedLink& link, const float* d_gO, const float* d_Ag,
                          const float* d_Fp, const float* d_CGP, float* d_Bg, float* d_part1, float* d_part2,
                          float* d_gF, int B, hipStream_t s);

// ---- fused inference forward (cg_product.hip)
int build_fwd_link(const cgnet_cg_plan* p, const cgnet_wmm_plan* w, FwdLink* link);
void free_fwd_link(FwdLink* link);
int launch_pack_w_mix(const cgnet_cg_plan* p, const FwdLink& link, const float* d_W, const float* d_stds, float eps, float* d_Af,
                      hipStream_t s);
// product tiles mixed in LDS + the sum of the tasks' partial outputs; d_Opart: link.opart * B complex entries
int launch_forward_fused(const cgnet_cg_plan* p, const FwdLink& link, const float* d_F, const float* d_CG, const float* d_Af,
                         float* d_Opart, float* d_O, int B, hipStream_t s);

}  // namespace cgnet
