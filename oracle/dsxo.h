/*
 * dsxo — CPU ORACLE for the 3D-Gaussian-Splatting rasterizer hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It is a serial restatement of the
 * arithmetic of the reference kernels (deepsense-ai/ds-splat, cpp/rasterizer_kernels.cu,
 * cpp/rasterizer_torch.cu, cpp/gsplat/backward.cu, cpp/gsplat/helpers.cuh,
 * cpp/gsplat/sh.cuh).  Only tests, the smoke check and the benchmark's CPU-baseline leg
 * may link or load it; the GPU library never does.
 *
 * Every function cites the reference lines it follows.  All matrices are row-major,
 * "math convention" (translation in elements 3, 7, 11), i.e. what the reference's native
 * code sees after ds_splat/rasterizer.py:147-148 has transposed the user's matrices.
 *
 * Pinning status (what fixes each function's results independently of this file):
 *   tile ranges          — the reference's own two known-answer tests
 *                          (tests/rasterizer_test.cpp:66-110) + brute force
 *   key packing          — tests/rasterizer_test.cpp:17-20 and the first golden key of :52
 *   cov3d, cov2d, conic, radius, frustum, pixel mean, tile rect, SH forward, offsets,
 *   sort, blend forward, blend backward, SH backward, projection backward
 *                        — no reference-held vector exists; pinned by closed forms,
 *                          invariants, brute force and float64 finite differences
 *                          (tests/test_oracle_*.py).
 *   Quirks that only the reference's source text fixes (last Gaussian never emitted,
 *   0.999/0.99 alpha clamps, un-normalised quaternion in backward, unclamped t in the
 *   EWA backward, atan/tan focal in backward): PARITY UNPINNED beyond the source text.
 */
#ifndef DSXO_H_
#define DSXO_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dsxo_settings
{
    int32_t image_height;
    int32_t image_width;
    float tanfovx;
    float tanfovy;
    float bg[3];
    float scale_modifier;
    float view[16]; /* row-major world->view            */
    float proj[16]; /* row-major world->clip (full P*V) */
    int32_t sh_degree;
    int32_t max_sh_degree;
    float campos[3];
} dsxo_settings;

/* counters filled by the blend stages (pair = one evaluated (pixel, Gaussian) pair) */
typedef struct dsxo_counters
{
    int64_t pairs_fwd;         /* pairs walked by in-image pixels until they stopped */
    int64_t pairs_fwd_applied; /* pairs that passed the alpha test and were blended   */
    int64_t pairs_bwd;         /* pairs walked back-to-front by in-image pixels       */
    int64_t pairs_bwd_valid;   /* pairs that passed the backward alpha test           */
} dsxo_counters;

int dsxo_num_threads(void);

/* Stage 1: rasterizer_kernels.cu:57-161 (per Gaussian, everything except the in-block scan).
 * Outputs (all may not be NULL): means2d[N,3]=(px,py,view depth), conic[N,3], rgb[N,3],
 * radii[N], tiles_touched[N], cov3d[N,6].  shs has row stride (max_sh_degree+1)^2*3.
 * cov3d_precomp / colors_precomp may be NULL. */
void dsxo_project_fwd(const dsxo_settings* s, int64_t n, const float* means3d, const float* scales,
                      const float* quats, const float* shs, const float* cov3d_precomp,
                      const float* colors_precomp, float* means2d, float* conic, float* rgb,
                      int32_t* radii, int32_t* tiles_touched, float* cov3d);

/* rasterizer_kernels.cu:131-152 + rasterizer_torch.cu:95-104: exclusive prefix of
 * tiles_touched; returns K = offsets[n-1] (the last Gaussian's own count is excluded). */
int64_t dsxo_offsets(int64_t n, const int32_t* tiles_touched, int32_t* offsets);

/* Stage 2a: rasterizer_kernels.cu:252-306. */
void dsxo_emit_keys(const dsxo_settings* s, int64_t n, int64_t k, const float* means2d,
                    const int32_t* radii, const int32_t* offsets, int64_t* keys, int32_t* values);

/* Stage 2b: rasterizer_torch.cu:70-76 (thrust::sort_by_key == stable ascending sort on the
 * signed 64-bit key). In place. */
void dsxo_sort_pairs(int64_t k, int64_t* keys, int32_t* values);

/* Stage 3: rasterizer_torch.cu:23-42 + rasterizer_kernels.cu:308-323.
 * ranges has num_tiles+1 entries. */
void dsxo_tile_ranges(int64_t k, const int64_t* keys, int32_t num_tiles, int32_t* ranges);

/* Stage 4: rasterizer_kernels.cu:341-431.  image[H,W,3], final_T[H,W], final_idx[H,W].
 * margin[H,W] (may be NULL) receives, per pixel, the smallest relative distance of any
 * threshold decision taken for that pixel (alpha vs 1/255, power vs 0, T vs 1e-4) — pixels
 * whose margin is below the accuracy of exp() are ambiguous in the reference itself. */
void dsxo_blend_fwd(const dsxo_settings* s, const int32_t* ranges, const int32_t* sorted_ids,
                    const float* means2d, const float* conic, const float* rgb,
                    const float* opacities, float* image, float* final_T, int32_t* final_idx,
                    float* margin, dsxo_counters* counters);

/* Stage 5a: gsplat/backward.cu:25-202.  v_out[H,W,3]; v_out_alpha may be NULL (= zeros,
 * rasterizer_torch.cu:285).  Outputs v_xy[N,2], v_conic[N,3], v_rgb[N,3], v_opacity[N];
 * per-pixel terms are evaluated in float exactly as the reference does, the sums over
 * pixels are accumulated in double and rounded once.  g_margin[N] (may be NULL): smallest
 * relative distance to the backward alpha threshold over the pairs of each Gaussian. */
void dsxo_blend_bwd(const dsxo_settings* s, int64_t n, const int32_t* ranges,
                    const int32_t* sorted_ids, const float* means2d, const float* conic,
                    const float* rgb, const float* opacities, const float* final_T,
                    const int32_t* final_idx, const float* v_out, const float* v_out_alpha,
                    float* v_xy, float* v_conic, float* v_rgb, float* v_opacity, float* g_margin,
                    dsxo_counters* counters);

/* The same, plus abs_sums[N,9] (may be NULL): for every Gaussian and every one of the nine sums,
 * in the order x y | conic a b c | opacity | r g b, the sum over pixels of the ABSOLUTE values of
 * the elementary terms (every product that enters v_alpha taken by its magnitude).  A float
 * summation in another order, or with other roundings of the terms, may differ from the exact
 * sum by a small multiple of machine epsilon times this figure: it is the scale that a
 * tolerance on these gradients has to be relative to. */
void dsxo_blend_bwd_ex(const dsxo_settings* s, int64_t n, const int32_t* ranges,
                       const int32_t* sorted_ids, const float* means2d, const float* conic,
                       const float* rgb, const float* opacities, const float* final_T,
                       const int32_t* final_idx, const float* v_out, const float* v_out_alpha,
                       float* v_xy, float* v_conic, float* v_rgb, float* v_opacity, float* g_margin,
                       dsxo_counters* counters, float* abs_sums);

/* Stage 5b: gsplat/sh.cuh:95-203 with viewdirs = means - campos (rasterizer_torch.cu:291).
 * v_shs[N, num_bases, 3] where num_bases follows rasterizer_torch.cu:224-239 / sh.cuh:18-29;
 * entries above the active degree are zero (gsplat/bindings.cu:38-39). */
void dsxo_sh_bwd(const dsxo_settings* s, int64_t n, int32_t num_bases, const float* means3d,
                 const float* v_rgb, float* v_shs);

/* Stage 5c: gsplat/backward.cu:216-393 + helpers.cuh:68-220, focal per
 * rasterizer_torch.cu:78-81,297-298.  Outputs are zero for radii<=0. */
void dsxo_project_bwd(const dsxo_settings* s, int64_t n, const float* means3d, const float* scales,
                      const float* quats, const float* conic, const float* cov3d,
                      const int32_t* radii, const float* v_xy, const float* v_conic,
                      float* v_mean3d, float* v_scale, float* v_quat, float* v_cov3d,
                      float* v_cov2d);

/* Whole forward / backward, used by the parity tests at small sizes and (OpenMP build) as
 * the timed CPU baseline.  The state object keeps everything backward needs. */
typedef struct dsxo_state dsxo_state;

dsxo_state* dsxo_forward(const dsxo_settings* s, int64_t n, const float* means3d,
                         const float* scales, const float* quats, const float* opacities,
                         const float* shs, const float* cov3d_precomp, const float* colors_precomp,
                         float* image, int32_t* radii);
int64_t dsxo_state_num_keys(const dsxo_state* st);
/* copies of the intermediate products, any pointer may be NULL */
void dsxo_state_get(const dsxo_state* st, float* means2d, float* conic, float* rgb,
                    int32_t* tiles_touched, int32_t* offsets, float* cov3d, int64_t* sorted_keys,
                    int32_t* sorted_ids, int32_t* ranges, float* final_T, int32_t* final_idx,
                    float* margin, dsxo_counters* counters);
/* unsorted keys/values as emitted (before the sort); kept only after dsxo_keep_emitted(1) */
void dsxo_keep_emitted(int on);
void dsxo_state_get_emitted(const dsxo_state* st, int64_t* keys, int32_t* values);
void dsxo_backward(dsxo_state* st, const dsxo_settings* s, int64_t n, int32_t num_bases,
                   const float* means3d, const float* scales, const float* quats,
                   const float* opacities, const float* v_image, float* v_mean3d, float* v_means2d,
                   float* v_shs, float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                   float* v_cov3d, float* g_margin);
/* dsxo_backward with the abs_sums[N,9] of dsxo_blend_bwd_ex (may be NULL) */
void dsxo_backward_ex(dsxo_state* st, const dsxo_settings* s, int64_t n, int32_t num_bases,
                      const float* means3d, const float* scales, const float* quats,
                      const float* opacities, const float* v_image, float* v_mean3d, float* v_means2d,
                      float* v_shs, float* v_colors, float* v_opacity, float* v_scale, float* v_quat,
                      float* v_cov3d, float* g_margin, float* abs_sums);
void dsxo_state_free(dsxo_state* st);

/* ---- float64 instances used only for finite-difference pinning of the backward ---- */
/* blend forward in double on packed per-Gaussian parameters; clamp selects the alpha
 * clamp (0.999 forward, 0.99 backward view of the same function).
 * Returns sum((image + final_T * bg) * w); bg may be NULL (= no background term). */
double dsxo_blend_loss_f64(int32_t width, int32_t height, const int32_t* ranges,
                           const int32_t* sorted_ids, int64_t n, const double* xy,
                           const double* conic, const double* rgb, const double* opac,
                           const double* weights, const double* bg, double alpha_clamp);
#ifdef __cplusplus
}
#endif
#endif
