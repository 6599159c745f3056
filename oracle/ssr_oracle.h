/* ssr_oracle.h -- C interface of the CPU oracle.
 *
 * TEST INFRASTRUCTURE ONLY. This library restates, on the CPU, the algorithm of the reference's
 * Gaussian-splat hot path (projection + SH colour, tile keys, sort, tile ranges, compositing
 * forward, compositing backward, projection backward). It exists to check the HIP kernels; the
 * product library never links, loads or calls it. Only tests, the smoke check and the
 * cpu_baseline leg of the benchmark may use it.
 *
 * Every function is checked against closed forms, float64 restatements or finite differences by
 * tests/test_oracle_*.py; nothing is left unpinned. The median-depth gradient of or_raster_bwd_ex omits the
 * far splat's own opacity term, as the reference states it does
 * (src/kernels/raster/RasterizationEval3DBwd_kernel.cuh:433-440): it is the gradient of the median with
 * ln(1 - alpha_far) held fixed, and is checked against finite differences of that function
 * (tests/test_oracle_raster_variants.py). or_raster_lane_stats is a measurement aid, not a restatement.
 *
 * Every pointer is a host pointer. Arrays use the reference's layouts
 * (src/primitives/PrimitiveBase3DGS.cuh:87-139,187-225):
 *   world:  means[N,3] quats[N,4](w,x,y,z) log_scales[N,3] opacity_logits[N] features_dc[N,3]
 *           features_sh[N,15,3]
 *   screen: xy[N,2] depth[N] conic[N,3] opac[N] rgb[N,3]
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { OR_CAM_PINHOLE = 0, OR_CAM_FISHEYE = 1, OR_CAM_EQUISOLID = 2, OR_CAM_EQUIRECT = 3 };   /* src/core/Common.cuh CameraModelType */
enum { OR_LENS_NONE = 0, OR_LENS_OPENCV = 1, OR_LENS_THIN_PRISM = 2, OR_LENS_RATIONAL = 3 };   /* CameraDistortionType, src/shaders/projection_utils.slang:220-225 */
enum { OR_SH_F32 = 0, OR_SH_REF_Q8 = 1, OR_SH_REF_Q16 = 2, OR_SH_I8_F16SCALE = 3 };

typedef struct {
    int32_t model;          /* OR_CAM_* */
    uint32_t width, height;
    float viewmat[16];      /* row-major world->camera [R t; 0 1] */
    float fx, fy, cx, cy;
    int32_t distortion;     /* OR_LENS_* */
    float dist_coeffs[8];   /* in the tier's own order, src/shaders/projection_utils.slang:242-295 */
    int32_t antialiased;    /* the "mip" variant of the primitive (the projection function's runtime `antialiased`
                               argument, src/shaders/primitive_3dgs.slang:528-543); carried here for convenience */
} or_camera;

typedef struct {
    int32_t codec;          /* OR_SH_* */
    const float* sh_f32;    /* [N,15,3] when codec == OR_SH_F32 */
    const uint8_t* packed;  /* ref q8: uint8[N*3*num_sh_buffer]; ref q16: uint16; i8: int8[N*45] */
    const float* bounds;    /* ref codecs: float2[n_bounds] (min,max) */
    int64_t bounds_stride;  /* cells per bound; 0 selects 256*3*num_sh_buffer */
    uint32_t num_sh_buffer; /* coefficients per splat in the packed buffer (15 for SH3) */
    const uint16_t* scale_f16; /* i8 codec: fp16 bits, one per splat */
} or_sh_source;

/* K1. Outputs: aabb[N,4], sort_depth[N], radii[N] (max-accumulated), screen rows. Rows of culled
 * splats are left untouched, as the reference leaves them. Returns the number of visible splats. */
int64_t or_projection_fwd(int64_t N, int sh_degree,
    const float* means, const float* quats, const float* log_scales, const float* opacity_logits,
    const float* features_dc, const or_sh_source* sh, const or_camera* cam,
    float* aabb, float* sort_depth, float* radii,
    float* xy, float* depth, float* conic, float* opac, float* rgb);

/* K2 */
void or_tile_count(int64_t N, const float* aabb, const float* xy, const float* conic,
    const float* opac, uint32_t width, uint32_t height, int64_t* tiles_per_splat);
/* K2/K4 with the tile-skip map (tile_active[tile_h*tile_w], 0 = skip; NULL = all live), and the
 * map itself from a [h_mask,w_mask] byte mask (src/kernels/tile/IntersectTile.cu:316-368). */
void or_tile_count_masked(int64_t N, const float* aabb, const float* xy, const float* conic,
    const float* opac, uint32_t width, uint32_t height, const int32_t* tile_active, int64_t* tiles_per_splat);
int64_t or_tile_write_masked(int64_t N, const float* aabb, const float* sort_depth, const float* xy,
    const float* conic, const float* opac, const int64_t* cum_tiles, uint32_t width,
    uint32_t height, const int32_t* tile_active, int64_t* isect_ids, int32_t* flatten_ids);
void or_compute_tile_active(const uint8_t* mask, int32_t h_mask, int32_t w_mask, uint32_t width, uint32_t height,
    int32_t* tile_active);
/* K3 */
void or_inclusive_sum_i64(int64_t n, const int64_t* in, int64_t* out);
/* K4. Returns the number of 0xffffffff pad keys written (0 when count and write agree). */
int64_t or_tile_write(int64_t N, const float* aabb, const float* sort_depth, const float* xy,
    const float* conic, const float* opac, const int64_t* cum_tiles, uint32_t width,
    uint32_t height, int64_t* isect_ids, int32_t* flatten_ids);
/* K5: stable sort on bits [begin_bit, end_bit) of the key. */
void or_sort_pairs(int64_t n, const int64_t* keys_in, const int32_t* vals_in, int begin_bit,
    int end_bit, int64_t* keys_out, int32_t* vals_out);
/* K6 */
void or_tile_offsets(int64_t n_isects, const int64_t* sorted_ids, uint32_t n_tiles,
    int32_t* offsets);

/* K7. stats (optional, 5 entries): K_f and K_b as defined for the bandwidth model, then the
 * number of (splat, 8x8 sub-tile) visits of the forward, of the backward, and of the backward
 * visits in which some pixel composited the splat. */
void or_raster_fwd(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    float* out_rgb, float* out_depth, float* out_T, int32_t* out_last_ids, int64_t* stats);

/* K8. v_* outputs are ACCUMULATED into (caller zero-fills). abs_* (optional, may be NULL) receive
 * the sum of absolute values of the same terms in double, as an error scale for comparisons. */
/* measurement aid: lane statistics of the compositing backward for pixel blocks of 8, 4 and 2 */
void or_raster_lane_stats(const float* xy, const float* depth, const float* conic, const float* opac, const float* rgb,
    uint32_t width, uint32_t height, const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    const int32_t* last_ids, int64_t* out);
void or_raster_bwd(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    const float* render_T, const int32_t* last_ids, const float* render_depth,
    const float* v_rgb, const float* v_depth, const float* v_T,
    float* v_xy, float* v_sdepth, float* v_conic, float* v_opac, float* v_srgb,
    double* abs_terms /* [N,10] or NULL: per output element the sum of term magnitudes (1 + 0.06 n), n = transmittance
                         undo steps behind the term, a term that is linear in v_alpha taken at |T0 (c.v_c)| + |v_T1 T0|
                         in place of their difference; 2e-6 of it bounds what summation order and rounding move */);

/* K7 / K8 with their variants. dist_type: 0 none, 1 depth (D), 2 rgb + depth (RGB_D).
 * Forward: out_dist_rgb [H,W,3] (RGB_D), out_dist_depth [H,W] (D, RGB_D), out_median [H,W] or NULL.
 * Backward: render_rgb / dist_*_img are the forward's outputs, v_dist_* and v_median (NULL = no
 * median) the cotangents; accum_mode 0 none, 1 max, 2 sum, 3 avg (numerators then denominators,
 * n_world rows each; gaussian_ids, or NULL, maps a screen row to its world row);
 * accum_weight is max-/add-accumulated into (caller zero-fills). */
void or_raster_fwd_ex(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    float* out_rgb, float* out_depth, float* out_T, int32_t* out_last_ids, int64_t* stats,
    int dist_type, float* out_dist_rgb, float* out_dist_depth, float* out_median);
void or_raster_bwd_ex(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    const float* render_T, const int32_t* last_ids, const float* render_depth,
    const float* v_rgb, const float* v_depth, const float* v_T,
    float* v_xy, float* v_sdepth, float* v_conic, float* v_opac, float* v_srgb, double* abs_terms,
    int dist_type, const float* render_rgb, const float* dist_rgb_img, const float* dist_depth_img,
    const float* v_dist_rgb, const float* v_dist_depth, const float* v_median,
    int accum_mode, const float* accum_map, const int32_t* gaussian_ids, int64_t n_world, float* accum_weight);

/* K9. Gradients are ACCUMULATED into v_* (caller zero-fills). */
void or_projection_bwd(int64_t N, int sh_degree,
    const float* means, const float* quats, const float* log_scales, const float* opacity_logits,
    const float* features_dc, const or_sh_source* sh, const or_camera* cam, const float* aabb,
    const float* v_xy, const float* v_sdepth, const float* v_conic, const float* v_opac,
    const float* v_srgb,
    float* v_means, float* v_quats, float* v_scales, float* v_opacities, float* v_dc, float* v_sh);
/* As or_projection_bwd, and the camera-pose gradient (the reference's v_viewmats,
 * src/kernels/projection/ProjectionBwd_kernel.cuh:89-127): the sums over the processed splats of dL/dR and dL/dt
 * are added to v_viewmat (16 floats, row-major [R|t]; may be NULL). */
void or_projection_bwd_pose(int64_t N, int sh_degree,
    const float* means, const float* quats, const float* log_scales, const float* opacity_logits,
    const float* features_dc, const or_sh_source* sh, const or_camera* cam, const float* aabb,
    const float* v_xy, const float* v_sdepth, const float* v_conic, const float* v_opac,
    const float* v_srgb,
    float* v_means, float* v_quats, float* v_scales, float* v_opacities, float* v_dc, float* v_sh, float* v_viewmat);

/* K9 fused with Adam (fp32-state branch of fused_projection_bwd_optimizer_3dgs,
 * src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:232-710): parameters and moments [N,...]
 * are updated in place. v_in (6 arrays, any may be NULL) are gradient contributions already
 * present. hyper = {lr_means, lr_quats, lr_scales, lr_opacs, lr_dc, lr_sh, max_gauss_ratio,
 * scale_reg_w, mcmc_opacity_w, mcmc_scale_w, quat_norm_w, sh_reg_w, erank_w, erank_w_s3, color_trust_linear (0 / 1),
 * eps_tr} (16 floats). steps may be NULL
 * (then `step`). */
void or_fused_projection_bwd_optimizer(int64_t N, int sh_degree,
    float* means, float* quats, float* log_scales, float* opacity_logits, float* features_dc, float* features_sh,
    const or_camera* cam, const float* aabb,
    const float* v_xy, const float* v_sdepth, const float* v_conic, const float* v_opac, const float* v_srgb,
    const float* const* v_in, float* const* g1, float* const* g2, float* densify_score,
    const float* hyper, int32_t step, const int32_t* steps,
    const float* radii /* optional [N]: the forward's radii; given = the scale-agnostic step of the means */);

/* The quantized SH state of the fused optimizer at the reference's quantization level 1
 * (src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:709-1030 with QUANT_BITS = 8, VALUE_BITS = 16):
 * per block of 256 splats, Adam moments as QuantizedAdamState<8,256> cells (2 bytes: u, log_s; bounds
 * float4) and SH values as QuantizedTensor<16,256> cells (bounds float2); num_sh_buffer coefficients per
 * splat in both buffers. Pass to or_fused_projection_bwd_optimizer_q. */
typedef struct {
    uint16_t* state_packed;     /* [N * 3 * num_sh_buffer] u_q | s_q << 8 */
    float* state_bounds;        /* float4[ceil(N / 256)] */
    uint16_t* value_packed;     /* [N * 3 * num_sh_buffer] */
    float* value_bounds;        /* float2[ceil(N / 256)] */
    uint32_t num_sh_buffer;
} or_sh_quant_state;
/* The quantized Adam state of the five non-SH tensors (NonShQuantState,
 * src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:97-143,373-638): QuantizedAdamState<16,256> cells
 * (u code | log_s code << 16), one float4 of bounds per 256 splats and tensor; order means, quats,
 * log_scales, opacity_logits, features_dc. */
typedef struct {
    uint32_t* packed[5];        /* [N * 3], [N * 4], [N * 3], [N], [N * 3] */
    float* bounds[5];           /* float4[ceil(N / 256)] each */
} or_non_sh_quant_state;
/* As or_fused_projection_bwd_optimizer, with the SH coefficients and their moments held in q and, when nq is
 * given, the moments of the non-SH tensors in nq (g1 / g2 entries 0..4 are then not used). */
void or_fused_projection_bwd_optimizer_q(int64_t N, int sh_degree,
    float* means, float* quats, float* log_scales, float* opacity_logits, float* features_dc, const or_sh_quant_state* q,
    const or_non_sh_quant_state* nq,
    const or_camera* cam, const float* aabb,
    const float* v_xy, const float* v_sdepth, const float* v_conic, const float* v_opac, const float* v_srgb,
    const float* const* v_in, float* const* g1, float* const* g2, float* densify_score,
    const float* hyper, int32_t step, const int32_t* steps, const float* radii);
/* The codecs on arrays: op 0 Adam-state encode (a = g1, b = g2, mm float4 -> codes), 1 Adam-state decode
 * (codes -> a = g1, b = g2), 2 value encode (a = v, mm float2 -> codes), 3 value decode (codes -> a), 4 / 5 the
 * 16-bit Adam-state encode / decode. */
void or_quant_codec(int op, int64_t n, float* a, float* b, const float* mm, uint32_t* codes);

/* The colour maps of the colour trust region on arrays: op 0 slope of the sRGB curve, 1 splat_dc_encode,
 * 2 splat_dc_decode (src/shaders/pixel_wise.slang:60-115). */
void or_colour_map(int op, int64_t n, const float* x, float* y);

/* erank_reg_3dgs (src/shaders/per_splat_losses.slang:3-15): the loss for one splat's three log-scales and
 * its gradient. */
float or_erank_reg(const float* log_scales, float w, float w3, float* grad);

/* Codecs (src/core/Tensor.h:1364-1392): block-wise (min,max) + uint8/uint16 codes. */
void or_quantize_ref(int bits, int64_t n_cells, int64_t bounds_stride, const float* values,
    uint8_t* packed, float* bounds /* float2[ceil(n_cells/stride)] */);
/* int8 codes with one fp16 scale per splat: v = code * scale. */
void or_quantize_i8_f16(int64_t N, int cells_per_splat, const float* values, int8_t* codes,
    uint16_t* scale_f16);
void or_decode_sh(int64_t gid, const or_sh_source* sh, float* out45);

/* Transcendentals of include/ssr_math.h evaluated elementwise (op: 0 exp, 1 log, 2 atan2(a,b),
 * 3 sigmoid), for checking them against libm and against the device. */
void or_math(int op, int64_t n, const float* a, const float* b, float* out);

int or_num_threads(void);
void or_set_num_threads(int n);

#ifdef __cplusplus
}
#endif
