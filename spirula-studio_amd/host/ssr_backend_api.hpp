// ssr_backend_api.hpp -- the reference's launch functions for the projection / tile / raster path,
// re-declared with the reference's own names, argument order and meaning, implemented on the C ABI
// of libssr_hip.so. A maintainer of the reference adds this backend by compiling these
// definitions in place of the CUDA (src/kernels/**) or Vulkan (src/backend/vulkan/kernels/**) ones.
//
//   projection_3dgs_forward        src/kernels/projection/ProjectionFwd.cuh:18-36
//   projection_3dgs_packed_forward src/kernels/projection/ProjectionPackedFwd.cuh:18-37
//   do_intersect_tile_generic      src/kernels/tile/IntersectTile.cuh:25-41
//   rasterize_to_pixels_3dgs_fwd   src/kernels/raster/RasterizationFwd.cuh:18-38
//   rasterize_to_pixels_3dgs_bwd   src/kernels/raster/RasterizationBwd.cuh:18-48
//   projection_3dgs_backward       src/kernels/projection/ProjectionBwd.cuh:18-46
//
// Outputs are slots of the process-global grow-only DevicePool, returned as non-owning views that
// stay valid until the same function runs again; the caller never frees. Unsupported variants
// throw std::runtime_error, as the reference does (src/kernels/projection/ProjectionFwd.cu:84-89).
// Not thread-safe across concurrent calls (one in-order stream, shared scratch), like the
// reference's sort scratch (src/backend/vulkan/SortScanVulkan.cpp:4-6).
#pragma once
#include "ssr_host_types.hpp"
#include "ssr_sortscan.hpp"

std::tuple<DeviceTensor2D<float4>, DeviceTensor2D<float>, std::vector<DeviceTensorFloatND>>
projection_3dgs_forward(
    const int64_t num_splats, const int max_sh_degree,
    const std::vector<DeviceTensorFloatND>& in_splats,
    TorchTensorView viewmats, TorchTensorView intrins,
    const uint32_t image_width, const uint32_t image_height,
    const std::string camera_model, const std::string distortion,
    const TorchTensorView dist_coeffs,
    DeviceVector<float> radii,
    const std::optional<TorchTensorView> sh_value_packed,
    const std::optional<TorchTensorView> sh_value_bounds,
    const uint32_t num_sh_buffer,
    const int sh_value_bits,
    const int64_t sh_bounds_stride);

// Packed form: (camera_ids[nnz], gaussian_ids[nnz], aabb[nnz], sorting depths[nnz], screen[5] with
// nnz rows), visible splats only, in ascending splat order. Blocks on the readback of nnz, as the
// reference does (src/kernels/projection/ProjectionPackedFwd.cu:112-119).
std::tuple<DeviceVector<int32_t>, DeviceVector<int32_t>, DeviceVector<float4>, DeviceVector<float>,
           std::vector<DeviceTensorFloatND>>
projection_3dgs_packed_forward(
    const int64_t num_splats, const int max_sh_degree,
    const std::vector<DeviceTensorFloatND>& in_splats,
    TorchTensorView viewmats, TorchTensorView intrins,
    const uint32_t image_width, const uint32_t image_height,
    const std::string camera_model, const std::string distortion,
    const TorchTensorView dist_coeffs,
    DeviceVector<float> radii,
    const std::optional<TorchTensorView> sh_value_packed,
    const std::optional<TorchTensorView> sh_value_bounds,
    const uint32_t num_sh_buffer,
    const int sh_value_bits,
    const int64_t sh_bounds_stride);

int64_t intersect_tile_count(int width, int height);
// src/kernels/tile/IntersectTile.cu:349-368; mask is [I, H_mask, W_mask] bool on the device
void compute_tile_active(TorchTensorView mask, int I, int width, int height, int32_t* tile_active);

std::tuple<DeviceVector<int64_t>, DeviceVector<int32_t>, DeviceTensor3D<int32_t>>
do_intersect_tile_generic(
    DeviceTensorFloatND aabb, DeviceTensorFloatND depths,
    DeviceTensorFloatND* proj_xy, DeviceTensorFloatND* proj_conic, DeviceTensorFloatND* proj_opac,
    const uint32_t I, TorchTensorView intrins,
    const uint32_t image_width, const uint32_t image_height,
    DeviceVector<int32_t>* image_ids, const int32_t* tile_active);

std::tuple<RenderOutput::TensorTuple, DeviceTensor3D<float>, DeviceTensor3D<int32_t>,
           RenderOutput::TensorTuple, DeviceTensor3D<float>>
rasterize_to_pixels_3dgs_fwd(
    int64_t num_splats,
    std::vector<DeviceTensorFloatND> splats_w, std::vector<DeviceTensorFloatND> splats_s,
    DeviceVector<int32_t> gaussian_ids,
    const uint32_t image_width, const uint32_t image_height,
    const DeviceTensor3D<int32_t> tile_offsets, const DeviceVector<int32_t> flatten_ids,
    DistortionType dist_type, bool output_median);

std::tuple<std::vector<DeviceTensorFloatND>, std::vector<DeviceTensorFloatND>, DeviceVector<float>>
rasterize_to_pixels_3dgs_bwd(
    int64_t num_splats,
    std::vector<DeviceTensorFloatND> splats_w, std::vector<DeviceTensorFloatND> splats_s,
    DeviceVector<int32_t> gaussian_ids,
    const uint32_t image_width, const uint32_t image_height,
    const DeviceTensor3D<int32_t> tile_offsets, const DeviceVector<int32_t> flatten_ids,
    const DeviceTensor3D<float> render_Ts, const DeviceTensor3D<int32_t> last_ids,
    RenderOutput::TensorTuple render_outputs_tuple,
    std::optional<RenderOutput::TensorTuple> distortion_fwd_outputs,
    DistortionType dist_type,
    DeviceTensor3D<float> accum_weight_map, DensifyAccumMode accum_mode,
    RenderOutput::TensorTuple v_render_outputs,
    const DeviceTensor3D<float> v_render_Ts, const DeviceTensor3D<float> v_median,
    std::optional<RenderOutput::TensorTuple> v_distortion_outputs,
    std::optional<std::vector<DeviceTensorFloatND>> v_splats_w,
    std::optional<std::vector<DeviceTensorFloatND>> v_splats_s);

void projection_3dgs_backward(
    const int64_t num_splats, const int max_sh_degree,
    const std::vector<DeviceTensorFloatND>& splats_world,
    TorchTensorView viewmats, TorchTensorView intrins,
    const uint32_t image_width, const uint32_t image_height,
    const std::string camera_model, const std::string distortion,
    const TorchTensorView dist_coeffs,
    const DeviceVector<int32_t> camera_ids, const DeviceVector<int32_t> gaussian_ids,
    const DeviceTensor2D<float4> aabb,
    const std::vector<DeviceTensorFloatND>& v_splats_screen,
    const std::vector<DeviceTensorFloatND>& v_splats_world,
    DeviceTensor2D<float>* v_viewmats,
    const std::optional<TorchTensorView> sh_value_packed,
    const std::optional<TorchTensorView> sh_value_bounds,
    const uint32_t num_sh_buffer, const int sh_value_bits, const int64_t sh_bounds_stride);

// src/kernels/optim/FusedProjectionBwdOptim.cuh:18-62: every argument is honoured (plain and packed rows,
// all regularizers, scale-agnostic mean step, colour trust region, quantization levels 0 and 1 with the
// non-SH quantized moments); with [C,4,4] cameras the other cameras'
// world gradients are summed first and one Adam step is taken.
void fused_projection_bwd_optimizer_3dgs(
    const int64_t num_splats, const int max_sh_degree,
    std::vector<DeviceTensorFloatND> splats_world,
    TorchTensorView viewmats, TorchTensorView intrins,
    const uint32_t image_width, const uint32_t image_height,
    const std::string camera_model, const std::string distortion,
    const TorchTensorView dist_coeffs,
    const DeviceVector<int32_t> camera_ids, const DeviceVector<int32_t> gaussian_ids,
    DeviceTensorFloatND aabb,
    const std::vector<DeviceTensorFloatND> v_splats_world,
    const std::vector<DeviceTensorFloatND> v_splats_screen,
    const std::vector<DeviceTensorFloatND> g1_splats_world,
    const std::vector<DeviceTensorFloatND> g2_splats_world,
    const std::optional<TorchTensorView> sh_packed,
    const std::optional<TorchTensorView> sh_quant_bounds,
    const std::optional<TorchTensorView> sh_value_packed,
    const std::optional<TorchTensorView> sh_value_bounds,
    NonShQuantState non_sh,
    DeviceVector<float> radii, DeviceVector<float> densify_score,
    const float lr_means, const float lr_quats, const float lr_scales, const float lr_opacs,
    const float lr_features_dc, const float lr_features_sh,
    const float max_gauss_ratio, const float scale_regularization_weight,
    const float mcmc_opacity_reg_weight, const float mcmc_scale_reg_weight,
    const float erank_reg_weight, const float erank_reg_weight_s3,
    const float quat_norm_reg_weight, const float sh_reg_weight,
    bool use_scale_agnostic_mean, bool color_trust_linear, float eps_tr,
    std::variant<int32_t, TorchTensorView> step, int quantization_level);

// The antialiased ("mip") primitive: the reference's projection_mip_* / rasterize_to_pixels_mip_* /
// fused_projection_bwd_optimizer_mip (src/kernels/projection/ProjectionFwd.cuh, ProjectionPackedFwd.cuh, ProjectionBwd.cuh,
// src/kernels/raster/RasterizationFwd.cuh, RasterizationBwd.cuh, src/kernels/optim/FusedProjectionBwdOptim.cuh) are the 3dgs
// functions instantiated with antialiased = true (src/primitives/Primitive3DGS.cuh:20): same arguments, the projection's
// runtime flag set; compositing does not depend on it.
namespace ssr_detail { struct AntialiasedScope { AntialiasedScope(); ~AntialiasedScope(); }; }
template <class... A> auto projection_mip_forward(A&&... a) { ssr_detail::AntialiasedScope s; return projection_3dgs_forward(std::forward<A>(a)...); }
template <class... A> auto projection_mip_packed_forward(A&&... a) { ssr_detail::AntialiasedScope s; return projection_3dgs_packed_forward(std::forward<A>(a)...); }
template <class... A> void projection_mip_backward(A&&... a) { ssr_detail::AntialiasedScope s; projection_3dgs_backward(std::forward<A>(a)...); }
template <class... A> void fused_projection_bwd_optimizer_mip(A&&... a) { ssr_detail::AntialiasedScope s; fused_projection_bwd_optimizer_3dgs(std::forward<A>(a)...); }
template <class... A> auto rasterize_to_pixels_mip_fwd(A&&... a) { return rasterize_to_pixels_3dgs_fwd(std::forward<A>(a)...); }
template <class... A> auto rasterize_to_pixels_mip_bwd(A&&... a) { return rasterize_to_pixels_3dgs_bwd(std::forward<A>(a)...); }

// ---- extensions of this backend (no counterpart in the reference) ----
namespace ssr_ext {
// Work the reference does that this backend can skip with identical results:
struct Options {
    // K1 also produces the per-splat tile count, so do_intersect_tile_generic skips its count
    // pass when the projection that produced `aabb` ran with this set.
    bool fuse_tile_count = false;
    // K1 also emits the list of visible splats; the key write (K4) and the projection backward (K9)
    // then run over that list instead of all N splats.
    bool visible_list = false;
    // K1 also writes each visible screen row as one 48-byte record; the compositing kernels gather
    // from it when they are handed the screen buffers of that same projection.
    bool packed_rows = false;
    // K9 stores gradients instead of adding them into zero-filled rows (with several cameras the first
    // camera's launch stores and the others add). Without the visible list every row is overwritten (zeros for
    // culled splats) and the caller may skip its zero-fill; with the list only visible rows are
    // stored and the zero-fill is still needed.
    bool overwrite_world_grads = false;
    // The compositing backward writes each splat's ten gradient channels as one 12-float row (its
    // atomics then touch one or two cache lines instead of five) and the projection backward / fused
    // optimizer read those rows when handed the v_splats_screen of that call; the five returned
    // tensors are then allocated but NOT filled.
    bool packed_vscreen = false;
    // The key sort partitions by tile (the tile bits only) and then sorts each tile's range on the
    // depth bits with one workgroup per tile, instead of six whole-array digit passes; same result.
    bool tile_sort = false;
    // With tile_sort: do_intersect_tile_generic does not wait for the intersection count (the reference blocks on
    // it, IntersectTile.cu:432-436). The key arrays are sized from the previous call's count (plus 1/16 and 65536
    // entries; or set_deferred_capacity), the count stays on the device and reaches the host asynchronously; the
    // returned id vectors then have the capacity as their size; only their first last_n_isects() entries are keys.
    // resolve_counts() waits for the numbers: it is called by everything here that needs them (last_n_isects,
    // last_n_visible, backward_overwrites_all_rows, projection_3dgs_backward, the fused optimizer) and throws if
    // the count did not fit; the images and gradients of that iteration are then incomplete and the next
    // intersection reads its count again. The first call, and any call with capacity 0, blocks as before.
    // A caller that only renders asks for none of these: a short frame is then counted in short_frames(), left in
    // backend::last_error(), and refused by engine_copy_render_to_host.
    bool deferred_counts = false;
    // projection_3dgs_packed_forward also keeps the parameters of every visible splat, 64 bytes in four planes, in the
    // order of the packed rows, and a projection_3dgs_backward that is handed the gaussian_ids and the parameter
    // tensors of that call reads those planes instead of gathering from five arrays (it pays where a view sees a
    // small, scattered part of the splats). For callers that do not change the parameters between a packed
    // projection and its backward: tensors are recognised by their addresses, not by their contents.
    bool packed_world_rows = false;
    // Which cut of the compositing backward runs where both can (no distortion, no median; weight sums only with
    // packed_vscreen): -1 lets the adapter choose from the tiles per visible splat it last saw, 0 a row of lanes per
    // fragment (SSR_BWD_SCHEDULE_ROWS), 1 a lane per fragment (SSR_BWD_SCHEDULE_LANES).
    int backward_schedule = -1;
    // int8 codes x per-splat fp16 scale as SH storage (the benchmark's format): sh_value_bits == 8
    // with sh_value_bounds holding the fp16 scales when this is set.
    bool sh_int8_f16scale = false;
};
Options& options();
// Per-stage device time of the most recent calls (ms), measured with events on the launch stream
// when profiling is on.
struct StageTimes { float k1 = 0, k2 = 0, k3 = 0, k4 = 0, k5 = 0, k6 = 0, k7 = 0, k8 = 0, k9 = 0; };
void set_stage_profiling(bool on);
StageTimes last_stage_times();
int64_t last_n_isects();
int64_t last_n_visible();   // -1 when the visible list is off
void resolve_counts();      // see Options::deferred_counts
// How many intersections so far turned out larger than the arrays they were left to (deferred counts). Each is also
// reported by the resolve_counts() that finds it (an exception) and left in backend::last_error(); the stages that
// settle an abandoned iteration's counts swallow the exception, so a caller that only renders learns of a short
// frame here, or from engine_copy_render_to_host, which settles the counts before it hands out the image.
int64_t short_frames();
void set_deferred_capacity(int64_t capacity);
int64_t deferred_capacity();
// The list the last projection_3dgs_backward ran over (device pointer) and its length; it stays
// intact until the projection after next (the two list buffers alternate). Null when it had none.
const int32_t* last_backward_list(int64_t* count);
// Drops the parameter rows kept under Options::packed_world_rows: for a caller that writes new parameter values
// into the same tensors between a packed projection and its backward.
void forget_packed_world_rows();
// Whether projection_3dgs_forward with this many cameras stores every row of `radii` (one camera: its launch is the
// only writer, so it stores what the caller's zero-fill and the atomic maximum would leave) -- a caller that
// owns the buffer may then skip the fill.
bool projection_stores_radii(int64_t cameras);
// True when the next projection_3dgs_backward (after the forward that just ran) will overwrite EVERY
// row of v_splats_world -- store mode, and either no work list or so many visible splats (half or
// more) that walking all rows is cheaper than a zero-fill plus the list. The caller may then skip
// its zero-fill.
bool backward_overwrites_all_rows(int64_t num_splats);
// Zeroes the rows of `ids` in six world-gradient tensors (ordered as v_splats_world).
// Rows of currently visible splats are skipped (a store-mode backward overwrites them): those with a non-empty
// `aabb` row, or those named in the ascending id list `sorted_now` (one camera's packed gaussian_ids).
void zero_world_rows(const std::vector<DeviceTensorFloatND>& v_splats_world, const int32_t* ids, int64_t n,
                     const DeviceTensor2D<float4>* aabb, const int32_t* sorted_now = nullptr, int64_t n_now = 0);
}  // namespace ssr_ext
