// ssr_engine.cpp -- engine harness (see ssr_engine.hpp) and its C entry points for Python.
#include "ssr_engine.hpp"

#include <cstring>

#include "../../include/ssr_backend.h"

static EngineState g_engine;
EngineState& engine() { return g_engine; }
void engine_reset() { g_engine = EngineState{}; }

namespace {

// host memory is copied into the slot, a device address is aliased (EngineCommon.h:90-105)
template <typename T>
DeviceVector<T> hv_to_dv(PoolSlot slot, const TorchTensorView& tv) {
    DeviceVector<T> view(tv);   // validates element size
    void* src = (void*)std::get<0>(tv);
    if (view.size() == 0 || backend::is_device_pointer(src)) return view;
    DeviceVector<T> out; out.resize(slot, view.size());
    backend::memcpy_sync(out.data_ptr(), src, (size_t)view.size() * sizeof(T), backend::MemcpyKind::HostToDevice);
    return out;
}

TorchTensorView device_copy_tv(PoolSlot slot, const TorchTensorView& tv) {
    void* src = (void*)std::get<0>(tv);
    int64_t n = 1;
    for (auto s : std::get<2>(tv)) n *= s;
    const size_t bytes = (size_t)n * std::get<1>(tv);
    if (bytes == 0 || backend::is_device_pointer(src)) return tv;
    uint8_t* p = DevicePool::global().acquire<uint8_t>(slot, bytes);
    backend::memcpy_sync(p, src, bytes, backend::MemcpyKind::HostToDevice);
    return TorchTensorView((uint64_t)p, std::get<1>(tv), std::get<2>(tv));
}

void alloc_grad_buffers() {
    // _alloc_grad_buffers: six fp32 world-gradient buffers, zeroed (src/engine/EngineLoss.cpp:20-127)
    auto& g = engine().grad;
    const int64_t n = engine().max_num_splats;
    g.means.resize(PoolSlot::GradMeans, n); g.quats.resize(PoolSlot::GradQuats, n);
    g.scales.resize(PoolSlot::GradScales, n); g.opacities.resize(PoolSlot::GradOpacities, n);
    g.features_dc.resize(PoolSlot::GradFeaturesDc, n); g.features_sh.resize(PoolSlot::GradFeaturesSh, n, engine().num_sh);
    const auto& o = ssr_ext::options();
    if (engine().optim.skip_grad_zero) return;
    const bool listed = o.visible_list || engine().packed;   // the backward touches listed rows only
    // K9 overwrites every row itself (rows past cur_num_splats, if any, are not its business: fill then)
    if (engine().cur_num_splats == n && ssr_ext::backward_overwrites_all_rows(n)) return;
    // Every row is zero except those the last backward wrote through its list (the visible-splat
    // list, or gaussian_ids in packed mode): when that list is short, zero just those rows instead
    // of refilling all N (the refill is 236 B per splat).
    if (listed && o.overwrite_world_grads && g.dirty_valid && g.dirty_key == (const void*)g.means.data_ptr() &&
        g.dirty_count * 2 < n) {
        std::vector<DeviceTensorFloatND> v_world = {
            DeviceTensorFloatND(g.means), DeviceTensorFloatND(g.quats), DeviceTensorFloatND(g.scales),
            DeviceTensorFloatND((float*)g.opacities.data_ptr(), {g.opacities.size(), 1}),
            DeviceTensorFloatND(g.features_dc), DeviceTensorFloatND(g.features_sh)};
        if (g.dirty_count > 0)
            // one camera's packed ids ascend, which is what the skip list needs
            ssr_ext::zero_world_rows(v_world, g.dirty_list, g.dirty_count, engine().packed ? nullptr : &engine().fwd.aabb,
                                     engine().packed && engine().camera.num == 1 ? engine().fwd.gaussian_ids.data_ptr() : nullptr,
                                     engine().fwd.gaussian_ids.size());
        return;
    }
    g.means.zero(); g.quats.zero(); g.scales.zero(); g.opacities.zero(); g.features_dc.zero(); g.features_sh.zero();
}

}  // namespace

void set_data_3dgs(int64_t num_splats, TorchTensorView means, TorchTensorView quats, TorchTensorView scales,
                   TorchTensorView opacities, TorchTensorView features_dc, TorchTensorView features_sh) {
    // Contract of src/engine/EngineSetup.cpp:11-47: the six tensors share their leading extent (the capacity),
    // num_splats of those rows are live, and only the first call uploads -- later calls just move the counts.
    struct Named { const char* name; const TorchTensorView* tv; };
    const Named all[6] = {{"means", &means}, {"quats", &quats}, {"scales", &scales},
                          {"opacities", &opacities}, {"features_dc", &features_dc}, {"features_sh", &features_sh}};
    auto rows_of = [](const TorchTensorView& tv) { return std::get<2>(tv).empty() ? int64_t(0) : std::get<2>(tv)[0]; };
    const int64_t capacity = rows_of(means);
    for (const Named& t : all)
        if (rows_of(*t.tv) != capacity)
            throw std::runtime_error(std::string("set_data_3dgs: '") + t.name + "' has " + std::to_string(rows_of(*t.tv)) +
                                     " rows where 'means' has " + std::to_string(capacity));
    if (num_splats > capacity)
        throw std::runtime_error("set_data_3dgs: num_splats " + std::to_string(num_splats) + " exceeds the " +
                                 std::to_string(capacity) + " rows given");
    ssr_ext::forget_packed_world_rows();   // new parameter values
    auto& E = engine();
    const auto& sh_dims = std::get<2>(features_sh);
    E.num_sh = sh_dims.size() > 1 ? (int)sh_dims[1] : 0;
    E.max_num_splats = capacity;
    E.cur_num_splats = num_splats;
    auto& w = E.world;
    if (w.initialized) return;
    w.means = hv_to_dv<float3>(PoolSlot::WorldMeans, means);
    w.quats = hv_to_dv<float4>(PoolSlot::WorldQuats, quats);
    w.scales = hv_to_dv<float3>(PoolSlot::WorldScales, scales);
    w.opacities = hv_to_dv<float>(PoolSlot::WorldOpacities, opacities);
    w.features_dc = hv_to_dv<float3>(PoolSlot::WorldFeaturesDc, features_dc);
    const TorchTensorView sh_dev = device_copy_tv(PoolSlot::WorldFeaturesSh, features_sh);
    w.features_sh = DeviceTensor2D<float3>((float3*)std::get<0>(sh_dev), capacity, E.num_sh);
    w.initialized = true;
}

void set_sh_value_quant(int sh_value_bits, TorchTensorView packed, TorchTensorView bounds, int64_t bounds_stride) {
    auto& w = engine().world;
    w.sh_value_bits = sh_value_bits;
    if (sh_value_bits == 32) { w.sh_packed.reset(); w.sh_bounds.reset(); return; }
    // codes and bounds given from the host are copied into pool slots; device addresses are aliased
    packed = device_copy_tv(PoolSlot::WorldShQuantPacked, packed);
    bounds = device_copy_tv(PoolSlot::WorldShQuantBounds, bounds);
    w.sh_packed = packed; w.sh_bounds = bounds; w.sh_bounds_stride = bounds_stride;
}

void set_camera_params(int width, int height, std::string camera_model, std::string distortion,
                       TorchTensorView viewmats, TorchTensorView intrins, TorchTensorView dist_coeffs) {
    auto& c = engine().camera;
    c.width = width; c.height = height;
    c.model_str = camera_model; c.distortion_str = distortion;
    c.num = (int)std::get<2>(viewmats)[0];
    if (std::get<2>(intrins)[0] != c.num || std::get<2>(dist_coeffs)[0] != c.num)
        throw std::runtime_error("setCameraParams: num_cameras mismatch");
    c.viewmats = device_copy_tv(PoolSlot::CamViewmats, viewmats);
    c.intrins = device_copy_tv(PoolSlot::CamIntrins, intrins);
    c.dist_coeffs = device_copy_tv(PoolSlot::CamDistCoeffs, dist_coeffs);
}

void engine_set_tile_mask(TorchTensorView mask) {
    auto& E = engine();
    if (E.camera.width <= 0) throw std::runtime_error("engine_set_tile_mask: set_camera_params must be called first");
    TorchTensorView dm = device_copy_tv(PoolSlot::EngTileMask, mask);
    E.fwd.tile_active.resize(PoolSlot::IsectTileActive, intersect_tile_count(E.camera.width, E.camera.height) * E.camera.num);
    compute_tile_active(dm, E.camera.num, E.camera.width, E.camera.height, E.fwd.tile_active.data_ptr());
}

void forward_3dgs(std::string primitive, int sh_degree, bool packed, bool output_median, int dist_type_int) {
    // "mip" is the antialiased 3dgs (src/engine/EngineForward.cpp:135,181,268 call the *_mip_* instantiations)
    if (primitive != "3dgs" && primitive != "mip")
        throw std::runtime_error("forward_3dgs: primitive '" + primitive + "' is not built in this backend");
    std::optional<ssr_detail::AntialiasedScope> antialiased;
    if (primitive == "mip") antialiased.emplace();
    auto& E = engine();
    if (!E.world.initialized) throw std::runtime_error("forward_3dgs: set_data_3dgs must be called first");
    E.primitive = primitive; E.sh_degree = sh_degree; E.packed = packed;
    const int64_t N = E.cur_num_splats;
    std::vector<DeviceTensorFloatND> in_splats = {
        DeviceTensorFloatND(E.world.means), DeviceTensorFloatND(E.world.quats), DeviceTensorFloatND(E.world.scales),
        DeviceTensorFloatND((float*)E.world.opacities.data_ptr(), {E.world.opacities.size(), 1}),
        DeviceTensorFloatND(E.world.features_dc), DeviceTensorFloatND(E.world.features_sh)};
    E.fwd.splats_w = in_splats;
    // radii: zeroed before projection, which accumulates with atomic max (EngineForward.cpp:66-69). A dense
    // projection of one camera stores all N rows itself; the fill is then needed only for rows it does not reach
    // (a new buffer, or fewer splats than the frame before).
    E.optim.radii.resize(PoolSlot::EngRadii, E.max_num_splats);
    {
        const float*& zeroed_ptr = E.optim.radii_zeroed_ptr;
        int64_t &zeroed_rows = E.optim.radii_zeroed_rows, &stored_rows = E.optim.radii_stored_rows;
        const bool stored = !packed && ssr_ext::projection_stores_radii(E.camera.num);
        static uint64_t generation = ~(uint64_t)0;   // of the pool the buffer comes from
        const bool same_pool = generation == DevicePool::global().generation();
        generation = DevicePool::global().generation();
        const bool covered = stored && same_pool && zeroed_ptr == E.optim.radii.data_ptr() && zeroed_rows == E.max_num_splats && N >= stored_rows;
        if (!covered && !E.optim.skip_grad_zero) {
            E.optim.radii.zero();
            zeroed_ptr = E.optim.radii.data_ptr(); zeroed_rows = E.max_num_splats;
        }
        stored_rows = stored ? N : E.max_num_splats;   // rows that may hold radii after this frame
    }

    DeviceTensorFloatND aabb_nd, depths_nd;
    std::vector<DeviceTensorFloatND> screen;
    if (packed) {   // src/engine/EngineForward.cpp:119-165
        auto [cam_ids, gauss_ids, aabb_vec, depths_vec, scr] = projection_3dgs_packed_forward(
            N, sh_degree, in_splats, E.camera.viewmats, E.camera.intrins, (uint32_t)E.camera.width,
            (uint32_t)E.camera.height, E.camera.model_str, E.camera.distortion_str, E.camera.dist_coeffs, E.optim.radii,
            E.world.sh_packed, E.world.sh_bounds, (uint32_t)E.num_sh, E.world.sh_value_bits, E.world.sh_bounds_stride);
        E.fwd.camera_ids = cam_ids; E.fwd.gaussian_ids = gauss_ids;
        E.fwd.aabb = DeviceTensor2D<float4>(aabb_vec.data_ptr(), aabb_vec.size(), 1);   // [nnz, 1] view for backward
        E.fwd.depths = DeviceTensor2D<float>(depths_vec.data_ptr(), 1, depths_vec.size());
        screen = scr;
        aabb_nd = DeviceTensorFloatND((float*)aabb_vec.data_ptr(), {aabb_vec.size(), 4});
        depths_nd = DeviceTensorFloatND(depths_vec.data_ptr(), {depths_vec.size()});
    } else {
        auto [aabb, depths, scr] = projection_3dgs_forward(
            N, sh_degree, in_splats, E.camera.viewmats, E.camera.intrins, (uint32_t)E.camera.width,
            (uint32_t)E.camera.height, E.camera.model_str, E.camera.distortion_str, E.camera.dist_coeffs, E.optim.radii,
            E.world.sh_packed, E.world.sh_bounds, (uint32_t)E.num_sh, E.world.sh_value_bits, E.world.sh_bounds_stride);
        E.fwd.camera_ids = DeviceVector<int32_t>(); E.fwd.gaussian_ids = DeviceVector<int32_t>();
        E.fwd.aabb = aabb; E.fwd.depths = depths;
        screen = scr;
        aabb_nd = DeviceTensorFloatND((float*)aabb.data_ptr(), {aabb.numel(), 4});
        depths_nd = DeviceTensorFloatND(depths.data_ptr(), {depths.numel()});
    }
    E.fwd.splats_s = screen;

    DeviceVector<int32_t>* image_ids_ptr = nullptr;   // EngineForward.cpp:215-217
    if (packed && E.fwd.camera_ids.data_ptr() != nullptr) image_ids_ptr = &E.fwd.camera_ids;
    auto [ids, flat, offsets] = do_intersect_tile_generic(
        aabb_nd, depths_nd, &screen[0], &screen[2], &screen[3], (uint32_t)E.camera.num, E.camera.intrins,
        (uint32_t)E.camera.width, (uint32_t)E.camera.height, image_ids_ptr, E.fwd.tile_active.data_ptr());
    E.fwd.isect_ids = ids; E.fwd.flatten_ids = flat; E.fwd.tile_offsets = offsets;
    E.fwd.tile_active = DeviceVector<int32_t>();   // one shot

    auto [renders, Ts, last, dist, median] = rasterize_to_pixels_3dgs_fwd(
        N, in_splats, screen, E.fwd.gaussian_ids, (uint32_t)E.camera.width, (uint32_t)E.camera.height, offsets, flat,
        (DistortionType)dist_type_int, output_median);
    E.fwd.renders = renders; E.fwd.render_Ts = Ts; E.fwd.last_ids = last;
    E.fwd.distortions = dist; E.fwd.dist_type = (DistortionType)dist_type_int; E.fwd.render_median = median;
}

namespace {
// stage the pixel cotangents and run the compositing backward; returns v_screen
struct VariantGrads {
    TorchTensorView v_dist_rgb{0, 4, {}}, v_dist_depth{0, 4, {}}, v_median{0, 4, {}}, accum_map{0, 4, {}};
    DensifyAccumMode accum_mode = DensifyAccumMode::None;
};

std::vector<DeviceTensorFloatND> raster_backward(TorchTensorView v_render_rgb, TorchTensorView v_render_depth,
                                                 TorchTensorView v_render_Ts, const VariantGrads& vg = VariantGrads{}) {
    auto& E = engine();
    const int64_t C = E.camera.num, H = E.camera.height, W = E.camera.width;
    auto stage = [&](PoolSlot slot, const TorchTensorView& src, int ch) -> float* {
        void* s = (void*)std::get<0>(src);
        if (backend::is_device_pointer(s)) return (float*)s;
        float* d = DevicePool::global().acquire<float>(slot, (size_t)(C * H * W * ch));
        backend::memcpy_sync(d, s, (size_t)(C * H * W * ch) * sizeof(float), backend::MemcpyKind::Auto);
        return d;
    };
    float* v_rgb = stage(PoolSlot::EngVRgb, v_render_rgb, 3);
    float* v_depth = stage(PoolSlot::EngVDepth, v_render_depth, 1);
    float* v_Ts = stage(PoolSlot::EngVTs, v_render_Ts, 1);
    RenderOutput::TensorTuple v_renders;
    std::get<0>(v_renders) = DeviceTensor3D<float3>((float3*)v_rgb, C, H, W);
    std::get<1>(v_renders) = DeviceTensor3D<float>(v_depth, C, H, W);
    DeviceTensor3D<float> v_Ts_t(v_Ts, C, H, W);
    // cotangents of the variants that the forward produced
    std::optional<RenderOutput::TensorTuple> dist_fwd, v_dist;
    if (E.fwd.dist_type != DistortionType::None) {
        if (!std::get<0>(vg.v_dist_depth)) throw std::runtime_error("backward: the forward ran with distortion; its gradient is required");
        RenderOutput::TensorTuple vd;
        std::get<1>(vd) = DeviceTensor3D<float>(stage(PoolSlot::EngVDistDepth, vg.v_dist_depth, 1), C, H, W);
        if (E.fwd.dist_type == DistortionType::RGB_D)
            std::get<0>(vd) = DeviceTensor3D<float3>((float3*)stage(PoolSlot::EngVDistRgb, vg.v_dist_rgb, 3), C, H, W);
        dist_fwd = E.fwd.distortions; v_dist = vd;
    }
    DeviceTensor3D<float> v_med, amap;
    if (E.fwd.render_median.data_ptr() && std::get<0>(vg.v_median))
        v_med = DeviceTensor3D<float>(stage(PoolSlot::EngVMedian, vg.v_median, 1), C, H, W);
    if (vg.accum_mode != DensifyAccumMode::None && std::get<0>(vg.accum_map))
        amap = DeviceTensor3D<float>(stage(PoolSlot::EngAccumMap, vg.accum_map, 1), C, H, W);
    auto [vw, vs, accum] = rasterize_to_pixels_3dgs_bwd(
        E.cur_num_splats, E.fwd.splats_w, E.fwd.splats_s, E.fwd.gaussian_ids, (uint32_t)W, (uint32_t)H,
        E.fwd.tile_offsets, E.fwd.flatten_ids, E.fwd.render_Ts, E.fwd.last_ids, E.fwd.renders, dist_fwd,
        E.fwd.dist_type, amap, vg.accum_mode, v_renders, v_Ts_t, v_med, v_dist, std::nullopt, std::nullopt);
    if (accum.data_ptr()) { E.fwd.accum_weight = accum; E.fwd.accum_mode = vg.accum_mode; }   // EngineLoss.cpp:243-246
    return vs;
}
}  // namespace

void engine_backward_from_render_grad(TorchTensorView v_render_rgb, TorchTensorView v_render_depth,
                                      TorchTensorView v_render_Ts, DeviceTensor2D<float>* v_viewmats) {
    auto& E = engine();
    if (std::get<0>(E.fwd.renders).data_ptr() == nullptr)
        throw std::runtime_error("engine_backward_from_render_grad: forward_3dgs must be called first");
    alloc_grad_buffers();
    const int64_t H = E.camera.height, W = E.camera.width;
    // _engine_raster_proj_backward, non-fused branch (src/engine/EngineLoss.cpp:218-240,294-390)
    auto vs = raster_backward(v_render_rgb, v_render_depth, v_render_Ts);
    E.grad.v_screen = vs;
    std::vector<DeviceTensorFloatND> v_world = {
        DeviceTensorFloatND(E.grad.means), DeviceTensorFloatND(E.grad.quats), DeviceTensorFloatND(E.grad.scales),
        DeviceTensorFloatND((float*)E.grad.opacities.data_ptr(), {E.grad.opacities.size(), 1}),
        DeviceTensorFloatND(E.grad.features_dc), DeviceTensorFloatND(E.grad.features_sh)};
    std::optional<ssr_detail::AntialiasedScope> antialiased;
    if (E.primitive == "mip") antialiased.emplace();
    projection_3dgs_backward(
        E.cur_num_splats, E.sh_degree, E.fwd.splats_w, E.camera.viewmats, E.camera.intrins, (uint32_t)W, (uint32_t)H,
        E.camera.model_str, E.camera.distortion_str, E.camera.dist_coeffs, E.fwd.camera_ids, E.fwd.gaussian_ids,
        E.fwd.aabb, vs, v_world, v_viewmats, E.world.sh_packed, E.world.sh_bounds, (uint32_t)E.num_sh, E.world.sh_value_bits,
        E.world.sh_bounds_stride);
    E.grad.dirty_list = ssr_ext::last_backward_list(&E.grad.dirty_count);
    E.grad.dirty_key = (const void*)E.grad.means.data_ptr();
    // with no list the backward may have written any row; with one, exactly the listed rows
    E.grad.dirty_valid = E.grad.dirty_list != nullptr || (E.packed && E.fwd.gaussian_ids.size() == 0);
}


void engine_backward_with_variants(TorchTensorView v_render_rgb, TorchTensorView v_render_depth, TorchTensorView v_render_Ts,
                                   TorchTensorView v_dist_rgb, TorchTensorView v_dist_depth, TorchTensorView v_median,
                                   TorchTensorView accum_map, int accum_mode) {
    auto& E = engine();
    if (std::get<0>(E.fwd.renders).data_ptr() == nullptr)
        throw std::runtime_error("engine_backward_with_variants: forward_3dgs must be called first");
    alloc_grad_buffers();
    VariantGrads vg;
    vg.v_dist_rgb = v_dist_rgb; vg.v_dist_depth = v_dist_depth; vg.v_median = v_median; vg.accum_map = accum_map;
    vg.accum_mode = (DensifyAccumMode)accum_mode;
    auto vs = raster_backward(v_render_rgb, v_render_depth, v_render_Ts, vg);
    E.grad.v_screen = vs;
    std::vector<DeviceTensorFloatND> v_world = {
        DeviceTensorFloatND(E.grad.means), DeviceTensorFloatND(E.grad.quats), DeviceTensorFloatND(E.grad.scales),
        DeviceTensorFloatND((float*)E.grad.opacities.data_ptr(), {E.grad.opacities.size(), 1}),
        DeviceTensorFloatND(E.grad.features_dc), DeviceTensorFloatND(E.grad.features_sh)};
    std::optional<ssr_detail::AntialiasedScope> antialiased;
    if (E.primitive == "mip") antialiased.emplace();
    projection_3dgs_backward(
        E.cur_num_splats, E.sh_degree, E.fwd.splats_w, E.camera.viewmats, E.camera.intrins, (uint32_t)E.camera.width,
        (uint32_t)E.camera.height, E.camera.model_str, E.camera.distortion_str, E.camera.dist_coeffs, E.fwd.camera_ids,
        E.fwd.gaussian_ids, E.fwd.aabb, vs, v_world, nullptr, E.world.sh_packed, E.world.sh_bounds, (uint32_t)E.num_sh,
        E.world.sh_value_bits, E.world.sh_bounds_stride);
    E.grad.dirty_list = ssr_ext::last_backward_list(&E.grad.dirty_count);
    E.grad.dirty_key = (const void*)E.grad.means.data_ptr();
    E.grad.dirty_valid = E.grad.dirty_list != nullptr || (E.packed && E.fwd.gaussian_ids.size() == 0);
}

void engine_backward_fused_optimizer(TorchTensorView v_render_rgb, TorchTensorView v_render_depth,
                                     TorchTensorView v_render_Ts, const float hyper[16], int step, bool scale_agnostic_mean,
                                     int quantization_level, int non_sh_optim_bits) {
    auto& E = engine();
    if (std::get<0>(E.fwd.renders).data_ptr() == nullptr)
        throw std::runtime_error("engine_backward_fused_optimizer: forward_3dgs must be called first");
    const int64_t n = E.max_num_splats;
    if (!E.optim.adam_ready) {
        const PoolSlot s1[6] = {PoolSlot::AdamG1Means, PoolSlot::AdamG1Quats, PoolSlot::AdamG1Scales, PoolSlot::AdamG1Opacities,
                                PoolSlot::AdamG1FeaturesDc, PoolSlot::AdamG1FeaturesSh};
        const PoolSlot s2[6] = {PoolSlot::AdamG2Means, PoolSlot::AdamG2Quats, PoolSlot::AdamG2Scales, PoolSlot::AdamG2Opacities,
                                PoolSlot::AdamG2FeaturesDc, PoolSlot::AdamG2FeaturesSh};
        const int64_t ch[6] = {3, 4, 3, 1, 3, 3 * (int64_t)E.num_sh};
        E.optim.g1.clear(); E.optim.g2.clear();
        for (int i = 0; i < 6; i++) {
            float* a = DevicePool::global().acquire<float>(s1[i], (size_t)(n * ch[i]));
            float* b = DevicePool::global().acquire<float>(s2[i], (size_t)(n * ch[i]));
            backend::memset_async(a, 0, (size_t)(n * ch[i]) * sizeof(float));
            backend::memset_async(b, 0, (size_t)(n * ch[i]) * sizeof(float));
            E.optim.g1.emplace_back(a, std::vector<int64_t>{n, ch[i]});
            E.optim.g2.emplace_back(b, std::vector<int64_t>{n, ch[i]});
        }
        E.optim.densify_score.resize(PoolSlot::EngDensifyScore, n);
        E.optim.adam_ready = true;
    }
    std::optional<TorchTensorView> sh_state, sh_state_bounds, sh_values, sh_value_bounds;
    if (quantization_level == 1) {
        // OptimConfig::quantization_level 1: the SH values are the engine's 16-bit codes (set_sh_value_quant with one
        // bound per 256 splats), updated in place; their moments live in two pool slots, all zeros at first
        const int64_t R = 3 * (int64_t)E.num_sh, nb = (n + 255) / 256;
        if (E.world.sh_value_bits != 16 || !E.world.sh_packed || E.world.sh_bounds_stride != 256 * R)
            throw std::runtime_error("engine_backward_fused_optimizer: quantization level 1 needs 16-bit SH values with one bound per 256 splats");
        uint8_t* st = DevicePool::global().acquire<uint8_t>(PoolSlot::AdamShStatePacked, (size_t)(n * R * 2));
        float* sb = DevicePool::global().acquire<float>(PoolSlot::AdamShStateBounds, (size_t)(nb * 4));
        if (!E.optim.sh_state_ready) {
            backend::memset_async(st, 0, (size_t)(n * R * 2));
            backend::memset_async(sb, 0, (size_t)(nb * 4) * sizeof(float));
            E.optim.sh_state_ready = true;
        }
        sh_state = TorchTensorView{(uint64_t)(uintptr_t)st, 1u, std::vector<int64_t>{n * R * 2}};
        sh_state_bounds = TorchTensorView{(uint64_t)(uintptr_t)sb, 4u, std::vector<int64_t>{nb, 4}};
        sh_values = E.world.sh_packed; sh_value_bounds = E.world.sh_bounds;
    }
    // OptimConfig::non_sh_optim_bits (src/engine/EngineConfig.h:120; the trainer sets 16 at every quantized level,
    // src/app/TrainerCore.cpp:383): the moments of the five non-SH tensors as 16-bit cells in two pool slots, tensor
    // after tensor, all zeros at first; read at a quantized level only (src/engine/EngineDensify.cpp:179-193)
    if (non_sh_optim_bits != 32 && non_sh_optim_bits != 16)
        throw std::runtime_error("engine_backward_fused_optimizer: non_sh_optim_bits must be 32 (off) or 16");
    NonShQuantState non_sh;
    if (non_sh_optim_bits == 16 && quantization_level == 1) {
        const int64_t nb = (n + 255) / 256;
        uint8_t* pk = DevicePool::global().acquire<uint8_t>(PoolSlot::AdamNonShPacked, (size_t)(n * 14 * 4));
        float* bd = DevicePool::global().acquire<float>(PoolSlot::AdamNonShBounds, (size_t)(5 * nb * 4));
        if (!E.optim.non_sh_state_ready) {
            backend::memset_async(pk, 0, (size_t)(n * 14 * 4));
            backend::memset_async(bd, 0, (size_t)(5 * nb * 4) * sizeof(float));
            E.optim.non_sh_state_ready = true;
        }
        non_sh.enabled = true;
        non_sh.means_packed = pk;                 non_sh.means_bounds = bd;
        non_sh.quats_packed = pk + n * 3 * 4;     non_sh.quats_bounds = bd + nb * 4;
        non_sh.scales_packed = pk + n * 7 * 4;    non_sh.scales_bounds = bd + 2 * nb * 4;
        non_sh.opacities_packed = pk + n * 10 * 4; non_sh.opacities_bounds = bd + 3 * nb * 4;
        non_sh.features_dc_packed = pk + n * 11 * 4; non_sh.features_dc_bounds = bd + 4 * nb * 4;
    }
    VariantGrads vg;   // the training step's loss map, when one is set: accumulated per splat as the densifier's score
    if (std::get<0>(E.optim.loss_map) && E.optim.loss_map_accum_mode != 0) {
        vg.accum_map = E.optim.loss_map;
        vg.accum_mode = (DensifyAccumMode)E.optim.loss_map_accum_mode;
    }
    E.grad.v_screen = raster_backward(v_render_rgb, v_render_depth, v_render_Ts, vg);
    const int64_t W = E.camera.width, H = E.camera.height;
    DeviceVector<int32_t> cam_ids, gauss_ids;
    DeviceTensorFloatND aabb((float*)E.fwd.aabb.data_ptr(), {E.fwd.aabb.numel(), 4});
    if (E.packed && E.fwd.gaussian_ids.size() > 0) {
        cam_ids = E.fwd.camera_ids; gauss_ids = E.fwd.gaussian_ids;   // aabb and v_screen hold the nnz packed rows
    } else if (E.packed) {
        // nothing visible: every splat still takes its moment decay, so run the plain form on empty extents
        float* zero = DevicePool::global().acquire<float>(PoolSlot::EngZeroAabb, (size_t)(E.cur_num_splats * 4));
        backend::memset_async(zero, 0, (size_t)(E.cur_num_splats * 4) * sizeof(float));
        aabb = DeviceTensorFloatND(zero, {E.cur_num_splats, 4});
    }
    std::optional<ssr_detail::AntialiasedScope> antialiased;
    if (E.primitive == "mip") antialiased.emplace();
    fused_projection_bwd_optimizer_3dgs(
        E.cur_num_splats, E.sh_degree, E.fwd.splats_w, E.camera.viewmats, E.camera.intrins, (uint32_t)W, (uint32_t)H,
        E.camera.model_str, E.camera.distortion_str, E.camera.dist_coeffs, cam_ids, gauss_ids, aabb, {}, E.grad.v_screen,
        E.optim.g1, E.optim.g2, sh_state, sh_state_bounds, sh_values, sh_value_bounds, non_sh,
        E.optim.radii, E.optim.densify_score, hyper[0], hyper[1], hyper[2], hyper[3], hyper[4], hyper[5], hyper[6], hyper[7],
        hyper[8], hyper[9], hyper[12], hyper[13], hyper[10], hyper[11], scale_agnostic_mean, hyper[14] != 0.0f, hyper[15], (int32_t)step,
        quantization_level);
}

void engine_copy_params_to_host(TorchTensorView means, TorchTensorView quats, TorchTensorView scales,
                                TorchTensorView opacities, TorchTensorView features_dc, TorchTensorView features_sh) {
    auto& w = engine().world;
    auto put = [](void* dst, const void* src, size_t bytes) {
        if (dst && src && bytes) backend::memcpy_sync(dst, src, bytes, backend::MemcpyKind::DeviceToHost);
    };
    put((void*)std::get<0>(means), w.means.data_ptr(), w.means.size() * sizeof(float3));
    put((void*)std::get<0>(quats), w.quats.data_ptr(), w.quats.size() * sizeof(float4));
    put((void*)std::get<0>(scales), w.scales.data_ptr(), w.scales.size() * sizeof(float3));
    put((void*)std::get<0>(opacities), w.opacities.data_ptr(), w.opacities.size() * sizeof(float));
    put((void*)std::get<0>(features_dc), w.features_dc.data_ptr(), w.features_dc.size() * sizeof(float3));
    put((void*)std::get<0>(features_sh), w.features_sh.data_ptr(), w.features_sh.numel() * sizeof(float3));
}

void engine_copy_render_to_host(TorchTensorView out_rgb, TorchTensorView out_depth, TorchTensorView out_Ts,
                                TorchTensorView, TorchTensorView) {
    // the copies below wait for the device anyway: settle counts that were left there, so that an image whose
    // intersection did not fit its arrays is refused instead of handed out with fragments missing
    ssr_ext::resolve_counts();
    auto& f = engine().fwd;
    auto& rgb = std::get<0>(f.renders);
    auto& depth = std::get<1>(f.renders);
    if (rgb.data_ptr() && std::get<0>(out_rgb))
        backend::memcpy_sync((void*)std::get<0>(out_rgb), rgb.data_ptr(), rgb.numel() * sizeof(float3), backend::MemcpyKind::DeviceToHost);
    if (depth.data_ptr() && std::get<0>(out_depth))
        backend::memcpy_sync((void*)std::get<0>(out_depth), depth.data_ptr(), depth.numel() * sizeof(float), backend::MemcpyKind::DeviceToHost);
    if (f.render_Ts.data_ptr() && std::get<0>(out_Ts))
        backend::memcpy_sync((void*)std::get<0>(out_Ts), f.render_Ts.data_ptr(), f.render_Ts.numel() * sizeof(float), backend::MemcpyKind::DeviceToHost);
}

void engine_copy_grads_to_host(TorchTensorView means, TorchTensorView quats, TorchTensorView scales,
                               TorchTensorView opacities, TorchTensorView features_dc, TorchTensorView features_sh) {
    auto& g = engine().grad;
    auto put = [](void* dst, const void* src, size_t bytes) {
        if (dst && src && bytes) backend::memcpy_sync(dst, src, bytes, backend::MemcpyKind::DeviceToHost);
    };
    put((void*)std::get<0>(means), g.means.data_ptr(), g.means.size() * sizeof(float3));
    put((void*)std::get<0>(quats), g.quats.data_ptr(), g.quats.size() * sizeof(float4));
    put((void*)std::get<0>(scales), g.scales.data_ptr(), g.scales.size() * sizeof(float3));
    put((void*)std::get<0>(opacities), g.opacities.data_ptr(), g.opacities.size() * sizeof(float));
    put((void*)std::get<0>(features_dc), g.features_dc.data_ptr(), g.features_dc.size() * sizeof(float3));
    put((void*)std::get<0>(features_sh), g.features_sh.data_ptr(), g.features_sh.numel() * sizeof(float3));
}

// ---------------------------------------------------------------------------------------------
// C entry points for Python (tests, smoke, bench). Exceptions become a return code and a message.
namespace {
thread_local std::string g_host_error;
template <class F> int guard(F&& f) {
    try { f(); return 0; }
    catch (const std::exception& e) { g_host_error = e.what(); return 1; }
}
TorchTensorView tv(const void* p, uint32_t elem, std::vector<int64_t> shape) { return TorchTensorView((uint64_t)p, elem, std::move(shape)); }
}  // namespace

extern "C" {

const char* ssrh_last_error(void) { static thread_local std::string out; out.swap(g_host_error); g_host_error.clear(); return out.c_str(); }

int ssrh_init(int device) { return guard([&] { if (!backend::device_select(device)) throw std::runtime_error(std::string("device_select failed: ") + backend::last_error()); }); }

int ssrh_reset(void) { return guard([&] { engine_reset(); }); }

int ssrh_set_options(int fuse_tile_count, int visible_list, int packed_rows, int overwrite_world_grads,
                     int sh_int8_f16scale, int stage_profiling, int packed_vscreen, int tile_sort) {
    return guard([&] {
        auto& o = ssr_ext::options();
        o.fuse_tile_count = fuse_tile_count != 0; o.visible_list = visible_list != 0;
        o.packed_rows = packed_rows != 0;
        o.overwrite_world_grads = overwrite_world_grads != 0;
        o.sh_int8_f16scale = sh_int8_f16scale != 0;
        o.packed_vscreen = packed_vscreen != 0;
        o.tile_sort = tile_sort != 0;
        ssr_ext::set_stage_profiling(stage_profiling != 0);
    });
}

// on: the intersection count stays on the device between the forward's stages (Options::deferred_counts);
// capacity >= 0 also sets the size of the next call's key arrays (0: that call reads its count).
int ssrh_set_deferred_counts(int on, int64_t capacity) {
    return guard([&] {
        ssr_ext::options().deferred_counts = on != 0;
        if (capacity >= 0) ssr_ext::set_deferred_capacity(capacity);
    });
}
int64_t ssrh_deferred_capacity(void) { return ssr_ext::deferred_capacity(); }

// on: the packed projection keeps the parameters of the visible splats (64 bytes each, in four planes) and the projection backward
// reads them (Options::packed_world_rows)
int ssrh_set_packed_world_rows(int on) {
    return guard([&] { ssr_ext::options().packed_world_rows = on != 0; });
}

// -1: the adapter chooses the cut of the compositing backward; 0 / 1: rows / lanes (Options::backward_schedule)
int ssrh_set_backward_schedule(int schedule) {
    return guard([&] {
        if (schedule < -1 || schedule > 1) throw std::runtime_error("ssrh_set_backward_schedule: -1 (auto), 0 (rows) or 1 (lanes)");
        ssr_ext::options().backward_schedule = schedule;
    });
}

// host or device pointers; num_sh = coefficients per splat excluding DC (15 for SH3)
int ssrh_set_data_3dgs(int64_t n, const float* means, const float* quats, const float* scales, const float* opacities,
                       const float* dc, const float* sh, int num_sh) {
    return guard([&] {
        set_data_3dgs(n, tv(means, 4, {n, 3}), tv(quats, 4, {n, 4}), tv(scales, 4, {n, 3}), tv(opacities, 4, {n, 1}),
                      tv(dc, 4, {n, 3}), tv(sh, 4, {n, num_sh, 3}));
    });
}

int ssrh_set_sh_value_quant(int bits, const void* packed, int64_t packed_count, int packed_elem, const void* bounds,
                            int64_t bounds_count, int bounds_elem, int64_t bounds_stride) {
    return guard([&] { set_sh_value_quant(bits, tv(packed, (uint32_t)packed_elem, {packed_count}), tv(bounds, (uint32_t)bounds_elem, {bounds_count}), bounds_stride); });
}

// dist_coeffs: [num_cameras, 8] lens coefficients in the tier's order, or NULL for all zeros
int ssrh_set_camera_params(int width, int height, const char* model, const char* distortion, const float* viewmats,
                           const float* intrins, const float* dist_coeffs, int num_cameras) {
    return guard([&] {
        static const float zero_coeffs[8 * 16] = {0};
        if (!dist_coeffs && num_cameras > 16) throw std::runtime_error("set_camera_params: pass dist_coeffs for more than 16 cameras");
        set_camera_params(width, height, model, distortion, tv(viewmats, 4, {num_cameras, 4, 4}), tv(intrins, 4, {num_cameras, 4}),
                          tv(dist_coeffs ? dist_coeffs : zero_coeffs, 4, {num_cameras, 8}));
    });
}

// Quantization level 1: copies the SH state to the host (any pointer may be NULL): moments [N * 3 * num_sh] uint16
// cells and float4 bounds per 256 splats, values [N * 3 * num_sh] uint16 codes and float2 bounds per 256 splats.
int ssrh_copy_sh_quant_state(uint16_t* state_packed, float* state_bounds, uint16_t* value_packed, float* value_bounds) {
    return guard([&] {
        auto& E = engine();
        const int64_t n = E.max_num_splats, R = 3 * (int64_t)E.num_sh, nb = (n + 255) / 256;
        auto get = [](void* dst, const void* src, size_t bytes) {
            if (dst && src && bytes) backend::memcpy_sync(dst, src, bytes, backend::MemcpyKind::DeviceToHost);
        };
        if (E.optim.sh_state_ready) {
            get(state_packed, DevicePool::global().acquire<uint8_t>(PoolSlot::AdamShStatePacked, (size_t)(n * R * 2)), (size_t)(n * R * 2));
            get(state_bounds, DevicePool::global().acquire<float>(PoolSlot::AdamShStateBounds, (size_t)(nb * 4)), (size_t)(nb * 4) * sizeof(float));
        }
        if (E.world.sh_packed) get(value_packed, (const void*)std::get<0>(*E.world.sh_packed), (size_t)(n * R * 2));
        if (E.world.sh_bounds) get(value_bounds, (const void*)std::get<0>(*E.world.sh_bounds), (size_t)(nb * 2) * sizeof(float));
    });
}

int ssrh_set_tile_mask(const uint8_t* mask, int h_mask, int w_mask) {
    // one mask per camera of the current camera set, [C, h_mask, w_mask]
    return guard([&] { engine_set_tile_mask(tv(mask, 1, {std::max<int64_t>(1, engine().camera.num), h_mask, w_mask})); });
}

int ssrh_forward_3dgs(const char* primitive, int sh_degree, int packed, int output_median, int dist_type) {
    return guard([&] { forward_3dgs(primitive, sh_degree, packed != 0, output_median != 0, dist_type); });
}

int ssrh_backward_from_render_grad(const float* v_rgb, const float* v_depth, const float* v_Ts) {
    return guard([&] {
        const int64_t C = engine().camera.num, H = engine().camera.height, W = engine().camera.width;
        engine_backward_from_render_grad(tv(v_rgb, 4, {C, H, W, 3}), tv(v_depth, 4, {C, H, W, 1}), tv(v_Ts, 4, {C, H, W, 1}));
    });
}

// The backward with the camera-pose gradient as well (the launch function's v_viewmats; the reference's engine
// itself always passes null): out16 receives dL/d[R|t] as a row-major 4x4 whose last row is zero.
int ssrh_backward_with_pose_grad(const float* v_rgb, const float* v_depth, const float* v_Ts, float* out16) {
    return guard([&] {
        const int64_t C = engine().camera.num, H = engine().camera.height, W = engine().camera.width;
        float* d = DevicePool::global().acquire<float>(PoolSlot::EngPoseGrad, (size_t)(16 * C));
        backend::memset_async(d, 0, (size_t)(16 * C) * sizeof(float));
        DeviceTensor2D<float> vm(d, C, 16);
        engine_backward_from_render_grad(tv(v_rgb, 4, {C, H, W, 3}), tv(v_depth, 4, {C, H, W, 1}), tv(v_Ts, 4, {C, H, W, 1}), &vm);
        backend::memcpy_sync(out16, d, (size_t)(16 * C) * sizeof(float), backend::MemcpyKind::DeviceToHost);
    });
}

int ssrh_backward_with_variants(const float* v_rgb, const float* v_depth, const float* v_Ts, const float* v_dist_rgb,
                                const float* v_dist_depth, const float* v_median, const float* accum_map, int accum_mode) {
    return guard([&] {
        const int64_t C = engine().camera.num, H = engine().camera.height, W = engine().camera.width;
        engine_backward_with_variants(tv(v_rgb, 4, {C, H, W, 3}), tv(v_depth, 4, {C, H, W, 1}), tv(v_Ts, 4, {C, H, W, 1}),
                                      tv(v_dist_rgb, 4, {C, H, W, 3}), tv(v_dist_depth, 4, {C, H, W, 1}), tv(v_median, 4, {C, H, W, 1}),
                                      tv(accum_map, 4, {C, H, W, 1}), accum_mode);
    });
}

// The loss map [C,H,W] (device or host pointer, kept by the caller until the backward has run) that the fused
// training step accumulates per splat with `accum_mode` (1 max, 2 sum, 3 avg); null or mode 0 switches it off.
int ssrh_set_loss_map(const float* map, int accum_mode) {
    return guard([&] {
        auto& E = engine();
        if (accum_mode < 0 || accum_mode > 3) throw std::runtime_error("ssrh_set_loss_map: accum_mode must be 0..3");
        const int64_t C = E.camera.num, H = E.camera.height, W = E.camera.width;
        E.optim.loss_map = map ? tv(map, 4, {C, H, W}) : TorchTensorView{0, 4, {}};
        E.optim.loss_map_accum_mode = map ? accum_mode : 0;
    });
}

int ssrh_backward_fused_optimizer(const float* v_rgb, const float* v_depth, const float* v_Ts, const float* hyper16, int step,
                                  int scale_agnostic_mean, int quantization_level, int non_sh_optim_bits) {
    return guard([&] {
        const int64_t C = engine().camera.num, H = engine().camera.height, W = engine().camera.width;
        engine_backward_fused_optimizer(tv(v_rgb, 4, {C, H, W, 3}), tv(v_depth, 4, {C, H, W, 1}), tv(v_Ts, 4, {C, H, W, 1}), hyper16, step,
                                        scale_agnostic_mean != 0, quantization_level, non_sh_optim_bits);
    });
}

// non_sh_optim_bits 16: copies the quantized non-SH moments to the host: 14 * N 32-bit cells (means, quats, scales,
// opacities, dc, tensor after tensor) and 5 x ceil(N / 256) float4 bounds in the same order.
int ssrh_copy_non_sh_quant_state(uint32_t* packed, float* bounds) {
    return guard([&] {
        auto& E = engine();
        const int64_t n = E.max_num_splats, nb = (n + 255) / 256;
        if (!E.optim.non_sh_state_ready) throw std::runtime_error("ssrh_copy_non_sh_quant_state: no quantized non-SH state yet");
        if (packed)
            backend::memcpy_sync(packed, DevicePool::global().acquire<uint8_t>(PoolSlot::AdamNonShPacked, (size_t)(n * 14 * 4)),
                                 (size_t)(n * 14 * 4), backend::MemcpyKind::DeviceToHost);
        if (bounds)
            backend::memcpy_sync(bounds, DevicePool::global().acquire<float>(PoolSlot::AdamNonShBounds, (size_t)(5 * nb * 4)),
                                 (size_t)(5 * nb * 4) * sizeof(float), backend::MemcpyKind::DeviceToHost);
    });
}

int ssrh_copy_params_to_host(float* means, float* quats, float* scales, float* opacities, float* dc, float* sh) {
    return guard([&] {
        const int64_t n = engine().max_num_splats;
        engine_copy_params_to_host(tv(means, 4, {n, 3}), tv(quats, 4, {n, 4}), tv(scales, 4, {n, 3}), tv(opacities, 4, {n, 1}),
                                   tv(dc, 4, {n, 3}), tv(sh, 4, {n, engine().num_sh, 3}));
    });
}

int ssrh_copy_render_to_host(float* rgb, float* depth, float* Ts) {
    return guard([&] {
        const int64_t C = engine().camera.num, H = engine().camera.height, W = engine().camera.width;
        engine_copy_render_to_host(tv(rgb, 4, {C, H, W, 3}), tv(depth, 4, {C, H, W, 1}), tv(Ts, 4, {C, H, W, 1}), tv(nullptr, 4, {0}), tv(nullptr, 4, {0}));
    });
}

int ssrh_copy_grads_to_host(float* means, float* quats, float* scales, float* opacities, float* dc, float* sh) {
    return guard([&] {
        const int64_t n = engine().max_num_splats;
        engine_copy_grads_to_host(tv(means, 4, {n, 3}), tv(quats, 4, {n, 4}), tv(scales, 4, {n, 3}), tv(opacities, 4, {n, 1}),
                                  tv(dc, 4, {n, 3}), tv(sh, 4, {n, engine().num_sh, 3}));
    });
}

// Device addresses of the forward cache, for tests that compare intermediate buffers.
//   which: 0 aabb, 1 sort depths, 2..6 screen xy/depth/conic/opac/rgb, 7 sorted keys, 8 sorted ids,
//          9 tile offsets, 10 last_ids, 11 radii, 12..16 v_screen xy/depth/conic/opac/rgb,
//          17 gaussian_ids, 18 camera_ids (packed projection), 19/20 distortion rgb/depth, 21 median depth,
//          22 accumulated weights
int ssrh_cache_pointer(int which, void** ptr, int64_t* count) {
    return guard([&] {
        auto& E = engine();
        auto nd = [&](const DeviceTensorFloatND& t) { *ptr = t.data_ptr(); *count = t.numel(); };
        switch (which) {
            case 0: *ptr = E.fwd.aabb.data_ptr(); *count = E.fwd.aabb.numel() * 4; break;
            case 1: *ptr = E.fwd.depths.data_ptr(); *count = E.fwd.depths.numel(); break;
            case 2: case 3: case 4: case 5: case 6: nd(E.fwd.splats_s.at(which - 2)); break;
            case 7: *ptr = E.fwd.isect_ids.data_ptr(); *count = E.fwd.isect_ids.size(); break;
            case 8: *ptr = E.fwd.flatten_ids.data_ptr(); *count = E.fwd.flatten_ids.size(); break;
            case 9: *ptr = E.fwd.tile_offsets.data_ptr(); *count = E.fwd.tile_offsets.numel(); break;
            case 10: *ptr = E.fwd.last_ids.data_ptr(); *count = E.fwd.last_ids.numel(); break;
            case 11: *ptr = E.optim.radii.data_ptr(); *count = E.optim.radii.size(); break;
            case 12: case 13: case 14: case 15: case 16: nd(E.grad.v_screen.at(which - 12)); break;
            case 19: *ptr = std::get<0>(E.fwd.distortions).data_ptr(); *count = std::get<0>(E.fwd.distortions).numel() * 3; break;
            case 20: *ptr = std::get<1>(E.fwd.distortions).data_ptr(); *count = std::get<1>(E.fwd.distortions).numel(); break;
            case 21: *ptr = E.fwd.render_median.data_ptr(); *count = E.fwd.render_median.numel(); break;
            case 22: *ptr = E.fwd.accum_weight.data_ptr(); *count = E.fwd.accum_weight.size(); break;
            case 17: *ptr = E.fwd.gaussian_ids.data_ptr(); *count = E.fwd.gaussian_ids.size(); break;
            case 18: *ptr = E.fwd.camera_ids.data_ptr(); *count = E.fwd.camera_ids.size(); break;
            default: throw std::runtime_error("unknown cache buffer");
        }
    });
}

// -2: the count did not fit the arrays it was left to (deferred counts); the message is in ssrh_last_error
int64_t ssrh_last_n_isects(void) { int64_t v = -2; guard([&] { v = ssr_ext::last_n_isects(); }); return v; }
int64_t ssrh_short_frames(void) { return ssr_ext::short_frames(); }
int64_t ssrh_last_n_visible(void) { int64_t v = -2; guard([&] { v = ssr_ext::last_n_visible(); }); return v; }

int ssrh_last_stage_times(float* out9) {
    return guard([&] {
        auto t = ssr_ext::last_stage_times();
        const float v[9] = {t.k1, t.k2, t.k3, t.k4, t.k5, t.k6, t.k7, t.k8, t.k9};
        std::memcpy(out9, v, sizeof(v));
    });
}

// Runs `iters` forward+backward iterations back to back with device-resident cotangents and
// returns the elapsed device time of each (events on the launch stream, one synchronise per
// iteration at its end).
int ssrh_time_iterations(int sh_degree, int packed, const float* v_rgb_dev, const float* v_depth_dev, const float* v_Ts_dev,
                         int iters, float* ms_out) {
    return guard([&] {
        ssr_event_t a = ssr_event_create(), b = ssr_event_create();
        const std::string primitive = engine().primitive.empty() ? "3dgs" : engine().primitive;   // as the last forward
        for (int i = 0; i < iters; i++) {
            ssr_event_record(a, nullptr);
            forward_3dgs(primitive, sh_degree, packed != 0, false, 0);
            const int64_t C = engine().camera.num, H = engine().camera.height, W = engine().camera.width;
            engine_backward_from_render_grad(tv(v_rgb_dev, 4, {C, H, W, 3}), tv(v_depth_dev, 4, {C, H, W, 1}), tv(v_Ts_dev, 4, {C, H, W, 1}));
            ssr_event_record(b, nullptr);
            float ms = 0;
            if (ssr_event_elapsed_ms(a, b, &ms)) throw std::runtime_error(ssr_last_error());
            ms_out[i] = ms;
        }
        ssr_event_destroy(a); ssr_event_destroy(b);
    });
}

size_t ssrh_pool_bytes(void) { return DevicePool::global().total_bytes(); }

// The sort / scan seam (ssr_sortscan.hpp) for callers without C++: device arrays in, *selector_out says which
// buffer of each pair holds the sorted data afterwards (0: keys_current / values_current).
int ssrh_sort_pairs_i64_i32(int64_t* keys_current, int64_t* keys_alternate, int32_t* values_current, int32_t* values_alternate,
                            int64_t num_items, int begin_bit, int end_bit, int* selector_out) {
    return guard([&] {
        backend::DoubleBuffer<int64_t> keys(keys_current, keys_alternate);
        backend::DoubleBuffer<int32_t> values(values_current, values_alternate);
        backend::sort_pairs<int64_t, int32_t>(keys, values, num_items, begin_bit, end_bit);
        if (keys.selector != values.selector) throw std::runtime_error("sort_pairs left keys and values in different buffers");
        if (selector_out) *selector_out = keys.selector;
    });
}
int ssrh_inclusive_sum_i64(const int64_t* in, int64_t* out, int64_t num_items) {
    return guard([&] { backend::inclusive_sum<int64_t>(in, out, num_items); });
}

}  // extern "C"
