// ssr_engine.hpp -- the caller side of the path: a process-global engine state that drives the
// launch functions in the reference's order, with the reference's zero-fills and buffer lifetimes.
//
//   set_data_3dgs                     src/engine/EngineSetup.cpp:11-47
//   set_camera_params                 src/engine/EngineSetup.cpp:50-87
//   forward_3dgs                      src/engine/EngineForward.cpp:24-311
//   engine_backward_from_render_grad  src/engine/EngineLoss.cpp:400-433 (-> :138-391, non-fused branch)
//   engine_copy_render_to_host        src/engine/EngineQuery.cpp:36-76
//   engine_copy_grads_to_host         src/engine/EngineQuery.cpp:122-140
//
// Inputs that are already device addresses are used in place; host memory is copied once
// (src/engine/EngineCommon.h:90-105). The forward cache is retained for the backward
// (src/engine/EngineState.h:127-160).
#pragma once
#include "ssr_backend_api.hpp"

struct EngineState {
    int64_t cur_num_splats = 0, max_num_splats = 0;
    int num_sh = 0, sh_degree = 0;
    std::string primitive;
    bool packed = false;
    struct {
        bool initialized = false;
        DeviceVector<float3> means; DeviceVector<float4> quats; DeviceVector<float3> scales;
        DeviceVector<float> opacities; DeviceVector<float3> features_dc; DeviceTensor2D<float3> features_sh;
        int sh_value_bits = 32;
        std::optional<TorchTensorView> sh_packed, sh_bounds;
        int64_t sh_bounds_stride = 0;
    } world;
    struct {
        int width = 0, height = 0, num = 0;
        std::string model_str = "PINHOLE", distortion_str = "NONE";
        TorchTensorView viewmats, intrins, dist_coeffs;
    } camera;
    struct {
        DeviceVector<float> radii; bool skip_grad_zero = false;
        // which rows of `radii` are known to hold zeros or the last projection's values (forward_3dgs)
        const float* radii_zeroed_ptr = nullptr; int64_t radii_zeroed_rows = 0, radii_stored_rows = 0;
        bool adam_ready = false;
        bool sh_state_ready = false;   // quantization level 1: the 8-bit SH moments have been zeroed
        bool non_sh_state_ready = false;   // non_sh_optim_bits 16: the 16-bit non-SH moments have been zeroed
        std::vector<DeviceTensorFloatND> g1, g2;   // Adam moments, shaped like the world tensors
        DeviceVector<float> densify_score;
        // the loss map of the training step and how the compositing backward accumulates it per splat
        // (cfg.loss.loss_map_accum_mode, src/engine/EngineTrainStep.cpp:256-258); null map: no accumulation
        TorchTensorView loss_map{0, 4, {}};
        int loss_map_accum_mode = 0;
    } optim;
    struct {
        std::vector<DeviceTensorFloatND> splats_w, splats_s;
        DeviceTensor2D<float4> aabb; DeviceTensor2D<float> depths;
        DeviceVector<int32_t> camera_ids, gaussian_ids;   // packed projection only
        // Tile-skip map for the NEXT forward only: whoever wants tiles skipped sets it right before,
        // so a later render cannot inherit it (src/engine/EngineForward.cpp:245-252).
        DeviceVector<int32_t> tile_active;
        DeviceVector<int64_t> isect_ids; DeviceVector<int32_t> flatten_ids; DeviceTensor3D<int32_t> tile_offsets;
        RenderOutput::TensorTuple renders; DeviceTensor3D<float> render_Ts; DeviceTensor3D<int32_t> last_ids;
        RenderOutput::TensorTuple distortions; DistortionType dist_type = DistortionType::None;   // EngineForward.cpp:287-291
        DeviceTensor3D<float> render_median;
        DeviceVector<float> accum_weight; DensifyAccumMode accum_mode = DensifyAccumMode::None;    // EngineLoss.cpp:243-246
    } fwd;
    struct {
        DeviceVector<float3> means; DeviceVector<float4> quats; DeviceVector<float3> scales;
        DeviceVector<float> opacities; DeviceVector<float3> features_dc; DeviceTensor2D<float3> features_sh;
        std::vector<DeviceTensorFloatND> v_screen;
        // rows that are not zero: those of the list the last backward wrote (valid while the
        // gradient buffers stay where they are and nobody else writes them)
        const int32_t* dirty_list = nullptr;
        int64_t dirty_count = 0;
        const void* dirty_key = nullptr;
        bool dirty_valid = false;
    } grad;
};
EngineState& engine();
void engine_reset();   // drop all state (not the pool)

void set_data_3dgs(int64_t num_splats, TorchTensorView means, TorchTensorView quats, TorchTensorView scales,
                   TorchTensorView opacities, TorchTensorView features_dc, TorchTensorView features_sh);
// quantized SH storage (engine().world.features_sh_quant*, src/engine/EngineForward.cpp:76-116)
void set_sh_value_quant(int sh_value_bits, TorchTensorView packed, TorchTensorView bounds, int64_t bounds_stride);
void set_camera_params(int width, int height, std::string camera_model, std::string distortion,
                       TorchTensorView viewmats, TorchTensorView intrins, TorchTensorView dist_coeffs);
// computes engine().fwd.tile_active from a [1, H_mask, W_mask] bool mask (host or device), as the
// training step does from the ground-truth alpha (src/engine/EngineTrainStep.cpp:100-104)
void engine_set_tile_mask(TorchTensorView mask);
void forward_3dgs(std::string primitive, int sh_degree, bool packed, bool output_median, int dist_type_int);
void engine_backward_from_render_grad(TorchTensorView v_render_rgb, TorchTensorView v_render_depth,
                                      TorchTensorView v_render_Ts, DeviceTensor2D<float>* v_viewmats = nullptr);
// Backward with the projection backward folded into the optimizer step
// (engine().optim.use_fused_proj_bwd_optim, src/engine/EngineLoss.cpp:286-290): compositing backward,
// then fused_projection_bwd_optimizer_3dgs on the engine's parameters with Adam moments kept in pool
// slots (zero on first use). hyper: lr_means, lr_quats, lr_scales, lr_opacs, lr_dc, lr_sh,
// max_gauss_ratio, scale_reg_w, mcmc_opacity_w, mcmc_scale_w, quat_norm_w, sh_reg_w, erank_w, erank_w_s3,
// color_trust_linear (0 / 1), eps_tr.
// scale_agnostic_mean: OptimConfig::use_scale_agnostic_mean (the means step on the forward's radii).
// quantization_level 1: SH values stay the 16-bit codes of set_sh_value_quant (one bound per 256 splats) and are
// updated in place, their moments are 8-bit cells in pool slots (OptimConfig::quantization_level).
// non_sh_optim_bits 16 (OptimConfig::non_sh_optim_bits; with a quantized level only): the moments of the five
// non-SH tensors are 16-bit cells in pool slots instead of the fp32 arrays.
void engine_backward_fused_optimizer(TorchTensorView v_render_rgb, TorchTensorView v_render_depth,
                                     TorchTensorView v_render_Ts, const float hyper[16], int step,
                                     bool scale_agnostic_mean = false, int quantization_level = 0, int non_sh_optim_bits = 32);
// engine_backward_from_render_grad with the cotangents of the variants of the forward that ran
// (any may be a null view): distortion image, median depth, and a pixel weight map to accumulate
// per splat (the reference feeds these from its loss, src/engine/EngineLoss.cpp:138-216).
void engine_backward_with_variants(TorchTensorView v_render_rgb, TorchTensorView v_render_depth, TorchTensorView v_render_Ts,
                                   TorchTensorView v_dist_rgb, TorchTensorView v_dist_depth, TorchTensorView v_median,
                                   TorchTensorView accum_map, int accum_mode);
void engine_copy_params_to_host(TorchTensorView means, TorchTensorView quats, TorchTensorView scales,
                                TorchTensorView opacities, TorchTensorView features_dc, TorchTensorView features_sh);
void engine_copy_render_to_host(TorchTensorView out_rgb, TorchTensorView out_depth, TorchTensorView out_Ts,
                                TorchTensorView out_rgb_raw, TorchTensorView out_median);
void engine_copy_grads_to_host(TorchTensorView means, TorchTensorView quats, TorchTensorView scales,
                               TorchTensorView opacities, TorchTensorView features_dc, TorchTensorView features_sh);
