// projection_device.h -- per-Gaussian projection and SH colour as device functions, shared by the
// forward (K1) and backward (K9) kernels.
//
// Follows projection_3dgs<camera_model, D, assume_valid, eval3d=false>
// (src/shaders/primitive_3dgs.slang:419-578), persp_proj_3dgs (:63-99), fisheye_proj_3dgs /
// equisolid_proj_3dgs (:148-192), equirect_proj_3dgs (:194-211), quat_scale_to_covar / covarW2C / inverse (src/shaders/projection_utils.slang:69-174),
// view_radius_3dgs (:1033-1043) and sh_coeffs_to_color (src/shaders/harmonics.slang:154-251).
//
// Every expression is evaluated in the order written, without contraction, so that the outputs
// that feed tile keys (extents, sorting depth, conic, opacity) have one defined bit pattern.
#pragma once
#include "common.h"
#include "../../include/ssr_camera.h"

namespace ssr {

struct CamD {
    int model;
    int tier;          // lens distortion tier, SSR_LENS_*
    float Wf, Hf;
    float R[3][3];
    float t[3];
    float fx, fy, cx, cy;
    float dc[8];       // lens coefficients (zero without distortion)
    bool aa;           // antialiased ("mip") variant: set by the kernel from its parameters, not part of the camera
};

// PINHOLE without lens distortion and EQUIRECTANGULAR have hand-written Jacobians; every other pair
// goes through the differentiated model functions of ssr_camera.h (kLens instantiations).
__host__ __device__ __forceinline__ bool camera_needs_lens_path(int model, int tier) {
    return !((model == SSR_CAM_PINHOLE && tier == SSR_LENS_NONE) || model == SSR_CAM_EQUIRECT);
}

__device__ __forceinline__ CamD load_camera(const ssr_camera& c) {
    // src/kernels/projection/ProjectionFwd_kernel.cuh:52-60 (row-major [R t; 0 1])
    CamD k;
    k.aa = false;
    k.model = c.camera_model;
    k.Wf = (float)c.width; k.Hf = (float)c.height;
#pragma unroll
    for (int i = 0; i < 3; i++) {
#pragma unroll
        for (int j = 0; j < 3; j++) k.R[i][j] = c.viewmats[4 * i + j];
        k.t[i] = c.viewmats[4 * i + 3];
    }
    k.fx = c.intrins[0]; k.fy = c.intrins[1]; k.cx = c.intrins[2]; k.cy = c.intrins[3];
    k.tier = c.distortion;
#pragma unroll
    for (int i = 0; i < 8; i++) k.dc[i] = (c.distortion != SSR_LENS_NONE) ? c.dist_coeffs[i] : 0.0f;
    return k;
}

struct ProjD {
    bool valid;
    float aabb[4];
    float sort_depth, radius;
    float xy[2], depth, conic[3], opac;
    float sig, comp, det_orig, det_blur, c2o[2];   // antialiased variant: sigmoid(logit), the compensation factor, both determinants, the diagonal before the blur
    // intermediates for the VJP
    float mc[3], qn[4], qinv, s[3], Rq[3][3], M[3][3], J[2][3], covc[3][3], c2[2][2];
    bool clamp_lo[2], clamp_hi[2];
};

__device__ __forceinline__ float dot3(const float a[3], const float b[3]) {
    return (a[0] * b[0] + a[1] * b[1]) + a[2] * b[2];
}

__device__ __forceinline__ float view_radius(const float mean[3], const float ls[3], float logit,
                                             const float campos[3]) {
    float extend = ssr_sqrt(2.0f * ssr_log(ssr_max(255.0f / (1.0f + ssr_exp(-logit)), 1.0f)));
    float radius = ssr_exp(ssr_max(ls[0], ssr_max(ls[1], ls[2]))) * extend;
    float d[3] = {mean[0] - campos[0], mean[1] - campos[1], mean[2] - campos[2]};
    float dist = ssr_sqrt(dot3(d, d));
    return radius / (ssr_max(dist, radius) + ssr_sqrt(ssr_max(dist * dist - radius * radius, 0.0f)));
}

// J[.][2] of a perspective camera is clamped to the cone of the (enlarged) image,
// src/shaders/primitive_3dgs.slang:84-95; the y limits reuse the x limits as written there.
__device__ __forceinline__ void clamp_pinhole_jacobian(const CamD& cam, float z, ProjD& p) {
    float (*J)[3] = p.J;
    const float lim_pos = cam.Wf + 0.3f * (0.5f * cam.Wf);
    const float lim_neg = 0.3f * (0.5f * cam.Wf);
    const float rz = 1.f / z;
    const float max_x = (-((-lim_neg) - cam.cx)) * rz, min_x = (-(lim_pos - cam.cx)) * rz;
    const float max_y = (-((-lim_neg) - cam.cy)) * rz, min_y = (-(lim_pos - cam.cy)) * rz;
    p.clamp_lo[0] = J[0][2] < min_x; p.clamp_hi[0] = !p.clamp_lo[0] && J[0][2] > max_x;
    p.clamp_lo[1] = J[1][2] < min_y; p.clamp_hi[1] = !p.clamp_lo[1] && J[1][2] > max_y;
    J[0][2] = ssr_min(ssr_max(J[0][2], min_x), max_x);
    J[1][2] = ssr_min(ssr_max(J[1][2], min_y), max_y);
}

template <bool kAssumeValid, bool kLens = false>
__device__ __forceinline__ void project(const CamD& cam, const float mean[3], const float quat[4],
                                        const float ls[3], float logit, ProjD& p) {
    p.valid = false;
#pragma unroll
    for (int i = 0; i < 4; i++) p.aabb[i] = 0.0f;
    p.sort_depth = 0.0f; p.radius = 0.0f;
    p.xy[0] = p.xy[1] = 0.0f; p.conic[0] = p.conic[1] = p.conic[2] = 0.0f; p.opac = 0.0f;
#pragma unroll
    for (int i = 0; i < 3; i++)
        p.mc[i] = ((cam.R[i][0] * mean[0] + cam.R[i][1] * mean[1]) + cam.R[i][2] * mean[2]) + cam.t[i];
    const float x = p.mc[0], y = p.mc[1], z = p.mc[2];
    const float len = ssr_sqrt(dot3(p.mc, p.mc));
    const float cull_z = (cam.model == SSR_CAM_PINHOLE) ? z : len;
    p.depth = len;
    if (!kAssumeValid && cull_z <= 0.0f) return;

    p.opac = 1.0f / (1.0f + ssr_exp(-logit));

    p.qinv = 1.0f / ssr_sqrt(((quat[0] * quat[0] + quat[1] * quat[1]) + quat[2] * quat[2]) + quat[3] * quat[3]);
#pragma unroll
    for (int i = 0; i < 4; i++) p.qn[i] = quat[i] * p.qinv;
#pragma unroll
    for (int i = 0; i < 3; i++) p.s[i] = ssr_exp(ls[i]);
    {
        const float w = p.qn[0], qx = p.qn[1], qy = p.qn[2], qz = p.qn[3];
        const float x2 = qx * qx, y2 = qy * qy, z2 = qz * qz;
        const float xy = qx * qy, xz = qx * qz, yz = qy * qz;
        const float wx = w * qx, wy = w * qy, wz = w * qz;
        p.Rq[0][0] = 1.f - 2.f * (y2 + z2); p.Rq[0][1] = 2.f * (xy - wz); p.Rq[0][2] = 2.f * (xz + wy);
        p.Rq[1][0] = 2.f * (xy + wz); p.Rq[1][1] = 1.f - 2.f * (x2 + z2); p.Rq[1][2] = 2.f * (yz - wx);
        p.Rq[2][0] = 2.f * (xz - wy); p.Rq[2][1] = 2.f * (yz + wx); p.Rq[2][2] = 1.f - 2.f * (x2 + y2);
    }
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++) p.M[i][j] = p.Rq[i][j] * p.s[j];
    float cov[3][3], tmp[3][3];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            cov[i][j] = (p.M[i][0] * p.M[j][0] + p.M[i][1] * p.M[j][1]) + p.M[i][2] * p.M[j][2];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            tmp[i][j] = (cam.R[i][0] * cov[0][j] + cam.R[i][1] * cov[1][j]) + cam.R[i][2] * cov[2][j];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            p.covc[i][j] = (tmp[i][0] * cam.R[j][0] + tmp[i][1] * cam.R[j][1]) + tmp[i][2] * cam.R[j][2];

    float (*J)[3] = p.J;
    p.clamp_lo[0] = p.clamp_lo[1] = p.clamp_hi[0] = p.clamp_hi[1] = false;
    if (kLens) {
        // *_proj<D, assume_valid> and *_proj_jac<D>: uv and its Jacobian from one first-order evaluation
        typedef SsrJet<3, 1> Jet;
        const Jet jx = ssr_jet_seed<3, 1>(x, 0), jy = ssr_jet_seed<3, 1>(y, 1), jz = ssr_jet_seed<3, 1>(z, 2);
        Jet u, v, du, dv;
        ssr_model_normalised<Jet>(cam.model, jx, jy, jz, u, v);
        if (!kAssumeValid && !ssr_distortion_valid(cam.tier, cam.dc, u.v, v.v)) return;
        ssr_distort<Jet>(cam.tier, cam.dc, u, v, du, dv);
        const Jet px = du * cam.fx + cam.cx, py = dv * cam.fy + cam.cy;
        p.xy[0] = px.v; p.xy[1] = py.v;
#pragma unroll
        for (int k = 0; k < 3; k++) { J[0][k] = px.d[k]; J[1][k] = py.d[k]; }
        if (cam.model == SSR_CAM_PINHOLE) clamp_pinhole_jacobian(cam, z, p);
    } else if (cam.model == SSR_CAM_PINHOLE) {
        const float z2 = z * z;
        p.xy[0] = cam.fx * (x / z) + cam.cx;
        p.xy[1] = cam.fy * (y / z) + cam.cy;
        J[0][0] = (z / z2) * cam.fx; J[0][1] = 0.0f; J[0][2] = ((0.0f - x) / z2) * cam.fx;
        J[1][0] = 0.0f; J[1][1] = (z / z2) * cam.fy; J[1][2] = ((0.0f - y) / z2) * cam.fy;
        clamp_pinhole_jacobian(cam, z, p);
    } else {
        const float h2 = x * x + z * z;
        const float h = ssr_sqrt(h2);
        const float r2 = h2 + y * y;
        p.xy[0] = cam.fx * ssr_atan2(x, z) + cam.cx;
        p.xy[1] = cam.fy * ssr_atan2(y, h) + cam.cy;
        const float hr2 = h * r2;
        J[0][0] = (z / h2) * cam.fx; J[0][1] = 0.0f; J[0][2] = ((0.0f - x) / h2) * cam.fx;
        J[1][0] = ((0.0f - x * y) / hr2) * cam.fy; J[1][1] = (h / r2) * cam.fy;
        J[1][2] = ((0.0f - z * y) / hr2) * cam.fy;
    }
    float jc[2][3];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            jc[i][j] = (J[i][0] * p.covc[0][j] + J[i][1] * p.covc[1][j]) + J[i][2] * p.covc[2][j];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
            p.c2[i][j] = (jc[i][0] * J[j][0] + jc[i][1] * J[j][1]) + jc[i][2] * J[j][2];
    if (kLens && !kAssumeValid && (cam.model == SSR_CAM_FISHEYE || cam.model == SSR_CAM_EQUISOLID)) {
        // a splat behind a wide lens that still reaches the image centre with visible opacity is dropped,
        // src/shaders/primitive_3dgs.slang:509-514 (before the blur is added)
        const float m0 = p.xy[0] - cam.cx, m1 = p.xy[1] - cam.cy;
        const float idet = 1.0f / (p.c2[0][0] * p.c2[1][1] - p.c2[0][1] * p.c2[1][0]);
        const float i00 = p.c2[1][1] * idet, i01 = (-p.c2[0][1]) * idet, i10 = (-p.c2[1][0]) * idet, i11 = p.c2[0][0] * idet;
        const float q = (i00 * m0 + i01 * m1) * m0 + (i10 * m0 + i11 * m1) * m1;
        const float seen = p.opac * ssr_exp(-0.5f * q);
        if (z < 0.0f && seen > kAlphaThreshold) return;
    }
    // add_blur (src/shaders/primitive_3dgs.slang:398-405,528-543): the antialiased variant blurs less and scales
    // the opacity by sqrt(det before / det after)
    const float eps2d = cam.aa ? 0.1f : 0.3f;
    p.det_orig = p.c2[0][0] * p.c2[1][1] - p.c2[0][1] * p.c2[1][0];
    p.c2o[0] = p.c2[0][0]; p.c2o[1] = p.c2[1][1];
    p.c2[0][0] = p.c2[0][0] + eps2d;
    p.c2[1][1] = p.c2[1][1] + eps2d;
    const float det = p.c2[0][0] * p.c2[1][1] - p.c2[0][1] * p.c2[1][0];
    p.det_blur = det;
    if (!kAssumeValid && det <= 0.f) return;
    p.sig = p.opac; p.comp = 1.0f;
    if (cam.aa) {
        p.comp = ssr_sqrt(ssr_max(0.0f, p.det_orig / det));
        p.opac = p.opac * p.comp;
    }
    const float invdet = 1.0f / det;
    p.conic[0] = p.c2[1][1] * invdet;
    p.conic[1] = (-p.c2[0][1]) * invdet;
    p.conic[2] = p.c2[0][0] * invdet;
    if (kAssumeValid) { p.valid = true; return; }   // the VJP needs nothing below
    if (p.opac < kAlphaThreshold) return;
    const float extend = ssr_min(3.33f, ssr_sqrt(2.0f * ssr_log(p.opac / kAlphaThreshold)));
    const float rx = extend * ssr_sqrt(p.c2[0][0]);
    const float ry = extend * ssr_sqrt(p.c2[1][1]);
    const float xmin = p.xy[0] - rx, xmax = p.xy[0] + rx, ymin = p.xy[1] - ry, ymax = p.xy[1] + ry;
    if (xmax <= 0 || xmin >= cam.Wf || ymax <= 0 || ymin >= cam.Hf) return;
    p.aabb[0] = xmin; p.aabb[1] = ymin; p.aabb[2] = xmax; p.aabb[3] = ymax;
    // get_sorting_depth, src/shaders/projection_utils.slang:1012-1029
    if (cam.model == SSR_CAM_PINHOLE) p.sort_depth = z;
    else if (cam.model == SSR_CAM_EQUIRECT) p.sort_depth = dot3(p.mc, p.mc);
    else p.sort_depth = ((z * z) * z) * z + ((1.0f / 512.0f) * (x * x + y * y)) * (x * x + y * y);
    float campos[3];
#pragma unroll
    for (int i = 0; i < 3; i++)
        campos[i] = -((cam.R[0][i] * cam.t[0] + cam.R[1][i] * cam.t[1]) + cam.R[2][i] * cam.t[2]);
    p.radius = view_radius(mean, ls, logit, campos);
    p.valid = true;
}

// ---- SH ----------------------------------------------------------------------------------

__device__ __forceinline__ float half_bits_to_float(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);   // exact widening conversion
}

// Decodes the 3*n_coef higher-order coefficients of splat `gid` into registers.
// REF codecs: src/shaders/harmonics.slang:114-140.
template <int kCoef>
__device__ __forceinline__ void decode_sh(const ssr_world& w, const ssr_sh_quant& q, int64_t gid,
                                          float* __restrict__ out) {
    constexpr int n = 3 * kCoef;
    if (q.codec == SSR_SH_F32) {
        const float* p = w.features_sh + gid * (int64_t)w.sh_stride;
#pragma unroll
        for (int i = 0; i < n; i++) out[i] = p[i];
    } else if (q.codec == SSR_SH_I8_F16SCALE) {
        const int8_t* p = reinterpret_cast<const int8_t*>(q.packed) + gid * 45;
        const float s = half_bits_to_float(q.scale_f16[gid]);
#pragma unroll
        for (int i = 0; i < n; i++) out[i] = (float)p[i] * s;
    } else {
        const int64_t base = (int64_t)3 * (int64_t)q.num_sh_buffer * gid;
        const int64_t stride = q.bounds_stride > 0 ? q.bounds_stride
                                                   : (int64_t)256 * 3 * (int64_t)q.num_sh_buffer;
        const bool q16 = q.codec == SSR_SH_REF_Q16;
        const float inv = q16 ? (1.0f / 65535.0f) : (1.0f / 255.0f);
        // one bound per 256 splats is the layout the optimizer keeps: the splat's cells then share a block,
        // and the block is gid / 256 (no 64-bit division, no per-cell test)
        if (stride == (int64_t)256 * 3 * (int64_t)q.num_sh_buffer) {
            const int64_t blk = gid >> 8;
            const float lo = q.bounds[2 * blk], hi = q.bounds[2 * blk + 1];
            if (q16 && n > 1 && (reinterpret_cast<uintptr_t>(q.packed) & 3) == 0) {
                // 16-bit codes through aligned 32-bit loads (half as many memory instructions): the splat's first
                // code sits in the low or the high half of its first word, by the parity of `base`
                const uint16_t* p16 = reinterpret_cast<const uint16_t*>(q.packed) + base;
                const bool odd = (base & 1) != 0;
                const uint32_t* p32 = reinterpret_cast<const uint32_t*>(p16 - (odd ? 1 : 0));
                constexpr int kWords = (n + 1) / 2 + ((n & 1) ? 0 : 1);   // words touched when the run starts in a high half
                uint32_t w[kWords];
#pragma unroll
                for (int k = 0; k < kWords - 1; k++) w[k] = p32[k];
                // the last word is only partly this splat's: take it whole when the run reaches into its high half,
                // else just the one code (the bytes after it may lie beyond the array)
                {
                    constexpr int kLast = kWords - 1;
                    // odd start: the run is halves 1..n of these words; even start: halves 0..n-1
                    const bool need = odd ? (2 * kLast <= n) : (2 * kLast <= n - 1);
                    const bool whole = odd ? (2 * kLast + 1 <= n) : (2 * kLast + 1 <= n - 1);
                    w[kLast] = 0u;
                    if (need) w[kLast] = whole ? p32[kLast] : (uint32_t)reinterpret_cast<const uint16_t*>(p32)[2 * kLast];
                }
#pragma unroll
                for (int i = 0; i < n; i++) {
                    const uint32_t even_code = (w[i >> 1] >> (16 * (i & 1))) & 0xffffu;
                    const uint32_t odd_code = (w[(i + 1) >> 1] >> (16 * ((i + 1) & 1))) & 0xffffu;
                    out[i] = lo + (hi - lo) * ((float)(odd ? odd_code : even_code) * inv);
                }
                return;
            }
#pragma unroll
            for (int i = 0; i < n; i++) {
                const float v = q16 ? (float)reinterpret_cast<const uint16_t*>(q.packed)[base + i]
                                    : (float)reinterpret_cast<const uint8_t*>(q.packed)[base + i];
                out[i] = lo + (hi - lo) * (v * inv);
            }
            return;
        }
        // otherwise bounds change at most once every `stride` cells: track the current block incrementally
        // (cells advance by one and `stride` is at least one, so a cell that reaches `next` is exactly `next`
        // and its block is the following one: one division for the splat, none per cell)
        int64_t blk = base / stride;
        int64_t next = (blk + 1) * stride;
        float lo = q.bounds[2 * blk], hi = q.bounds[2 * blk + 1];
#pragma unroll
        for (int i = 0; i < n; i++) {
            const int64_t cell = base + i;
            if (cell >= next) {
                blk += 1; next += stride;
                lo = q.bounds[2 * blk]; hi = q.bounds[2 * blk + 1];
            }
            const float v = q16 ? (float)reinterpret_cast<const uint16_t*>(q.packed)[cell]
                                : (float)reinterpret_cast<const uint8_t*>(q.packed)[cell];
            out[i] = lo + (hi - lo) * (v * inv);
        }
    }
}

// Real spherical harmonics of bands 1..3 in the product form
//   Y(l, +m) = A_lm(z) Re (x + i y)^m,   Y(l, -m) = A_lm(z) Im (x + i y)^m,   Y(l, 0) = B_l(z),
// with the sign and ordering convention of src/shaders/harmonics.slang:172-217 (index j runs -l..l
// inside band l). The colour feeds bit-exact tile keys downstream, so each Y_j is formed by the
// operations the oracle uses; (x + i y)^m comes from the complex-power recurrence (x y + y x is
// exactly 2 x y). The direction gradient in projection_vjp differentiates the same product form.
struct ShBasisD {
    float Y[15];
    float x, y, z, inorm;
    float re[4], im[4];   // Re / Im (x + i y)^m, m = 0..3
};

namespace shk {   // normalisation constants of the product form
constexpr float k1 = 0.48860251190292f;
constexpr float k20a = 0.9461746957575601f, k20b = 0.3153915652525201f, k21 = 1.092548430592079f, k22 = 0.5462742152960395f;
constexpr float k30a = 1.865881662950577f, k30b = 1.119528997770346f, k31a = 2.285228997322329f, k31b = 0.4570457994644658f,
                k32 = 1.445305721320277f, k33 = 0.5900435899266435f;
}  // namespace shk

template <int kDegree>
__device__ __forceinline__ void sh_basis(const float dir[3], ShBasisD& b) {
#pragma unroll
    for (int i = 0; i < 15; i++) b.Y[i] = 0.0f;
    b.inorm = 1.0f / ssr_sqrt((dir[0] * dir[0] + dir[1] * dir[1]) + dir[2] * dir[2]);
    const float x = dir[0] * b.inorm, y = dir[1] * b.inorm, z = dir[2] * b.inorm;
    b.x = x; b.y = y; b.z = z;
    b.re[0] = 1.0f; b.im[0] = 0.0f; b.re[1] = x; b.im[1] = y;
#pragma unroll
    for (int m = 1; m < 3; m++) {
        b.re[m + 1] = x * b.re[m] - y * b.im[m];
        b.im[m + 1] = x * b.im[m] + y * b.re[m];
    }
    if (kDegree < 1) return;
    b.Y[0] = -shk::k1 * b.im[1];
    b.Y[1] = shk::k1 * z;
    b.Y[2] = -shk::k1 * b.re[1];
    if (kDegree < 2) return;
    const float zz = z * z;
    const float a21 = -shk::k21 * z;
    b.Y[3] = shk::k22 * b.im[2];
    b.Y[4] = a21 * b.im[1];
    b.Y[5] = shk::k20a * zz - shk::k20b;
    b.Y[6] = a21 * b.re[1];
    b.Y[7] = shk::k22 * b.re[2];
    if (kDegree < 3) return;
    const float a31 = -shk::k31a * zz + shk::k31b;
    const float a32 = shk::k32 * z;
    b.Y[8] = -shk::k33 * b.im[3];
    b.Y[9] = a32 * b.im[2];
    b.Y[10] = a31 * b.im[1];
    b.Y[11] = z * (shk::k30a * zz - shk::k30b);
    b.Y[12] = a31 * b.re[1];
    b.Y[13] = a32 * b.re[2];
    b.Y[14] = -shk::k33 * b.re[3];
}

// colour before the +0.5 shift (src/shaders/harmonics.slang:154-223)
template <int kDegree>
__device__ __forceinline__ void sh_color_raw(const ShBasisD& b, const float dc[3], const float* c,
                                             float out[3]) {
#pragma unroll
    for (int ch = 0; ch < 3; ch++) {
        float col = 0.2820947917738781f * dc[ch];
        if (kDegree >= 1) {
            col = col + 0.48860251190292f *
                            (((-b.y) * c[0 * 3 + ch] + b.z * c[1 * 3 + ch]) - b.x * c[2 * 3 + ch]);
        }
        if (kDegree >= 2) {
            float s = b.Y[3] * c[3 * 3 + ch] + b.Y[4] * c[4 * 3 + ch];
            s = s + b.Y[5] * c[5 * 3 + ch];
            s = s + b.Y[6] * c[6 * 3 + ch];
            s = s + b.Y[7] * c[7 * 3 + ch];
            col = col + s;
        }
        if (kDegree >= 3) {
            float s = b.Y[8] * c[8 * 3 + ch] + b.Y[9] * c[9 * 3 + ch];
#pragma unroll
            for (int j = 10; j < 15; j++) s = s + b.Y[j] * c[j * 3 + ch];
            col = col + s;
        }
        out[ch] = col;
    }
}

__device__ __forceinline__ void view_dir(const CamD& cam, const float m[3], float dir[3]) {
    // mean + R^T t (src/shaders/harmonics.slang:145-149)
#pragma unroll
    for (int i = 0; i < 3; i++)
        dir[i] = m[i] + ((cam.R[0][i] * cam.t[0] + cam.R[1][i] * cam.t[1]) + cam.R[2][i] * cam.t[2]);
}

// ---- tile geometry (shared by K1's fused count, K2 and K4) ---------------------------------

// src/kernels/tile/IntersectTile.cu:34-53
__device__ __forceinline__ void ellipse_range_bound(const float ic[3], float y0, float y1, float out[2]) {
    const float a = ic[0], b = ic[1], c = ic[2];
    const float ym = ((-b) / c) * ssr_sqrt(c / (a * c - b * b));
    const float v0 = ssr_min(ssr_max(-ym, y0), y1);
    const float v1 = ssr_min(ssr_max(ym, y0), y1);
    const float bv0 = (-b) * v0, bv1 = (-b) * v1;
    const float inv_a = 1.0f / a;
    out[0] = inv_a * (bv0 - ssr_sqrt(bv0 * bv0 - a * ((c * v0) * v0 - 1.f)));
    out[1] = inv_a * (bv1 + ssr_sqrt(bv1 * bv1 - a * ((c * v1) * v1 - 1.f)));
}

__device__ __forceinline__ int clampi(int x, int a, int b) { return x < a ? a : (x > b ? b : x); }

struct TileGeomD {
    float xy[2];
    float ic[3];
    int xmin, xmax, ymin, ymax;
    bool by_rows;
};

// prologue of both tile passes (src/kernels/tile/IntersectTile.cu:124-164)
__device__ __forceinline__ void tile_geom(const float aabb[4], const float xy[2], const float conic[3],
                                          float opac, int tile_w, int tile_h, TileGeomD& g) {
    g.xy[0] = xy[0]; g.xy[1] = xy[1];
    const float k = 0.5f / ssr_log(opac / kAlphaThreshold);
#pragma unroll
    for (int i = 0; i < 3; i++) g.ic[i] = conic[i] * k;
    g.xmin = min(max(0, ssr_f2i_sat(ssr_floor((aabb[0] + 0.5f) / (float)kTile))), tile_w);
    g.ymin = min(max(0, ssr_f2i_sat(ssr_floor((aabb[1] + 0.5f) / (float)kTile))), tile_h);
    g.xmax = min(max(0, ssr_f2i_sat(ssr_ceil((aabb[2] + 0.5f) / (float)kTile))), tile_w);
    g.ymax = min(max(0, ssr_f2i_sat(ssr_ceil((aabb[3] + 0.5f) / (float)kTile))), tile_h);
    g.by_rows = (g.ymax - g.ymin) * kTile <= (g.xmax - g.xmin) * kTile;
}

// Tile interval [lo, hi) that the ellipse covers in one band: band index `r` is a tile row when
// g.by_rows (the interval is then over tile columns) and a tile column otherwise. Same arithmetic
// as the reference's count pass (IntersectTile.cu:55-101) and write pass (:198-247).
__device__ __forceinline__ void tile_band_interval(const TileGeomD& g, int r, int& lo, int& hi) {
    float bd[2];
    if (g.by_rows) {
        const float y0 = (float)(r * kTile) - g.xy[1];
        const float y1 = y0 + (float)kTile;
        ellipse_range_bound(g.ic, y0, y1, bd);
        lo = clampi(ssr_f2i_sat(ssr_floor((bd[0] + g.xy[0]) / (float)kTile)), g.xmin, g.xmax);
        hi = clampi(ssr_f2i_sat(ssr_ceil((bd[1] + g.xy[0]) / (float)kTile)), g.xmin, g.xmax);
    } else {
        const float sw[3] = {g.ic[2], g.ic[1], g.ic[0]};
        const float x0 = (float)(r * kTile) - g.xy[0];
        const float x1 = x0 + (float)kTile;
        ellipse_range_bound(sw, x0, x1, bd);
        lo = clampi(ssr_f2i_sat(ssr_floor((bd[0] + g.xy[1]) / (float)kTile)), g.ymin, g.ymax);
        hi = clampi(ssr_f2i_sat(ssr_ceil((bd[1] + g.xy[1]) / (float)kTile)), g.ymin, g.ymax);
    }
}

// Visits every band the ellipse touches in the reference's enumeration order: emit(lo, hi, band, by_rows).
template <class F>
__device__ __forceinline__ void for_each_tile(const TileGeomD& g, F&& emit) {
    const int b0 = g.by_rows ? g.ymin : g.xmin, b1 = g.by_rows ? g.ymax : g.xmax;
    for (int r = b0; r < b1; r++) {
        int lo, hi;
        tile_band_interval(g, r, lo, hi);
        emit(lo, hi, r, g.by_rows);
    }
}

__device__ __forceinline__ int64_t count_tiles(const TileGeomD& g) {
    int64_t n = 0;
    for_each_tile(g, [&](int lo, int hi, int, bool) { n += max(hi - lo, 0); });
    return n;
}

// Tile-skip map (src/kernels/tile/IntersectTile.cu:62,76-80,95-98,225): live[y * tile_w + x] == 0
// marks a tile that neither pass emits.
__device__ __forceinline__ bool tile_is_live(const int32_t* __restrict__ live, int tile_w, int fixed, int v, bool rows) {
    return live[rows ? ((int64_t)fixed * tile_w + v) : ((int64_t)v * tile_w + fixed)] != 0;
}

__device__ __forceinline__ int count_live(const int32_t* __restrict__ live, int tile_w, int lo, int hi, int fixed, bool rows) {
    int n = 0;
    for (int v = lo; v < hi; v++) n += tile_is_live(live, tile_w, fixed, v, rows) ? 1 : 0;
    return n;
}

__device__ __forceinline__ int64_t count_tiles_masked(const TileGeomD& g, const int32_t* __restrict__ live, int tile_w) {
    int64_t n = 0;
    for_each_tile(g, [&](int lo, int hi, int fixed, bool rows) { n += count_live(live, tile_w, lo, hi, fixed, rows); });
    return n;
}

}  // namespace ssr
