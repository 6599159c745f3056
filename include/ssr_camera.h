// ssr_camera.h -- camera models and lens-distortion tiers, with their first and second derivatives,
// in one definition shared by the host restatement and the device kernels.
//
// The reference defines each model as a differentiable function p_view -> uv
// (src/shaders/projection_utils.slang: persp_proj_uv :331-341, fisheye_proj :379-384 / _uv :400-410,
// equisolid_proj :388-395 / _uv :432-442, the distortion tiers :235-295), takes its 2x3 Jacobian
// with forward-mode differentiation (persp/fisheye/equisolid_proj_jac, :362-375, :463-493) and lets
// the compiler differentiate that Jacobian again for the backward pass. The same is done here with
// truncated Taylor arithmetic ("jets"): a value, its gradient with respect to N seeds and, for the
// backward pass, its symmetric Hessian. One templated statement of each model serves the forward
// (order 1: uv and J) and the backward (order 2: also dJ/dp).
//
// Only IEEE add, subtract, multiply, divide, sqrt and the functions of ssr_math.h are used, so with
// contraction off the host and the device produce the same bits.
#pragma once

#include "ssr_math.h"

#if defined(__HIPCC__)
#define SSR_UNROLL _Pragma("unroll")
#else
#define SSR_UNROLL
#endif

enum { SSR_MODEL_PINHOLE = 0, SSR_MODEL_FISHEYE = 1, SSR_MODEL_EQUISOLID = 2, SSR_MODEL_EQUIRECT = 3 };
// CameraDistortionType, src/shaders/projection_utils.slang:220-225 (coefficient order per tier: :242-295)
enum { SSR_TIER_NONE = 0, SSR_TIER_OPENCV = 1, SSR_TIER_THIN_PRISM = 2, SSR_TIER_RATIONAL = 3 };

// The (model, tier) pairs the reference instantiates (src/kernels/projection/CameraVariants.cuh:11-22).
SSR_HD bool ssr_camera_variant_supported(int model, int tier) {
    if (model == SSR_MODEL_PINHOLE) return tier >= SSR_TIER_NONE && tier <= SSR_TIER_RATIONAL;
    if (model == SSR_MODEL_FISHEYE || model == SSR_MODEL_EQUISOLID) return tier >= SSR_TIER_NONE && tier <= SSR_TIER_THIN_PRISM;
    return model == SSR_MODEL_EQUIRECT && tier == SSR_TIER_NONE;
}

// sin and cos on [0, pi/2] (single-precision Cephes polynomials on [0, pi/4], the upper half by
// reflection about pi/4).
SSR_HD void ssr_sincos_quarter(float x, float* s, float* c) {
    const float kHalfPi = 1.57079632679489661923f;
    const bool flip = x > 0.78539816339744830962f;
    const float y = flip ? kHalfPi - x : x;
    const float z = y * y;
    float ps = -1.9515295891e-4f;
    ps = ssr_fma(ps, z, 8.3321608736e-3f);
    ps = ssr_fma(ps, z, -1.6666654611e-1f);
    const float sy = ssr_fma(ps * z, y, y);
    float pc = 2.443315711809948e-5f;
    pc = ssr_fma(pc, z, -1.388731625493765e-3f);
    pc = ssr_fma(pc, z, 4.166664568298827e-2f);
    const float cy = ssr_fma(pc * z, z, ssr_fma(-0.5f, z, 1.0f));
    *s = flip ? cy : sy;
    *c = flip ? sy : cy;
}

// ---- jets ---------------------------------------------------------------------------------------
// v, d[j] = dv/ds_j, h[idx(j,k)] = d2v/ds_j ds_k for j <= k (kOrder == 2 only).
template <int N, int kOrder>
struct SsrJet {
    static constexpr int kH = kOrder == 2 ? N * (N + 1) / 2 : 1;
    float v;
    float d[N];
    float h[kH];
};

template <int N>
SSR_HD constexpr int ssr_jet_idx(int j, int k) { return j * N - j * (j - 1) / 2 + (k - j); }   // j <= k

template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_const(float c) {
    SsrJet<N, O> r;
    r.v = c;
    SSR_UNROLL
    for (int j = 0; j < N; j++) r.d[j] = 0.0f;
    SSR_UNROLL
    for (int j = 0; j < SsrJet<N, O>::kH; j++) r.h[j] = 0.0f;
    return r;
}
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_seed(float value, int which) {
    SsrJet<N, O> r = ssr_jet_const<N, O>(value);
    r.d[which] = 1.0f;
    return r;
}

template <int N, int O>
SSR_HD SsrJet<N, O> operator+(const SsrJet<N, O>& a, const SsrJet<N, O>& b) {
    SsrJet<N, O> r;
    r.v = a.v + b.v;
    SSR_UNROLL
    for (int j = 0; j < N; j++) r.d[j] = a.d[j] + b.d[j];
    SSR_UNROLL
    for (int j = 0; j < SsrJet<N, O>::kH; j++) r.h[j] = a.h[j] + b.h[j];
    return r;
}
template <int N, int O>
SSR_HD SsrJet<N, O> operator+(const SsrJet<N, O>& a, float c) { SsrJet<N, O> r = a; r.v = a.v + c; return r; }
template <int N, int O>
SSR_HD SsrJet<N, O> operator*(const SsrJet<N, O>& a, float c) {
    SsrJet<N, O> r;
    r.v = a.v * c;
    SSR_UNROLL
    for (int j = 0; j < N; j++) r.d[j] = a.d[j] * c;
    SSR_UNROLL
    for (int j = 0; j < SsrJet<N, O>::kH; j++) r.h[j] = a.h[j] * c;
    return r;
}
template <int N, int O>
SSR_HD SsrJet<N, O> operator*(const SsrJet<N, O>& a, const SsrJet<N, O>& b) {
    SsrJet<N, O> r;
    r.v = a.v * b.v;
    SSR_UNROLL
    for (int j = 0; j < N; j++) r.d[j] = a.v * b.d[j] + b.v * a.d[j];
    if (O == 2) {
        SSR_UNROLL
        for (int j = 0; j < N; j++)
            SSR_UNROLL
            for (int k = j; k < N; k++) {
                const int i = ssr_jet_idx<N>(j, k);
                r.h[i] = (a.v * b.h[i] + b.v * a.h[i]) + (a.d[j] * b.d[k] + a.d[k] * b.d[j]);
            }
    } else {
        r.h[0] = 0.0f;
    }
    return r;
}
// f(a) for a scalar function with first and second derivative f1, f2 at a.v
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_apply(const SsrJet<N, O>& a, float f, float f1, float f2) {
    SsrJet<N, O> r;
    r.v = f;
    SSR_UNROLL
    for (int j = 0; j < N; j++) r.d[j] = f1 * a.d[j];
    if (O == 2) {
        SSR_UNROLL
        for (int j = 0; j < N; j++)
            SSR_UNROLL
            for (int k = j; k < N; k++) {
                const int i = ssr_jet_idx<N>(j, k);
                r.h[i] = f1 * a.h[i] + f2 * (a.d[j] * a.d[k]);
            }
    } else {
        r.h[0] = 0.0f;
    }
    return r;
}
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_recip(const SsrJet<N, O>& a) {
    const float f = 1.0f / a.v;
    const float f1 = -(f * f);
    return ssr_jet_apply(a, f, f1, -2.0f * (f1 * f));
}
template <int N, int O>
SSR_HD SsrJet<N, O> operator/(const SsrJet<N, O>& a, const SsrJet<N, O>& b) { return a * ssr_jet_recip(b); }
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_sqrt(const SsrJet<N, O>& a) {
    // the derivative is guarded as the reference's differentiated sqrt is: 0.5 / sqrt(max(1e-7, x))
    // (src/generated/projection_utils.cuh:366-370), which keeps the on-axis Jacobians finite
    const float f = ssr_sqrt(a.v);
    const float m = ssr_max(1e-7f, a.v);
    const float f1 = 0.5f / ssr_sqrt(m);
    return ssr_jet_apply(a, f, f1, a.v > 1e-7f ? -0.5f * (f1 / m) : 0.0f);
}
template <int N, int O>
SSR_HD SsrJet<N, O> operator-(const SsrJet<N, O>& a, const SsrJet<N, O>& b) { return a + b * -1.0f; }
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_exp(const SsrJet<N, O>& a) {
    const float f = ssr_exp(a.v);
    return ssr_jet_apply(a, f, f, f);
}
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_log(const SsrJet<N, O>& a) {
    const float i = 1.0f / a.v;
    return ssr_jet_apply(a, ssr_log(a.v), i, -(i * i));
}
// max / min: the derivative follows the selected operand; on a tie each side takes half
// (the rule of the reference's differentiated max, src/generated/per_splat_losses.cuh:19-45)
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_max(const SsrJet<N, O>& a, const SsrJet<N, O>& b) {
    if (a.v > b.v) return a;
    if (a.v < b.v) return b;
    return (a + b) * 0.5f;
}
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_min(const SsrJet<N, O>& a, const SsrJet<N, O>& b) {
    if (a.v < b.v) return a;
    if (a.v > b.v) return b;
    return (a + b) * 0.5f;
}
// atan2(y, x)
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_atan2(const SsrJet<N, O>& y, const SsrJet<N, O>& x) {
    SsrJet<N, O> r;
    r.v = ssr_atan2(y.v, x.v);
    const float r2 = x.v * x.v + y.v * y.v;
    const float fy = x.v / r2, fx = -(y.v / r2);
    SSR_UNROLL
    for (int j = 0; j < N; j++) r.d[j] = fy * y.d[j] + fx * x.d[j];
    if (O == 2) {
        const float r4 = r2 * r2;
        const float fxx = (2.0f * (x.v * y.v)) / r4, fyy = -fxx, fxy = (y.v * y.v - x.v * x.v) / r4;
        SSR_UNROLL
        for (int j = 0; j < N; j++)
            SSR_UNROLL
            for (int k = j; k < N; k++) {
                const int i = ssr_jet_idx<N>(j, k);
                r.h[i] = (fy * y.h[i] + fx * x.h[i]) +
                         ((fyy * (y.d[j] * y.d[k]) + fxx * (x.d[j] * x.d[k])) + fxy * (y.d[j] * x.d[k] + y.d[k] * x.d[j]));
            }
    } else {
        r.h[0] = 0.0f;
    }
    return r;
}
// sin(a) for a.v in [0, pi/2]
template <int N, int O>
SSR_HD SsrJet<N, O> ssr_jet_sin_quarter(const SsrJet<N, O>& a) {
    float s, c;
    ssr_sincos_quarter(a.v, &s, &c);
    return ssr_jet_apply(a, s, c, -s);
}

// ---- distortion tiers (src/shaders/projection_utils.slang:235-295) ---------------------------------
template <class T>
SSR_HD void ssr_distort(int tier, const float* c, const T& u, const T& v, T& ou, T& ov) {
    if (tier == SSR_TIER_NONE) { ou = u; ov = v; return; }
    // all eight read up front, so that the tier selects among values, not among addresses
    const float c0 = c[0], c1 = c[1], c2 = c[2], c3 = c[3], c4 = c[4], c5 = c[5], c6 = c[6], c7 = c[7];
    const T r2 = u * u + v * v;
    const T uv = u * v;
    T radial;
    float p1, p2, s1 = 0.0f, s2 = 0.0f;
    if (tier == SSR_TIER_OPENCV) {             // k1 k2 p1 p2
        radial = r2 * (r2 * c1 + c0) + 1.0f;
        p1 = c2; p2 = c3;
    } else if (tier == SSR_TIER_THIN_PRISM) {  // k1 k2 k3 k4 p1 p2 sx1 sy1
        radial = r2 * (r2 * (r2 * (r2 * c3 + c2) + c1) + c0) + 1.0f;
        p1 = c4; p2 = c5; s1 = c6; s2 = c7;
    } else {                                   // k1 k2 k3 k4 k5 k6 p1 p2; k4..k6 in the denominator
        const T num = r2 * (r2 * (r2 * c2 + c1) + c0) + 1.0f;
        const T den = r2 * (r2 * (r2 * c5 + c4) + c3) + 1.0f;
        radial = num / den;
        p1 = c6; p2 = c7;
    }
    T tx = uv * (2.0f * p1) + (r2 + (u * u) * 2.0f) * p2;
    T ty = uv * (2.0f * p2) + (r2 + (v * v) * 2.0f) * p1;
    if (tier == SSR_TIER_THIN_PRISM) { tx = tx + r2 * s1; ty = ty + r2 * s2; }
    ou = u * radial + tx;
    ov = v * radial + ty;
}

// is_valid_distortion, src/shaders/projection_utils.slang:310-321
SSR_HD bool ssr_distortion_valid(int tier, const float* c, float u, float v) {
    if (tier == SSR_TIER_NONE) return true;
    typedef SsrJet<2, 1> J2;
    J2 du, dv;
    ssr_distort<J2>(tier, c, ssr_jet_seed<2, 1>(u, 0), ssr_jet_seed<2, 1>(v, 1), du, dv);
    const float det = du.d[0] * dv.d[1] - du.d[1] * dv.d[0];
    const float jdet = ssr_min(det, ssr_min(du.d[0], dv.d[1]));
    return jdet > 0.25f && jdet < 4.0f && (u * du.v + v * dv.v) >= 0.0f;
}

// ---- camera models: p_view -> normalised coordinates before distortion -----------------------------
// PINHOLE (x/z, y/z); FISHEYE theta * (x, y)/r, :379-384; EQUISOLID 2 sin(theta/2) * (x, y)/r, :388-395
template <class T>
SSR_HD void ssr_model_normalised(int model, const T& x, const T& y, const T& z, T& u, T& v) {
    if (model == SSR_MODEL_PINHOLE) {
        u = x / z;
        v = y / z;
        return;
    }
    const T r = ssr_jet_sqrt(x * x + y * y);
    const T theta = ssr_jet_atan2(r, z);
    T k;
    if (model == SSR_MODEL_FISHEYE) {
        if (theta.v < 1e-3f) k = ((theta * theta) * (-1.0f / 3.0f) + 1.0f) / z;
        else k = theta / r;
    } else {
        if (r.v < 1e-6f) k = ((theta * theta) * (-1.0f / 24.0f) + 1.0f) / z;
        else k = (ssr_jet_sin_quarter(theta * 0.5f) * 2.0f) / r;
    }
    u = x * k;
    v = y * k;
}

// Pixel coordinates: model, then distortion, then the intrinsics (the *_proj_uv functions).
template <class T>
SSR_HD void ssr_model_pixel(int model, int tier, const float* coeffs, float fx, float fy, float cx, float cy, const T& x,
                            const T& y, const T& z, T& px, T& py) {
    T u, v, du, dv;
    ssr_model_normalised<T>(model, x, y, z, u, v);
    ssr_distort<T>(tier, coeffs, u, v, du, dv);
    px = du * fx + cx;
    py = dv * fy + cy;
}

// ---- effective-rank regularizer of the scales ------------------------------------------------------
// erank_reg_3dgs (src/shaders/per_splat_losses.slang:3-15): with s_i the normalised squared scales,
// reg = max(-log(exp(entropy(s)) - 0.99999), 0); loss = w * reg + w3 * s_min. Returns the loss, writes its
// gradient with respect to the three log-scales.
SSR_HD float ssr_erank_reg_grad(const float log_scales[3], float w, float w3, float grad[3]) {
    typedef SsrJet<3, 1> Jet;
    const Jet x = ssr_jet_exp(ssr_jet_seed<3, 1>(log_scales[0], 0) * 2.0f);
    const Jet y = ssr_jet_exp(ssr_jet_seed<3, 1>(log_scales[1], 1) * 2.0f);
    const Jet z = ssr_jet_exp(ssr_jet_seed<3, 1>(log_scales[2], 2) * 2.0f);
    const Jet s = (x + y) + z;
    const Jet s1 = ssr_jet_max(ssr_jet_max(x, y), z) / s;
    const Jet s3 = ssr_jet_min(ssr_jet_min(x, y), z) / s;
    const Jet s2 = (s1 * -1.0f + 1.0f) - s3;
    const Jet r = ssr_jet_exp(((s1 * ssr_jet_log(s1)) * -1.0f - s2 * ssr_jet_log(s2)) - s3 * ssr_jet_log(s3));
    const Jet reg = ssr_jet_max(ssr_jet_log(r + -0.99999f) * -1.0f, ssr_jet_const<3, 1>(0.0f));
    const Jet loss = reg * w + s3 * w3;
    grad[0] = loss.d[0]; grad[1] = loss.d[1]; grad[2] = loss.d[2];
    return loss.v;
}
