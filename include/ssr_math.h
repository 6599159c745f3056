// ssr_math.h -- transcendental functions with one defined bit pattern on host and device.
//
// Every function here is built from IEEE-754 binary32 add, subtract, multiply, divide, sqrt,
// fused multiply-add (explicit, never implicit) and integer bit manipulation only. All of these
// are correctly rounded on x86-64 (SSE/FMA) and on gfx950, so the same source compiled with
// `-ffp-contract=off` and no fast-math yields bit-identical results on the CPU and on the GPU.
// That is what lets tile keys (which depend on exp/log/atan2 through the projected extents) be
// compared bit for bit between a host restatement and the device kernels.
//
// The reference evaluates these through `__expf/__logf` under `--use_fast_math`
// (src/primitives/Primitive3DGS.cuh:257, src/kernels/tile/IntersectTile.cu:156,
// cmake/SsBackendCuda.cmake:96) on CUDA and through driver-defined exp/log on Vulkan, so its own
// bits differ between its two backends; the functions below are the definition used here.
//
// Polynomials: the single-precision Cephes minimax sets (expf, logf, atanf); each is within
// about 1-2 ulp of the correctly rounded result on the ranges the rasterizer uses.
#pragma once

#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define SSR_HD __host__ __device__ __forceinline__
#else
#define SSR_HD static inline
#endif

SSR_HD float ssr_fma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
SSR_HD float ssr_sqrt(float x) { return __builtin_sqrtf(x); }
SSR_HD float ssr_fabs(float x) { return __builtin_fabsf(x); }
SSR_HD float ssr_floor(float x) { return __builtin_floorf(x); }
SSR_HD float ssr_ceil(float x) { return __builtin_ceilf(x); }
SSR_HD float ssr_rint(float x) { return __builtin_rintf(x); }  // round-half-even, default mode

SSR_HD uint32_t ssr_f2u(float f) {
    uint32_t u;
#if defined(__HIP_DEVICE_COMPILE__)
    u = __float_as_uint(f);
#else
    memcpy(&u, &f, 4);
#endif
    return u;
}
SSR_HD float ssr_u2f(uint32_t u) {
    float f;
#if defined(__HIP_DEVICE_COMPILE__)
    f = __uint_as_float(u);
#else
    memcpy(&f, &u, 4);
#endif
    return f;
}

// fminf/fmaxf semantics the reference relies on (a NaN operand is ignored), written as
// compare-and-select so that the choice between +0 and -0 is the same on host and device.
SSR_HD float ssr_min(float a, float b) { return (a != a) ? b : ((b < a) ? b : a); }
SSR_HD float ssr_max(float a, float b) { return (a != a) ? b : ((b > a) ? b : a); }

SSR_HD bool ssr_isfinite(float x) { return (ssr_f2u(x) & 0x7f800000u) != 0x7f800000u; }

// 2^k for integer k in [-126, 127] by writing the exponent field.
SSR_HD float ssr_pow2i(int k) { return ssr_u2f((uint32_t)(k + 127) << 23); }

// exp(x). x < -87.3 returns 0 (no subnormal outputs); x > 88.72 gives +inf.
SSR_HD float ssr_exp(float x) {
    if (!(x == x)) return x;                   // NaN
    if (x > 88.72283905206835f) return ssr_u2f(0x7f800000u);
    if (x < -87.3f) return 0.0f;               // keeps every non-zero result a normal number
    float k = ssr_rint(x * 1.44269504088896341f);
    float r = ssr_fma(k, -0.693359375f, x);     // Cody-Waite, high part exact for |k| < 2^15
    r = ssr_fma(k, 2.12194440e-4f, r);
    float z = r * r;
    float p = 1.9875691500e-4f;
    p = ssr_fma(p, r, 1.3981999507e-3f);
    p = ssr_fma(p, r, 8.3334519073e-3f);
    p = ssr_fma(p, r, 4.1665795894e-2f);
    p = ssr_fma(p, r, 1.6666665459e-1f);
    p = ssr_fma(p, r, 5.0000001201e-1f);
    float y = ssr_fma(p, z, r) + 1.0f;
    int ki = (int)k;                            // |k| <= 128
    // split the scaling so that both factors are normal numbers
    int k1 = ki / 2, k2 = ki - k1;
    return (y * ssr_pow2i(k1)) * ssr_pow2i(k2);
}

// log of a normal positive finite number whose bits are u, with e added to the exponent
SSR_HD float ssr_log_core(uint32_t u, int e) {
    e += (int)(u >> 23) - 126;                  // x = m * 2^e, m in [0.5, 1)
    float m = ssr_u2f((u & 0x007fffffu) | 0x3f000000u);
    if (m < 0.707106781186547524f) {
        e -= 1;
        m = (m + m) - 1.0f;
    } else {
        m = m - 1.0f;
    }
    float z = m * m;
    float p = 7.0376836292e-2f;
    p = ssr_fma(p, m, -1.1514610310e-1f);
    p = ssr_fma(p, m, 1.1676998740e-1f);
    p = ssr_fma(p, m, -1.2420140846e-1f);
    p = ssr_fma(p, m, 1.4249322787e-1f);
    p = ssr_fma(p, m, -1.6668057665e-1f);
    p = ssr_fma(p, m, 2.0000714765e-1f);
    p = ssr_fma(p, m, -2.4999993993e-1f);
    p = ssr_fma(p, m, 3.3333331174e-1f);
    float y = (p * m) * z;
    float fe = (float)e;
    y = ssr_fma(fe, -2.12194440e-4f, y);
    y = ssr_fma(z, -0.5f, y);
    float r = m + y;
    r = ssr_fma(fe, 0.693359375f, r);
    return r;
}

// natural log. log(0) = -inf, log(x<0) = NaN, log(inf) = inf; subnormal inputs are handled.
SSR_HD float ssr_log(float x) {
    if (!(x == x)) return x;
    if (x < 0.0f) return ssr_u2f(0x7fc00000u);
    if (x == 0.0f) return ssr_u2f(0xff800000u);
    uint32_t u = ssr_f2u(x);
    if (u == 0x7f800000u) return x;
    int e = 0;
    if (u < 0x00800000u) {                      // subnormal: scale by 2^23 (exact)
        x = x * 8388608.0f;
        u = ssr_f2u(x);
        e = -23;
    }
    return ssr_log_core(u, e);
}

// ssr_log for x >= 1 (or NaN): the same value with the tests for zero, negative and subnormal inputs left out
SSR_HD float ssr_log_ge1(float x) {
    if (!(x < 3.0e38f)) return ssr_log(x);      // infinity, NaN and the last binade take the general path
    return ssr_log_core(ssr_f2u(x), 0);
}

// atan(x) for finite x, result in (-pi/2, pi/2).
SSR_HD float ssr_atan(float x) {
    float ax = ssr_fabs(x);
    float y0, t;
    if (ax > 2.414213562373095f) {              // tan(3 pi / 8)
        y0 = 1.5707963267948966f;
        t = -(1.0f / ax);
    } else if (ax > 0.4142135623730950f) {      // tan(pi / 8)
        y0 = 0.7853981633974483f;
        t = (ax - 1.0f) / (ax + 1.0f);
    } else {
        y0 = 0.0f;
        t = ax;
    }
    float z = t * t;
    float p = 8.05374449538e-2f;
    p = ssr_fma(p, z, -1.38776856032e-1f);
    p = ssr_fma(p, z, 1.99777106478e-1f);
    p = ssr_fma(p, z, -3.33329491539e-1f);
    float r = ssr_fma(p * z, t, t);
    r = y0 + r;
    return (ssr_f2u(x) >> 31) ? -r : r;
}

// atan2(y, x) with the usual quadrant convention; atan2(0, 0) = 0.
SSR_HD float ssr_atan2(float y, float x) {
    if (!(x == x) || !(y == y)) return x + y;
    const float kPi = 3.14159265358979323846f;
    if (x == 0.0f) {
        if (y > 0.0f) return 1.5707963267948966f;
        if (y < 0.0f) return -1.5707963267948966f;
        return 0.0f;
    }
    float a = ssr_atan(y / x);
    if (x < 0.0f) a = (y >= 0.0f) ? (a + kPi) : (a - kPi);
    return a;
}

SSR_HD float ssr_sigmoid(float x) { return 1.0f / (1.0f + ssr_exp(-x)); }

// Adam's inverse bias corrections 1 / (1 - beta^t) for beta1 = 0.9f and beta2 = 0.999f, evaluated as the
// reference does in float (src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:369-370:
// 1.0f / (1.0f - powf(beta, step)), beta being the FLOAT constant: 0.999f is 0.99900001287..., and
// ln 0.999f differs from ln 0.999 by 1.3e-5 relative, which would scale every step at small t).
// beta^t = exp(t ln beta) with ln beta split into two floats, so that the product keeps its low bits:
// within about 1.5 ulp of the power, the accuracy class of a device powf.
SSR_HD float ssr_pow_split(float t, float ln_hi, float ln_lo) {
    const float x = t * ln_hi;
    const float rest = ssr_fma(t, ln_hi, -x) + t * ln_lo;   // t ln beta - x
    const float e = ssr_exp(x);
    return ssr_fma(e, rest, e);                              // e^x (1 + rest)
}
SSR_HD float ssr_adam_inv_bias1(float t) { return 1.0f / (1.0f - ssr_pow_split(t, -0.10536054521799088f, 3.0692108854424305e-09f)); }
SSR_HD float ssr_adam_inv_bias2(float t) { return 1.0f / (1.0f - ssr_pow_split(t, -0.0010004874784499407f, 3.235708576077023e-11f)); }

// float -> int32 / uint32 conversions with saturating, NaN -> 0 semantics. The reference casts
// floor()/ceil() results that can be NaN or negative (src/kernels/tile/IntersectTile.cu:72-75,
// 208-213); CUDA's conversion saturates while the C cast is undefined there, so the behaviour is
// pinned here.
SSR_HD int32_t ssr_f2i_sat(float x) {
    if (!(x == x)) return 0;
    if (x >= 2147483648.0f) return 2147483647;
    if (x <= -2147483648.0f) return (int32_t)0x80000000;
    return (int32_t)x;
}
SSR_HD uint32_t ssr_f2u_sat(float x) {
    if (!(x == x)) return 0u;
    if (x >= 4294967296.0f) return 0xffffffffu;
    if (x <= 0.0f) return 0u;
    return (uint32_t)x;
}
