// ssr_colour.h -- the colour maps the fused optimizer's colour trust region steps through, one definition for
// the host restatement and the device kernels (src/shaders/pixel_wise.slang:60-115).
#pragma once

#include "ssr_math.h"

// d/dx of the sRGB transfer curve linear_rgb_to_srgb(x) = x < 0.0031308 ? 12.92 x : 1.055 x^(1/2.4) - 0.055
// (linear_rgb_to_srgb_grad: forward-mode derivative of that expression; the power through exp / log)
SSR_HD float ssr_srgb_slope(float x) {
    if (x < 0.0031308f) return 12.92f;
    return (1.055f * (1.0f / 2.4f)) * ssr_exp((1.0f / 2.4f - 1.0f) * ssr_log(x));
}

// splat_dc_encode / splat_dc_decode: the DC coefficient <-> an affine map of sqrt(colour) with slope 1 at colour
// 0.5, continued linearly below colour 0; a = 1/255 is the square root of the black floor
SSR_HD float ssr_splat_dc_encode(float dc) {
    const float kSh0 = 0.28209479177387814f, a = 1.0f / 255.0f;
    const float s = ssr_sqrt(0.5f + a * a);
    const float u = kSh0 * dc + 0.5f;
    const float w = u >= 0.0f ? 2.0f * ssr_sqrt(u + a * a) : 2.0f * a + u / a;
    return ((w - 2.0f * s) * s) / kSh0;
}
SSR_HD float ssr_splat_dc_decode(float x) {
    const float kSh0 = 0.28209479177387814f, a = 1.0f / 255.0f;
    const float s = ssr_sqrt(0.5f + a * a);
    const float w = (x * kSh0) / s + 2.0f * s;
    const float u = w >= 2.0f * a ? (0.25f * w) * w - a * a : (w - 2.0f * a) * a;
    return (u - 0.5f) / kSh0;
}
