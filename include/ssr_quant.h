// ssr_quant.h -- the block-wise codecs of the quantized optimizer state, one definition for the host
// restatement and the device kernels.
//
// QuantizedAdamState<8, 256> and <16, 256> (src/core/Tensor.h:936-1133): per cell two codes (bytes, or
// 16-bit halves of a word), the linearly quantized u = g1 / (sqrt(g2) + eps) and
// log_s = log1p(sqrt(g2) / eps), against per-block bounds (u_min, u_max, log_s_min, log_s_max). QuantizedTensor<16, 256> (src/core/Tensor.h:1300-1405): one
// 16-bit linear code per cell against per-block (min, max). Both are endpoint-exact and keep 0 <-> 0.
// The encoders multiply by levels / range (the reference divides, under fast-math): codes can differ from a
// correctly rounded quotient at a rounding tie only.
//
// log1p / expm1 are built on ssr_log / ssr_exp (the reference calls the CUDA math library), so codes can
// differ from the reference's by one step where its log1pf rounds differently; here host and device
// agree bit for bit.
#pragma once

#include "ssr_math.h"

#define SSR_ADAMQ_EPS 1e-15f   /* QuantizedAdamState::kEps, the Adam denominator's epsilon */

SSR_HD float ssr_log1p(float x) {   // x >= 0
    const float u = 1.0f + x;
    if (u == 1.0f) return x;
    const float um1 = u - 1.0f;        // u > 1 from here on
    if (um1 == x) return ssr_log_ge1(u);   // the correction factor x / (u - 1) is exactly 1 (always so from 2^25 on)
    return ssr_log_ge1(u) * (x / um1);
}
SSR_HD float ssr_expm1(float y) {
    const float u = ssr_exp(y);
    if (u == 1.0f) return y;
    const float um1 = u - 1.0f;
    if (um1 == -1.0f) return -1.0f;
    return um1 * (y / ssr_log(u));
}
// roundf (half away from zero) for the codes; negative inputs only need to land at or below zero
SSR_HD float ssr_round_code(float x) {
    const float r = ssr_floor(x);
    return (x - r >= 0.5f) ? r + 1.0f : r;
}

// (g1, g2) -> (u, log_s): QuantizedAdamState::g1g2_to_us / forward_sqrt_g2
SSR_HD void ssr_adamq_to_us(float g1, float g2, float* u, float* log_s) {
    const float sq = ssr_sqrt(ssr_max(g2, 0.0f));
    *u = g1 / (sq + SSR_ADAMQ_EPS);
    *log_s = ssr_log1p(ssr_max(sq, 0.0f) * (1.0f / SSR_ADAMQ_EPS));
}
// The two codes of one cell against bounds mm = (u_min, u_max, log_s_min, log_s_max) at qmax = 2^bits - 1
// levels: encode_us. The 8-bit state keeps them as u_q | s_q << 8, the 16-bit state as u_q | s_q << 16.
SSR_HD void ssr_adamq_codes(float g1, float g2, const float mm[4], float qmax, uint32_t* u_q, uint32_t* s_q) {
    float u, ls;
    ssr_adamq_to_us(g1, g2, &u, &ls);
    // codes per unit of u / log_s: depends on the bounds alone, so a loop over a block's cells divides once
    const float ku = qmax / ssr_max(mm[1] - mm[0], SSR_ADAMQ_EPS), ks = qmax / ssr_max(mm[3] - mm[2], SSR_ADAMQ_EPS);
    *u_q = (uint32_t)ssr_min(ssr_max(ssr_round_code((u - mm[0]) * ku), 0.0f), qmax);
    *s_q = (uint32_t)ssr_min(ssr_max(ssr_round_code((ls - mm[2]) * ks), 0.0f), qmax);
}
SSR_HD uint32_t ssr_adamq_encode(float g1, float g2, const float mm[4]) {     // 8-bit cell: encode_g1g2_code
    uint32_t uq, sq;
    ssr_adamq_codes(g1, g2, mm, 255.0f, &uq, &sq);
    return uq | (sq << 8);
}
SSR_HD uint32_t ssr_adamq16_encode(float g1, float g2, const float mm[4]) {   // 16-bit cell
    uint32_t uq, sq;
    ssr_adamq_codes(g1, g2, mm, 65535.0f, &uq, &sq);
    return uq | (sq << 16);
}
// decode_g1g2, in two steps: sqrt(g2) depends on the log_s code alone, so a kernel can tabulate it per
// block (256 entries for the 8-bit state) instead of evaluating expm1 per cell
SSR_HD float ssr_adamq_decode_sqrt_g2(uint32_t s_code, const float mm[4]) {
    const float kInv = 1.0f / 255.0f;
    const float ls = mm[2] + (mm[3] - mm[2]) * ((float)s_code * kInv);
    return SSR_ADAMQ_EPS * ssr_expm1(ls);
}
SSR_HD void ssr_adamq_decode_with(uint32_t code, const float mm[4], float sq, float* g1, float* g2) {
    const float kInv = 1.0f / 255.0f;
    const float u = mm[0] + (mm[1] - mm[0]) * ((float)(code & 255u) * kInv);
    *g1 = u * (sq + SSR_ADAMQ_EPS);
    *g2 = sq * sq;
}
SSR_HD void ssr_adamq_decode(uint32_t code, const float mm[4], float* g1, float* g2) {
    ssr_adamq_decode_with(code, mm, ssr_adamq_decode_sqrt_g2((code >> 8) & 255u, mm), g1, g2);
}
SSR_HD void ssr_adamq16_decode(uint32_t code, const float mm[4], float* g1, float* g2) {
    const float kInv = 1.0f / 65535.0f;
    const float u = mm[0] + (mm[1] - mm[0]) * ((float)(code & 65535u) * kInv);
    const float ls = mm[2] + (mm[3] - mm[2]) * ((float)(code >> 16) * kInv);
    const float sq = SSR_ADAMQ_EPS * ssr_expm1(ls);
    *g1 = u * (sq + SSR_ADAMQ_EPS);
    *g2 = sq * sq;
}

// QuantizedTensor<16>::encode_v_code / decode_v against bounds (lo, hi)
SSR_HD uint32_t ssr_q16_encode(float v, float lo, float hi) {
    const float k = 65535.0f / ssr_max(hi - lo, 1e-30f);
    return (uint32_t)ssr_min(ssr_max(ssr_round_code((v - lo) * k), 0.0f), 65535.0f);
}
SSR_HD float ssr_q16_decode(uint32_t code, float lo, float hi) {
    return lo + (hi - lo) * ((float)code * (1.0f / 65535.0f));
}
