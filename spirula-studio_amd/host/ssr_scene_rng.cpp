// ssr_scene_rng.cpp -- counter-based random streams for the synthetic benchmark scenes, in native
// code because the large configurations draw several hundred million values.
// splitmix64(seed ^ stream*golden) + index -> splitmix64 -> 53-bit uniform; normals by Box-Muller
// on consecutive pairs in double; the cast to float is the last step. Same definition as the
// numpy implementation in scenes.py.
#include <cmath>
#include <cstdint>
#include <cstring>

namespace {
inline uint64_t splitmix64(uint64_t z) {
    z += 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}
inline double u01(uint64_t base, uint64_t i) {
    return (double)(splitmix64(base + i) >> 11) * (1.0 / 9007199254740992.0);
}
// binary32 -> binary16, round to nearest even, subnormals and overflow to infinity handled
inline uint16_t float_to_half(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    x &= 0x7fffffffu;
    if (x >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (x > 0x7f800000u ? 0x200u : 0u));
    if (x >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);            // rounds to infinity
    if (x < 0x33000001u) return (uint16_t)sign;                          // rounds to zero
    int e = (int)(x >> 23) - 127;
    uint32_t m = (x & 0x7fffffu) | 0x800000u;
    int shift = e < -14 ? 13 + (-14 - e) : 13;                           // subnormal halves lose more bits
    uint32_t half_m = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u), mid = 1u << (shift - 1);
    if (rem > mid || (rem == mid && (half_m & 1u))) half_m++;
    if (e < -14) return (uint16_t)(sign | half_m);                       // a carry lands in the exponent field correctly
    return (uint16_t)(sign | ((((uint32_t)(e + 15)) << 10) + (half_m - 0x400u)));
}
inline float half_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, x;
    if (e == 0) {
        if (m == 0) { x = sign; }
        else { int k = 0; while (!(m & 0x400u)) { m <<= 1; k++; } x = sign | ((uint32_t)(113 - k) << 23) | ((m & 0x3ffu) << 13); }
    } else if (e == 31) x = sign | 0x7f800000u | (m << 13);
    else x = sign | ((e + 112) << 23) | (m << 13);
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}
}  // namespace

extern "C" {

void ssrh_rng_uniform(uint64_t seed, uint64_t stream, int64_t start, int64_t n, double lo, double hi, float* out) {
    const uint64_t base = splitmix64(seed ^ (stream * 0x9E3779B97F4A7C15ull));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) out[i] = (float)(lo + (hi - lo) * u01(base, (uint64_t)(start + i)));
}

void ssrh_rng_normal(uint64_t seed, uint64_t stream, int64_t n, double mean, double sigma, float* out) {
    const uint64_t base = splitmix64(seed ^ (stream * 0x9E3779B97F4A7C15ull));
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; i++) {
        const uint64_t pair = (uint64_t)i >> 1;
        const double u1 = 1.0 - u01(base, 2 * pair);
        const double u2 = u01(base, 2 * pair + 1);
        const double r = std::sqrt(-2.0 * std::log(u1));
        const double a = 6.283185307179586476925 * u2;
        out[i] = (float)(mean + sigma * ((i & 1) ? r * std::sin(a) : r * std::cos(a)));
    }
}

// int8 codes with one fp16 scale per row: scale = half(max|v| / 127) (smallest subnormal if that
// rounds to zero for a non-zero row), code = clamp(rint(v / scale), -127, 127), decoded = code * scale.
// Same definition as quantize_i8_f16 in scenes.py; here because ten million rows of 45 take numpy half a minute.
void ssrh_quantize_i8_f16(int64_t rows, int cells, const float* values, int8_t* codes, uint16_t* scale_f16, float* decoded) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        const float* v = values + r * cells;
        float amax = 0.0f;
        for (int i = 0; i < cells; i++) amax = std::fmax(amax, std::fabs(v[i]));
        uint16_t h = float_to_half(amax / 127.0f);
        if (h == 0 && amax > 0.0f) h = 1;
        const float s = half_to_float(h);
        scale_f16[r] = h;
        for (int i = 0; i < cells; i++) {
            float q = s > 0.0f ? std::nearbyint(v[i] / s) : 0.0f;
            q = q < -127.0f ? -127.0f : (q > 127.0f ? 127.0f : q);
            codes[r * cells + i] = (int8_t)q;
            decoded[r * cells + i] = (float)(int8_t)q * s;
        }
    }
}

}  // extern "C"
