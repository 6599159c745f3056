// ssr_scene_rng.cpp -- counter-based random streams for the synthetic benchmark scenes, in native
// code because the large configurations draw several hundred million values.
// splitmix64(seed ^ stream*golden) + index -> splitmix64 -> 53-bit uniform; normals by Box-Muller
// on consecutive pairs in double; the cast to float is the last step. Same definition as the
// numpy implementation in scenes.py.
#include <cmath>
#include <cstdint>

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

}  // extern "C"
