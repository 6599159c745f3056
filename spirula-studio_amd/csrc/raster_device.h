// raster_device.h -- fragment staging and alpha evaluation shared by the compositing forward (K7)
// and backward (K8) kernels.
//
// Work decomposition (native to 64-wide wavefronts): one 256-thread workgroup per 16x16 binning
// tile; each of its 4 wavefronts owns one 8x8 sub-tile, one lane per pixel. The tile's sorted
// range is staged through LDS in batches of 256 fragments (one fragment per thread, read once per
// tile instead of once per sub-tile), together with a 4-bit footprint mask: bit m says whether
// the splat's alpha >= 1/255 ellipse reaches sub-tile m. That is the reference's per-sub-tile
// cull (src/kernels/raster/RasterizationEval3DFwd_kernel.cuh:203-209,
// src/kernels/raster/RasterizationEval3DBwd_kernel.cuh:336-342 with ellipse_box_overlap_test,
// src/core/Common.cuh:55-77); a wavefront walks only the fragments whose bit is set, with a
// scalar bit-scan over a 64-bit ballot, so the skip costs no vector work.
#pragma once
#include "common.h"

namespace ssr {

constexpr int kRasterBlock = 256;
constexpr int kBatch = 256;

// One staged fragment: 3 x 16 bytes, read back with broadcast 128-bit LDS loads.
//   q0 = (x, y, 0.5*conic.x, conic.y)   q1 = (0.5*conic.z, opac, r, g)   q2 = (b, depth, hitmask, sigma cut)
struct FragLds {
    float4 q0, q1, q2;
};

__device__ __forceinline__ bool ellipse_box_overlap(const float ic[3], float x0, float x1, float y0, float y1) {
    float a = ic[0], b = ic[1], c = ic[2];
    const float wx = (-b) / c, wy = (-b) / a;
    const float u0 = ssr_min(ssr_max(x0 * wx, y0), y1);
    const float u1 = ssr_min(ssr_max(x1 * wx, y0), y1);
    const float v0 = ssr_min(ssr_max(y0 * wy, x0), x1);
    const float v1 = ssr_min(ssr_max(y1 * wy, x0), x1);
    b = b * 2.0f;
    const float mx = ssr_min(((a * x0) * x0 + (b * x0) * u0) + (c * u0) * u0,
                             ((a * x1) * x1 + (b * x1) * u1) + (c * u1) * u1);
    const float my = ssr_min(((a * v0) * v0 + (b * v0) * y0) + (c * y0) * y0,
                             ((a * v1) * v1 + (b * v1) * y1) + (c * y1) * y1);
    const float mc = ssr_max(ssr_max(x0, -x1), ssr_max(y0, -y1));
    return ssr_min(mc, ssr_min(mx, my) - 1.0f) < 0.f;
}

// Per-splat values that do not depend on the tile: the sigma cut (above it alpha <= 1/255 for
// certain: ln(255 opac) plus a margin far larger than the rounding of log/exp, so no lane is
// skipped that the reference would keep) and the conic scale of the footprint ellipse.
__device__ __forceinline__ void fragment_constants(float opac, float& cut, float& kk) {
    cut = 0.0f; kk = 0.0f;
    if (opac > kAlphaThreshold) {
        const float lg = ssr_log(opac / kAlphaThreshold);
        // exp_neg_small() is exact down to -87; only a caller-supplied opac beyond e^80 exceeds that
        cut = ssr_min(lg + 1e-3f, 80.0f);
        kk = 0.5f / lg;
    }
}

// A fragment row as K1 can lay it out in HBM: 48 contiguous bytes per splat,
//   (x, y, 0.5 conic.x, conic.y | 0.5 conic.z, opac, r, g | b, depth, sigma cut, footprint scale),
// one or two cache lines per gather instead of five.
constexpr int kPackedRowFloats = 12;

// Brings splat `g` into the staged form and computes its sub-tile footprint mask, either from a
// packed row or by gathering the five screen arrays.
__device__ __forceinline__ FragLds stage_fragment(const ssr_screen& s, const float* __restrict__ packed, int32_t g,
                                                  float tile_x0, float tile_y0, float* kk_out = nullptr) {
    FragLds f;
    float cut, kk;
    if (packed) {
        const float4* row = reinterpret_cast<const float4*>(packed) + 3 * (int64_t)g;
        f.q0 = row[0]; f.q1 = row[1];
        const float4 r2 = row[2];
        f.q2 = make_float4(r2.x, r2.y, 0.0f, r2.z);
        cut = r2.z; kk = r2.w;
    } else {
        const float2 xy = *reinterpret_cast<const float2*>(s.xy + 2 * (int64_t)g);
        const float* cn = s.conic + 3 * (int64_t)g;
        const float opac = s.opac[g];
        const float* rg = s.rgb + 3 * (int64_t)g;
        fragment_constants(opac, cut, kk);
        f.q0 = make_float4(xy.x, xy.y, 0.5f * cn[0], cn[1]);
        f.q1 = make_float4(0.5f * cn[2], opac, rg[0], rg[1]);
        f.q2 = make_float4(rg[2], s.depth[g], 0.0f, cut);
    }
    uint32_t hits = 0;
    if (f.q1.y > kAlphaThreshold) {
        // conic.x = 2 * (0.5 conic.x) exactly, conic.z likewise
        const float ic[3] = {(f.q0.z + f.q0.z) * kk, f.q0.w * kk, (f.q1.x + f.q1.x) * kk};
        const float x = f.q0.x, y = f.q0.y;
#pragma unroll
        for (int m = 0; m < 4; m++) {
            const float bx0 = tile_x0 + (float)((m & 1) * kMicro), by0 = tile_y0 + (float)((m >> 1) * kMicro);
            if (ellipse_box_overlap(ic, bx0 - x, (bx0 + (float)kMicro) - x, by0 - y, (by0 + (float)kMicro) - y))
                hits |= 1u << m;
        }
    }
    f.q2.z = __uint_as_float(hits);
    if (kk_out) *kk_out = kk;
    return f;
}

// ---- 4x4-pixel blocks: the row-granular kernels ------------------------------------------------
//
// The row-granular variants of K7 / K8 cut a 16x16 tile into sixteen 4x4-pixel blocks. Block id =
// 4 * sub_tile + quadrant (sub_tile m as above, quadrant = (y bit 2) * 2 + (x bit 2) inside it), so the
// four 16-lane rows of wavefront m own the four blocks of sub-tile m. Every staged fragment carries a
// 16-bit block mask in the upper half of the word that holds the 4-bit sub-tile mask: bit b is set when
// the reference's sub-tile test passes for b's sub-tile AND the alpha >= 1/255 ellipse, grown by a
// margin far above rounding, reaches the box of b's pixel centres -- a superset of the blocks in which
// any pixel composites the splat, so the pixel results are those of the sub-tile walk.
constexpr int kBlock = 4;
constexpr int kBlocksPerTile = 16;

// Block bits of the two block rows (bands of four pixel-centre lines) of tile half `half` (sub-tiles 2 half
// and 2 half + 1): bit 4 (column >> 1) + 2 band + (column & 1), i.e. 4 (m & 1) + quadrant. Conservative test
// of "the ellipse q(d) = a dx^2 + 2 b dx dy + c dy^2 <= 1 + margin reaches a pixel centre of the block": the
// part of the ellipse inside the band dy in [Y0, Y1] is convex, so its extent in x is one interval --
// between the band's two end lines, or out to the ellipse's extreme points when those lie inside the band --
// and a block is reached exactly when its centres' x range meets that interval. The margin (1e-3) is far
// above the rounding of this arithmetic and of the alpha evaluation; a degenerate conic keeps every block.
__device__ __forceinline__ uint32_t block_bits_of_half(float a, float b, float c, float x, float y, float tile_x0,
                                                       float tile_y0, int half) {
    const float t = 1.001f;
    const float det = a * c - b * b;
    if (!(det > 0.0f) || !(a > 0.0f) || !(c > 0.0f)) return 0xFFu;
    const float inv_det = __builtin_amdgcn_rcpf(det), inv_a = __builtin_amdgcn_rcpf(a);
    const float ymax = __builtin_amdgcn_sqrtf((a * t) * inv_det) * 1.0001f;
    const float xmax = __builtin_amdgcn_sqrtf((c * t) * inv_det) * 1.0001f;
    const float y_r = -(b * __builtin_amdgcn_rcpf(c)) * xmax;   // dy at which dx is largest; -y_r where it is smallest
    const float nba = -b * inv_a, at = a * t;
    uint32_t bits = 0;
#pragma unroll
    for (int band = 0; band < 2; band++) {
        const float Y0 = (tile_y0 + (float)(half * kMicro + band * kBlock) + 0.5f) - y, Y1 = Y0 + (float)(kBlock - 1);
        const float yl = __builtin_fmaxf(Y0, -ymax), yh = __builtin_fminf(Y1, ymax);
        if (!(yl <= yh)) continue;
        const float hl = __builtin_amdgcn_sqrtf(__builtin_fmaxf(ssr_fma(-det * yl, yl, at), 0.0f)) * inv_a * 1.0001f + 1e-4f;
        const float hh = __builtin_amdgcn_sqrtf(__builtin_fmaxf(ssr_fma(-det * yh, yh, at), 0.0f)) * inv_a * 1.0001f + 1e-4f;
        const float cl = nba * yl, ch = nba * yh;
        float xr = __builtin_fmaxf(cl + hl, ch + hh), xl = __builtin_fminf(cl - hl, ch - hh);
        if (yl <= y_r && y_r <= yh) xr = xmax;
        if (yl <= -y_r && -y_r <= yh) xl = -xmax;
#pragma unroll
        for (int col = 0; col < 4; col++) {
            const float X0 = (tile_x0 + (float)(col * kBlock) + 0.5f) - x;
            if (X0 <= xr && X0 + (float)(kBlock - 1) >= xl) bits |= 1u << (4 * (col >> 1) + 2 * band + (col & 1));
        }
    }
    return bits;
}

// The eight block bits (bit 4 (m & 1) + quadrant) of tile half `half` (sub-tiles 2 half and 2 half + 1) for a fragment
// given by the first two quarters of its row (x, y, 0.5 conic.x, conic.y | 0.5 conic.z, opac, ..) and its footprint
// scale kk: the reference's sub-tile test, then the block tests of the sub-tiles that pass.
__device__ __forceinline__ uint32_t fragment_block_bits_half(const float4& q0, const float4& q1, float kk, float tile_x0,
                                                             float tile_y0, int half) {
    if (!(q1.y > kAlphaThreshold)) return 0u;
    // conic.x = 2 * (0.5 conic.x) exactly, conic.z likewise
    const float ic[3] = {(q0.z + q0.z) * kk, q0.w * kk, (q1.x + q1.x) * kk};
    const float x = q0.x, y = q0.y;
    uint32_t sub = 0;   // the reference's test for the two sub-tiles of this half
#pragma unroll
    for (int mm = 0; mm < 2; mm++) {
        const int m = 2 * half + mm;
        const float sx0 = tile_x0 + (float)((m & 1) * kMicro), sy0 = tile_y0 + (float)((m >> 1) * kMicro);
        if (ellipse_box_overlap(ic, sx0 - x, (sx0 + (float)kMicro) - x, sy0 - y, (sy0 + (float)kMicro) - y)) sub |= 0xFu << (4 * mm);
    }
    return sub ? sub & block_bits_of_half(ic[0], ic[1], ic[2], x, y, tile_x0, tile_y0, half) : 0u;
}

// Stages splat g for the row-granular backward, where two threads share a fragment: thread `half`
// (0 / 1) runs the reference's sub-tile test for sub-tiles 2 half and 2 half + 1 and the block tests of
// those that pass; it returns their eight block bits (bit 4 (m & 1) + quadrant). The fragment record
// itself is the same from either thread.
// `mask` (optional): the sixteen block bits the forward recorded for this sorted entry; the tests are then skipped.
__device__ __forceinline__ FragLds stage_fragment_half(const ssr_screen& s, const float* __restrict__ packed, int32_t g,
                                                       float tile_x0, float tile_y0, int half, uint32_t& bits8,
                                                       const uint16_t* __restrict__ mask = nullptr) {
    FragLds f;
    float cut, kk;
    if (packed) {
        const float4* row = reinterpret_cast<const float4*>(packed) + 3 * (int64_t)g;
        f.q0 = row[0]; f.q1 = row[1];
        const float4 r2 = row[2];
        f.q2 = make_float4(r2.x, r2.y, 0.0f, r2.z);
        cut = r2.z; kk = r2.w;
    } else {
        const float2 xy = *reinterpret_cast<const float2*>(s.xy + 2 * (int64_t)g);
        const float* cn = s.conic + 3 * (int64_t)g;
        const float opac = s.opac[g];
        const float* rg = s.rgb + 3 * (int64_t)g;
        fragment_constants(opac, cut, kk);
        f.q0 = make_float4(xy.x, xy.y, 0.5f * cn[0], cn[1]);
        f.q1 = make_float4(0.5f * cn[2], opac, rg[0], rg[1]);
        f.q2 = make_float4(rg[2], s.depth[g], 0.0f, cut);
    }
    bits8 = mask ? ((uint32_t)*mask >> (8 * half)) & 0xFFu : fragment_block_bits_half(f.q0, f.q1, kk, tile_x0, tile_y0, half);
    return f;
}

// Adds the block mask to a fragment staged by stage_fragment (bits 16..31 of the mask word; bit 4 m + quadrant).
__device__ __forceinline__ void add_block_mask(FragLds& f, float kk, float tile_x0, float tile_y0) {
    const uint32_t hits = __float_as_uint(f.q2.z);
    uint32_t blocks = 0;
    if (hits) {
        const float a = (f.q0.z + f.q0.z) * kk, b = f.q0.w * kk, c = (f.q1.x + f.q1.x) * kk;
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const uint32_t sub = ((hits >> (2 * half)) & 1u ? 0x0Fu : 0u) | ((hits >> (2 * half + 1)) & 1u ? 0xF0u : 0u);
            if (sub) blocks |= (sub & block_bits_of_half(a, b, c, f.q0.x, f.q0.y, tile_x0, tile_y0, half)) << (8 * half);
        }
    }
    f.q2.z = __uint_as_float(hits | (blocks << 16));
}

// exp(x) for x in [-87, 0] (and NaN): the same operations as ssr_exp() on that range, where its
// overflow / underflow branches are dead and 2^k (k in [-126, 0], result normal) can be applied by
// adding k to the exponent field -- exact, so the bits equal ssr_exp(x).
__device__ __forceinline__ float exp_neg_small(float x) {
    const float k = ssr_rint(x * 1.44269504088896341f);
    float r = ssr_fma(k, -0.693359375f, x);
    r = ssr_fma(k, 2.12194440e-4f, r);
    const float z = r * r;
    float p = 1.9875691500e-4f;
    p = ssr_fma(p, r, 1.3981999507e-3f);
    p = ssr_fma(p, r, 8.3334519073e-3f);
    p = ssr_fma(p, r, 4.1665795894e-2f);
    p = ssr_fma(p, r, 1.6666665459e-1f);
    p = ssr_fma(p, r, 5.0000001201e-1f);
    const float y = ssr_fma(p, z, r) + 1.0f;
    int ki;   // hardware conversion: saturating, NaN -> 0 (a C cast of NaN would be undefined)
    asm("v_cvt_i32_f32 %0, %1" : "=v"(ki) : "v"(k));
    return __uint_as_float(__float_as_uint(y) + ((uint32_t)ki << 23));
}

// FragmentFwd::evaluate_alpha (src/primitives/Primitive3DGS.cuh:250-260): sigma = 0.5 (a dx^2 + c dy^2)
// + b dx dy with the fused operations placed as written here, alpha = min(0.999, opac exp(-sigma)),
// 0 for sigma < 0. The exponential is taken without its range handling: identical results wherever
// alpha > 1/255 can hold (0 <= sigma <= cut), and alpha = 0 -- the skipped case -- elsewhere.
__device__ __forceinline__ float eval_alpha_fast(const float4& q0, const float4& q1, float cut, float px, float py,
                                                 float& dx, float& dy, float& vis, float& sigma) {
    dx = q0.x - px; dy = q0.y - py;
    sigma = ssr_fma(q0.z * dx, dx, ssr_fma(q1.x * dy, dy, (q0.w * dx) * dy));
    // outside [0, cut] the exponent arithmetic of exp_neg_small is meaningless: force vis = 0 there,
    // which also makes alpha 0 and keeps every product formed from vis finite
    const float e = exp_neg_small(-sigma);
    vis = (sigma < 0.f || sigma > cut) ? 0.f : e;
    return ssr_min(0.999f, q1.y * vis);
}

// Workgroup id -> tile id so that each of the 8 XCDs (workgroups are dealt to them round-robin)
// works on one contiguous band of tiles and its L2 keeps that band's splat rows.
__device__ __forceinline__ int xcd_tile_of(int wg, int n_tiles) {
    const int chunk = (n_tiles + 7) >> 3;
    return (wg & 7) * chunk + (wg >> 3);
}
inline int xcd_grid_size(int n_tiles) { return ((n_tiles + 7) >> 3) * 8; }
// With a caller's launch order (ssr_tile_order: all tiles, longest first) workgroup w takes its w-th entry: the
// round-robin dealing then gives every XCD the same mix of long and short tiles.
__device__ __forceinline__ int tile_of_workgroup(const int32_t* __restrict__ order, int wg, int n_tiles) {
    if (!order) return xcd_tile_of(wg, n_tiles);
    return wg < n_tiles ? order[wg] : -1;
}

// K8's plain variant with one lane per fragment (raster_bwd_lanes.hip); validated arguments, launch only.
int launch_raster_bwd_lanes(const ssr_raster_bwd_params& p, int tw, int th, int nimg, hipStream_t st);

}  // namespace ssr
