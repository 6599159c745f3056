// raster_bwd.hip -- K8: compositing backward. Replays each tile's sorted range back to front,
// undoing the transmittance recursion, and accumulates per-Gaussian screen-space gradients.
//
// Follows rasterize_to_pixels_bwd_kernel with IS_EVAL3D=0, dist_type=None, no median, no
// accumulation weights (src/kernels/raster/RasterizationEval3DBwd_kernel.cuh:48-636) and the
// fragment VJPs of src/primitives/Primitive3DGS.cuh:262-300:
//   per pixel   v_T <- v_T + depth_out * v_depth / W,  v_depth <- v_depth / W,  W = max(1-T,1e-10)
//   per splat k <= last_id with alpha > 1/255:
//     T0 = T1/(1-alpha); v_alpha = T0 (c.v_c) - v_T1 T0; v_c_k = alpha T0 v_c;
//     v_T0 = alpha (c.v_c) + v_T1 (1-alpha)
//
// Native schedule instead of the reference's 32-lane systolic sweep: one workgroup per 16x16 tile, a wavefront per
// 8x8 sub-tile, and within it each 16-lane row holds one 4x4-pixel block (pixel state in registers). Fragments are
// staged per tile in LDS, back to front, shared by the tile's four wavefronts; every row walks its OWN list of the
// staged fragments -- those whose block bit is set (raster_device.h) and whose sorted index does not exceed the
// block's largest last_id. A splat of a few pixels' radius touches about half of the blocks of the sub-tiles it
// touches, so far fewer lanes idle than when all 64 lanes visit every fragment of the sub-tile. Lists are built per
// batch by the wavefront that walks them (ballot + rank, slot numbers as bytes). The scan starts at the tile's
// largest last_id rather than at the end of the range; splats beyond it are skipped by every pixel anyway.
// The ten per-splat sums are reduced inside each row by a transposing reduction over the four lane bits (row_ror:8,
// row_half_mirror, two quad permutations): every level halves the number of live registers by keeping one channel in
// the lanes with the bit clear and another in those with it set, so 23 operations leave each of ten lanes of the
// row holding one finished channel. What is summed are moments of u = vis * v_alpha: (u, u dx, u dy, u dx^2,
// u dx dy, u dy^2) and the four colour / depth weights; the gradients of position, conic and opacity are linear in
// them and are formed once per fragment when its sums leave LDS for global memory -- one set of atomics per (splat,
// tile), non-finite sums dropped and zeros skipped as in the reference (src/core/Common.cuh:791-856).
// exp(-sigma) comes from the hardware exponential; whenever a lane's alpha falls within 1.6e-7 of the 1/255
// threshold or within 4e-5 of the 0.999 gate, the wavefront re-evaluates with the bit-defined exponential, so every
// decision is the one the forward took.
#include <type_traits>

#include "raster_device.h"

namespace ssr {

// float atomic max through the integer orderings (src/core/Common.cuh:784-788)
__device__ __forceinline__ void atomic_max_f32(float* p, float v) {
    if (__float_as_int(v) >= 0) atomicMax(reinterpret_cast<int*>(p), __float_as_int(v));
    else atomicMin(reinterpret_cast<unsigned*>(p), __float_as_uint(v));
}

// kDist (SSR_DIST_*), kMedian and kAccum (SSR_ACCUM_*) select the variants
// (RasterizationEval3DBwd_kernel.cuh:150-172,207-279,433-585); <0, false, 0> is the plain kernel and
// compiles to exactly the code it had without them.
// Row of accum_weight a screen row adds into: its world row. Packed rows carry it in gaussian_ids;
// [C,N] rows are c * N + n (RasterizationEval3DBwd_kernel.cuh:368).
__device__ __forceinline__ int64_t accum_row(const ssr_raster_bwd_params& P, uint32_t g) {
    if (P.gaussian_ids) return (int64_t)P.gaussian_ids[g];
    return P.num_images > 1 ? (int64_t)(g % (uint32_t)P.num_world) : (int64_t)g;
}

template <int kCtrl>
__device__ __forceinline__ float dpp_full(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xf, 0xf, true));
}
// lanes with `sel` clear end with a[l] + a[partner], lanes with it set with b[l] + b[partner]
template <int kCtrl>
__device__ __forceinline__ float fold_pair(float a, float b, bool sel) {
    const float keep = sel ? b : a, send = sel ? a : b;
    return keep + dpp_full<kCtrl>(send);
}
constexpr int kDppQuadXor2 = 0x4E, kDppQuadXor1 = 0xB1;

constexpr int kRowBatch = 128;   // fragments staged per batch by the row-granular kernel

// kAccum: the pixel-weight accumulation of the densifier (RasterizationEval3DBwd_kernel.cuh:553-562,574-585). Sum and
// average ride as two more channels (map * w and w) through the same reduction, in lanes that hold copies otherwise;
// the maximum takes a reduction of its own.
template <int kDist, bool kMedian, int kAccum>
__device__ __forceinline__ void raster_bwd_rows_body(const ssr_raster_bwd_params& P, int tile_w, int tile_h) {
    constexpr bool kSums = kAccum == SSR_ACCUM_SUM || kAccum == SSR_ACCUM_AVG;
    constexpr int kCh = kSums ? 12 : 10;   // channels per fragment slot
    // Fragments per batch: with twelve channels in four copies a batch of 128 would take 33 KB of LDS and leave four
    // workgroups per compute unit instead of five, which costs this latency-bound kernel more than the shorter batch
    constexpr int kB = kSums ? 112 : kRowBatch;
    static_assert(kB <= 128 && 2 * kB <= kRasterBlock && (4 * kB) % 8 == 0, "two threads stage a fragment; a wavefront blanks its lists with 8-byte stores");
    __shared__ FragLds frags[kB + 1];   // the last one is the blank fragment that ends every list
    __shared__ int32_t s_ids[kB];
    __shared__ int s_wave_max[4];
    // Moment sums per (wavefront, fragment, channel). Each wavefront adds into its own copy with a plain
    // read-add-write: a float atomic in LDS costs about three cycles per active lane on this hardware,
    // which at forty lanes a step would make LDS, not arithmetic, the limit of this kernel.
    __shared__ float s_acc[4 * kB * kCh];
    [[maybe_unused]] __shared__ float s_max[kAccum == SSR_ACCUM_MAX ? 4 * kB : 1];   // per wavefront and slot: largest map * w
    __shared__ uint8_t s_bits[2 * kB];                       // block bits of sub-tiles {0,1} and {2,3}
    // distortion composites ln(max(z, 1e-6)): the value and the factor d ln z / dz per staged fragment
    [[maybe_unused]] __shared__ float s_lz[kDist != SSR_DIST_NONE ? kB + 1 : 1];
    [[maybe_unused]] __shared__ float s_iz[kDist != SSR_DIST_NONE ? kB + 1 : 1];
    __shared__ __attribute__((aligned(8))) uint8_t s_list[kBlocksPerTile * kB + 16];
    const int n_tiles = tile_w * tile_h * (P.num_images > 1 ? P.num_images : 1);
    const int tile = tile_of_workgroup(P.tile_order, blockIdx.x, n_tiles);
    if (tile < 0 || tile >= n_tiles) return;
    const int tid = threadIdx.x, lane = tid & 63, mt = tid >> 6, row = lane >> 4, l16 = lane & 15;
    const int gy = tile / tile_w, tx = tile - gy * tile_w;
    const int img = gy / tile_h, ty = gy - img * tile_h;
    const int j = tx * kTile + (mt & 1) * kMicro + (row & 1) * kBlock + (l16 & 3);
    const int i = ty * kTile + (mt >> 1) * kMicro + (row >> 1) * kBlock + (l16 >> 2);
    const float px = (float)j + 0.5f, py = (float)i + 0.5f;
    const bool inside = (uint32_t)i < P.height && (uint32_t)j < P.width;
    const int64_t pid = ((int64_t)img * P.height + i) * P.width + j;

    const int32_t bin_final = inside ? P.last_ids[pid] : -1;
    float T1 = inside ? P.render_T[pid] : 0.0f;
    float vT1 = inside ? P.v_render_T[pid] : 0.0f;
    float vr = 0.f, vg = 0.f, vb = 0.f, vd = 0.f;
    if (inside) {
        const float* v = P.v_render_rgb + 3 * pid;
        vr = v[0]; vg = v[1]; vb = v[2];
        vd = P.v_render_depth[pid];
    }
    // totals of the forward held constant during the sweep (distortion), median state
    [[maybe_unused]] float Cr = 0.f, Cg = 0.f, Cb = 0.f, Cd = 0.f, Sr = 0.f, Sg = 0.f, Sb = 0.f, Sd = 0.f;
    [[maybe_unused]] float vDr = 0.f, vDg = 0.f, vDb = 0.f, vDd = 0.f, Wd = 0.f;
    [[maybe_unused]] float med_v = 0.f, pend_zgrad = 0.f, pend_zfar = 0.f, pend_Tfar = 0.f;
    {
        const float inv_alpha = 1.0f / ssr_max(1.0f - T1, 1e-10f);
        const float exp_depth = inside ? P.render_depth[pid] : 0.0f;
        if constexpr (kDist != SSR_DIST_NONE) {
            // log-depth render: depth = exp(C_lnz / W)  (RasterizationEval3DBwd_kernel.cuh:212-218)
            const float m = ssr_log(ssr_max(exp_depth, 1e-6f));
            vT1 = vT1 + ((exp_depth * vd) * m) * inv_alpha;
            vd = vd * (exp_depth * inv_alpha);
            // C, S = (D + C^2) / W, W and the distortion cotangent (:228-257)
            Cd = m * ssr_max(1.0f - T1, 1e-10f);
            Wd = inside ? (1.0f - T1) : 0.0f;
            const float invW = Wd > 1e-10f ? (1.0f / Wd) : 0.0f;
            float Dd = 0.f, Dr = 0.f, Dg = 0.f, Db = 0.f;
            if (inside) {
                Dd = P.distortion_depth[pid]; vDd = P.v_distortion_depth[pid];
                if constexpr (kDist == SSR_DIST_RGB_D) {
                    const float* c = P.render_rgb + 3 * pid; Cr = c[0]; Cg = c[1]; Cb = c[2];
                    const float* d = P.distortion_rgb + 3 * pid; Dr = d[0]; Dg = d[1]; Db = d[2];
                    const float* v = P.v_distortion_rgb + 3 * pid; vDr = v[0]; vDg = v[1]; vDb = v[2];
                }
            }
            Sd = (Dd + Cd * Cd) * invW;
            if constexpr (kDist == SSR_DIST_RGB_D) {
                Sr = (Dr + Cr * Cr) * invW; Sg = (Dg + Cg * Cg) * invW; Sb = (Db + Cb * Cb) * invW;
            }
        } else {
            vT1 = vT1 + (exp_depth * vd) * inv_alpha;
            vd = vd * inv_alpha;
        }
        if constexpr (kMedian) med_v = inside ? P.v_render_median[pid] : 0.0f;
    }
    [[maybe_unused]] float amap = 0.0f;
    if constexpr (kAccum != SSR_ACCUM_NONE) amap = inside ? P.accum_weight_map[pid] : 0.0f;

    const int32_t range_start = P.tile_offsets[tile];
    const int32_t range_end = (tile == n_tiles - 1 && !P.tile_offsets_closed) ? (int32_t)P.n_isects : P.tile_offsets[tile + 1];
    // largest last_id per block (row), per wavefront, per tile
    int row_last = bin_final;
#pragma unroll
    for (int d = 8; d >= 1; d >>= 1) row_last = max(row_last, __shfl_xor(row_last, d, 16));
    const int blk_last[4] = {__builtin_amdgcn_readlane(row_last, 0), __builtin_amdgcn_readlane(row_last, 16),
                             __builtin_amdgcn_readlane(row_last, 32), __builtin_amdgcn_readlane(row_last, 48)};
    const int wave_last = max(max(blk_last[0], blk_last[1]), max(blk_last[2], blk_last[3]));
    if (lane == 0) s_wave_max[mt] = wave_last;
    __syncthreads();
    const int tile_last = max(max(s_wave_max[0], s_wave_max[1]), max(s_wave_max[2], s_wave_max[3]));
    const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);

    // which finished channel this lane holds after the reduction (see the fold order below): -1 none
    const bool b3 = (l16 & 8) != 0, b2 = (l16 & 4) != 0, b1 = (l16 & 2) != 0, b0 = (l16 & 1) != 0;
    int chan = -1;
    if (!b0) chan = 4 * (b1 ? 1 : 0) + 2 * (b2 ? 1 : 0) + (b3 ? 1 : 0);
    else if (!b1 && (!b2 || kSums)) chan = 8 + 2 * (b2 ? 1 : 0) + (b3 ? 1 : 0);
    for (int e = tid; e < 4 * kB * kCh; e += kRasterBlock) s_acc[e] = 0.0f;
    if constexpr (kAccum == SSR_ACCUM_MAX) { for (int e = tid; e < 4 * kB; e += kRasterBlock) s_max[e] = 0.0f; }
    // A list is read without asking where it ends: behind its entries stands slot kB, a fragment of opacity
    // zero, which no pixel takes up and whose sums stay zero. The tail of the last list is filled here, the rest by
    // each wavefront before it builds its lists (the first barrier of the batch loop orders this with the reads).
    for (int e = tid; e < (int)sizeof(s_list); e += kRasterBlock) s_list[e] = (uint8_t)kB;
    if (tid == 0) {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        // the blank fragment: no opacity, and a conic that puts every pixel far beyond any band (its sigma is huge)
        frags[kB].q0 = make_float4(0.f, 0.f, 1e30f, 0.f); frags[kB].q1 = z; frags[kB].q2 = z;
        if constexpr (kDist != SSR_DIST_NONE) { s_iz[kB] = 0.0f; s_lz[kB] = 0.0f; }
    }
    float* my_acc = s_acc + mt * (kB * kCh);
    char* my_cells = reinterpret_cast<char*>(my_acc + (chan >= 0 ? chan : 0));   // + 4 kCh bytes per fragment slot

    // Two neighbouring threads own fragment slot t / 2: they add up the four wavefronts' moment sums, turn
    // them into the ten gradient channels (x, y, depth, conic[3], opac, rgb[3]) and leave those in the first
    // copy; then all threads move the batch to global memory in the order of the destination rows, so that
    // a row's atomics travel as one or two requests.
    auto flush = [&]() {
        if (tid < 2 * kB) {
            const int slot = tid >> 1;
            const bool geom = (tid & 1) == 0;   // this thread: u, ux, uy, uxx, uxy, uyy; its neighbour: the colour / depth weights
            float m[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            const int c0 = geom ? 0 : 6, nc = geom ? 6 : kCh - 6;
#pragma unroll
            for (int w = 0; w < 4; w++)
#pragma unroll
                for (int c = 0; c < 6; c++)
                    if (c < nc) { m[c] += s_acc[(w * kB + slot) * kCh + c0 + c]; }
#pragma unroll
            for (int w = 1; w < 4; w++)
#pragma unroll
                for (int c = 0; c < 6; c++)
                    if (c < nc) s_acc[(w * kB + slot) * kCh + c0 + c] = 0.0f;
            float o[6];
            if (geom) {
                const float4 q0 = frags[slot].q0, q1 = frags[slot].q1;
                const float k = -q1.y;                       // v_sigma = -(opac vis) v_alpha = k u
                const float sx = k * m[1], sy = k * m[2];
                o[0] = ssr_fma(q0.z + q0.z, sx, q0.w * sy);  // conic.x = 2 * (0.5 conic.x), conic.z likewise
                o[1] = ssr_fma(q0.w, sx, (q1.x + q1.x) * sy);
                o[2] = (0.5f * k) * m[3]; o[3] = k * m[4]; o[4] = (0.5f * k) * m[5];
                o[5] = m[0];
            } else {
                o[0] = m[3]; o[1] = m[0]; o[2] = m[1]; o[3] = m[2]; o[4] = 0.f; o[5] = 0.f;
            }
            // both threads of a slot sit in one wavefront: order that wavefront's reads above before the writes below
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            float* dst = s_acc + slot * kCh;
            if (geom) {
                dst[0] = ssr_isfinite(o[0]) ? o[0] : 0.f; dst[1] = ssr_isfinite(o[1]) ? o[1] : 0.f;
                dst[3] = ssr_isfinite(o[2]) ? o[2] : 0.f; dst[4] = ssr_isfinite(o[3]) ? o[3] : 0.f;
                dst[5] = ssr_isfinite(o[4]) ? o[4] : 0.f; dst[6] = ssr_isfinite(o[5]) ? o[5] : 0.f;
            } else {
                dst[2] = ssr_isfinite(o[0]) ? o[0] : 0.f;
                dst[7] = ssr_isfinite(o[1]) ? o[1] : 0.f; dst[8] = ssr_isfinite(o[2]) ? o[2] : 0.f;
                dst[9] = ssr_isfinite(o[3]) ? o[3] : 0.f;
                if constexpr (kSums) { dst[10] = ssr_isfinite(m[4]) ? m[4] : 0.f; dst[11] = ssr_isfinite(m[5]) ? m[5] : 0.f; }
            }
        }
        __syncthreads();
        if (P.v_rows) {
            // with weight sums, those leave in the row's two spare floats: the same cache line and request as the ten
            // gradients (atomics of their own to the weight arrays double this kernel's L2 atomic requests);
            // accum_from_rows_kernel moves them on afterwards
            for (int e = tid; e < kB * kCh; e += kRasterBlock) {
                const int slot = e / kCh, ch = e - slot * kCh;
                const float x = s_acc[slot * kCh + ch];
                if (x != 0.0f) {
                    s_acc[slot * kCh + ch] = 0.0f;
                    atomicAdd(P.v_rows + (int64_t)12 * s_ids[slot] + ch, x);
                }
            }
        } else if (tid < kB) {
            float v[10];
            bool any = false;
#pragma unroll
            for (int c = 0; c < 10; c++) { v[c] = s_acc[tid * kCh + c]; any |= v[c] != 0.0f; }
            if (any) {
#pragma unroll
                for (int c = 0; c < 10; c++) s_acc[tid * kCh + c] = 0.0f;
                const int64_t g = s_ids[tid];
                auto add = [](float* p, float x) { if (x != 0.0f) atomicAdd(p, x); };
                add(P.v_screen.xy + 2 * g, v[0]); add(P.v_screen.xy + 2 * g + 1, v[1]);
                add(P.v_screen.depth + g, v[2]);
                add(P.v_screen.conic + 3 * g, v[3]); add(P.v_screen.conic + 3 * g + 1, v[4]); add(P.v_screen.conic + 3 * g + 2, v[5]);
                add(P.v_screen.opac + g, v[6]);
                add(P.v_screen.rgb + 3 * g, v[7]); add(P.v_screen.rgb + 3 * g + 1, v[8]); add(P.v_screen.rgb + 3 * g + 2, v[9]);
            }
        }
        if constexpr (kSums) {   // without gradient rows the weight sums of slot t leave with thread t
            if (!P.v_rows && tid < kB) {
                const float a = s_acc[tid * kCh + 10], b = s_acc[tid * kCh + 11];
                if (a != 0.0f || b != 0.0f) {
                    s_acc[tid * kCh + 10] = 0.0f; s_acc[tid * kCh + 11] = 0.0f;
                    const int64_t wid = accum_row(P, (uint32_t)s_ids[tid]);
                    if (a != 0.0f) atomicAdd(P.accum_weight + wid, a);
                    if (kAccum == SSR_ACCUM_AVG && b != 0.0f) atomicAdd(P.accum_weight + P.num_world + wid, b);
                }
            }
        }
        if constexpr (kAccum == SSR_ACCUM_MAX) {
            if (tid < kB) {
                float mx = 0.0f;
#pragma unroll
                for (int w = 0; w < 4; w++) { mx = ssr_max(mx, s_max[w * kB + tid]); s_max[w * kB + tid] = 0.0f; }
                if (mx > 0.0f) atomic_max_f32(P.accum_weight + accum_row(P, (uint32_t)s_ids[tid]), mx);   // the running maximum starts at 0
            }
        }
        __syncthreads();   // s_ids, frags and s_acc are free for the next batch
    };

    const uint8_t* my_list = s_list + (4 * mt + row) * kB;
    bool first = true;
    // the splat id a thread stages next is read one batch ahead: the fragment gather of the next batch then waits for
    // one memory round trip, not two in a row
    int32_t g_ahead = 0;
    {
        const int32_t idx0 = min(range_end - 1, tile_last) - (tid >= kB ? tid - kB : tid);
        if (idx0 >= range_start && tid < 2 * kB) g_ahead = P.flatten_ids[idx0];
    }
    for (int32_t hi = min(range_end - 1, tile_last); hi >= range_start; hi -= kB) {
        // Explicit wait for this wavefront's LDS traffic (the read-add-writes and float atomics of the walk):
        // the compiler does not place one ahead of this loop-header barrier on the path that leaves the walk,
        // and a pending float atomic is overtaken by the reads that follow the barrier.
        lds_wait();
        __syncthreads();   // previous batch fully consumed (first pass: the zero fill of s_acc is complete)
        if (!first) flush();   // its sums leave before the slots are reused
        first = false;
        bool near_cap = false;   // this thread's fragment can reach the 0.999 cap of alpha
        {
            // slot t holds sorted index hi - t: ascending t is back to front. Thread pair (slot, half) shares the staging.
            const int half = tid >= kB ? 1 : 0, slot = tid - half * kB;   // threads past 2 kB stage nothing
            const int32_t idx = hi - slot;
            uint32_t bits8 = 0;
            if (idx >= range_start && tid < 2 * kB) {
                const int32_t g = g_ahead;
                const FragLds f = stage_fragment_half(P.screen, P.packed_rows, g, tile_x0, tile_y0, half, bits8, P.block_masks ? P.block_masks + idx : nullptr);
                near_cap = f.q1.y >= 0.9989f;
                if (half == 0) {
                    s_ids[slot] = g; frags[slot] = f;
                    // the lower edge of the band around sigma = ln(255 opac) = cut - 1e-3 in which the exact exponential decides
                    frags[slot].q2.z = ssr_max(f.q2.w - 1.008e-3f, 0.0f);
                    if constexpr (kDist != SSR_DIST_NONE) {
                        s_lz[slot] = ssr_log(ssr_max(f.q2.y, 1e-6f));
                        s_iz[slot] = 1.0f / ssr_max(f.q2.y, 1e-6f);   // d/d ln z -> d/dz
                    }
                }
            }
            if (tid < 2 * kB) s_bits[half * kB + slot] = (uint8_t)bits8;
            if (idx - kB >= range_start && tid < 2 * kB) g_ahead = P.flatten_ids[idx - kB];
        }
        // one answer per batch instead of a vote per step: batches without such a fragment (most) walk without the
        // cap's operations
        const bool sat_batch = __syncthreads_or(near_cap ? 1 : 0) != 0;
        // this wavefront's four lists: slots whose block bit is set and whose sorted index hi - slot is
        // not beyond the block's largest last_id
        const int n_batch = min(kB, hi - range_start + 1);
        int cnt[4] = {0, 0, 0, 0};
        if (lane < 4 * kB / 8)   // 8-byte stores blank the wavefront's four lists
            reinterpret_cast<uint64_t*>(s_list + 4 * mt * kB)[lane] = 0x0101010101010101ull * (uint64_t)kB;
        for (int c = 0; c * 64 < n_batch; c++) {
            const int slot = c * 64 + lane;
            const uint32_t bits = slot < kB ? (uint32_t)s_bits[(mt >> 1) * kB + slot] >> (4 * (mt & 1)) : 0u;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const bool in = ((bits >> r) & 1u) != 0 && hi - slot <= blk_last[r];
                const uint64_t bal = __ballot(in);
                if (in) s_list[(4 * mt + r) * kB + cnt[r] + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0u))] = (uint8_t)slot;
                cnt[r] += __builtin_popcountll(bal);
            }
        }
        // the lists are written and read by this wavefront only: order its LDS accesses, no workgroup barrier
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        const int n_steps = max(max(cnt[0], cnt[1]), max(cnt[2], cnt[3]));
        // Steps in which two rows of this wavefront sit on the same fragment: their read-add-writes would
        // overwrite each other, so those steps add atomically. One bit per step, found here (lane = step).
        uint64_t clash_lo = 0, clash_hi = 0;
        {
            const uint8_t* base = s_list + 4 * mt * kB;
#pragma unroll
            for (int c = 0; c < 2; c++) {
                const int stp = c * 64 + lane;
                const int e0 = stp < cnt[0] ? (int)base[stp] : -1, e1 = stp < cnt[1] ? (int)base[kB + stp] : -2,
                          e2 = stp < cnt[2] ? (int)base[2 * kB + stp] : -3, e3 = stp < cnt[3] ? (int)base[3 * kB + stp] : -4;
                const bool cl = (e0 == e1) | (e0 == e2) | (e0 == e3) | (e1 == e2) | (e1 == e3) | (e2 == e3);
                const uint64_t m = (c * 64 < n_steps) ? __ballot(cl) : 0ull;
                if (c == 0) clash_lo = m; else clash_hi = m;
            }
        }
        // One step of a row: fragment k (registers q*) against the row's sixteen pixels.
        const int k_min = hi - bin_final;
        uint64_t clash_run = clash_lo;   // bit 0: the step at hand
        auto step = [&](auto sat_tag, int k, const float4& q0, const float4& q1, const float4& q2w) {
            const float2 q2 = make_float2(q2w.x, q2w.y);
            const float cut = q2w.w;
            constexpr bool kSat = decltype(sat_tag)::value;
            const float dx = q0.x - px, dy = q0.y - py;
            const float sigma = ssr_fma(q0.z * dx, dx, ssr_fma(q1.x * dy, dy, (q0.w * dx) * dy));
            // alpha > 1/255 <=> sigma < ln(255 opac) = cut - 1e-3 (fragment_constants): decided by comparing sigma, except
            // within 8e-6 of that bound, where the rounding of the exponential could decide; there, and where alpha
            // comes within 4e-5 of the 0.999 cap, the wavefront re-evaluates with the bit-defined exponential, so that
            // every decision is the forward's. A lane on a fragment behind its pixel's last one (sorted index
            // hi - k > bin_final) is out; so is the blank fragment past the end of a list (cut 0: no sigma is below).
            const uint32_t lo_bits = __float_as_uint(q2w.z);   // max(cut - 1.008e-3, 0), left there when the fragment was staged
            const bool in_list = k >= k_min;
            const bool below = __float_as_uint(sigma) < lo_bits;      // 0 <= sigma < bound - band
            const uint64_t m_in = __builtin_amdgcn_ballot_w64(in_list), m_lo = __builtin_amdgcn_ballot_w64(below),
                           m_off = __builtin_amdgcn_ballot_w64(sigma > q2w.z + 1.6e-5f);
            bool active = in_list & below;
            float vis = active ? __builtin_amdgcn_exp2f(sigma * -1.44269504088896341f) : 0.0f;
            float ov = q1.y * vis;
            uint64_t unsure = m_in & ~(m_lo | m_off);
            if constexpr (kSat) unsure |= __builtin_amdgcn_ballot_w64(ssr_fabs(ov - 0.999f) <= 4e-5f);
            float alpha = ov;
            if (unsure != 0ull) {   // decisions exactly as the forward took them
                const bool in_range = in_list & !(sigma < 0.f || sigma > cut);
                vis = in_range ? exp_neg_small(-sigma) : 0.0f;
                ov = q1.y * vis;
                // min(0.999, ov) as the one instruction it is (a NaN ov gives 0.999, as ssr_min does); the compiler's own
                // minimum spends a second instruction on quieting a signalling NaN first
                asm("v_min_f32 %0, %1, %2" : "=v"(alpha) : "s"(0.999f), "v"(ov));
                active = alpha > kAlphaThreshold;
                alpha = active ? alpha : 0.0f;
                vis = (active & (ov <= 0.999f)) ? vis : 0.0f;   // evaluate_alpha_vjp gate (src/primitives/Primitive3DGS.cuh:273)
            } else if constexpr (kSat) {
                asm("v_min_f32 %0, %1, %2" : "=v"(alpha) : "s"(0.999f), "v"(ov));
                vis = ov <= 0.999f ? vis : 0.0f;                // the same gate; without a fragment near the cap it never closes
            }
            // no vote on whether any lane is active (a step without one is rare, and the vote costs every step), except
            // with the median, whose step is long enough for the vote to pay
            bool any_active = true;
            if constexpr (kMedian) any_active = __builtin_amdgcn_ballot_w64(active) != 0ull;
            if (any_active) {
                // inactive lanes run with alpha = 0 and vis = 0: T and v_T unchanged, every term zero
                const float a = alpha;
                const float T0 = T1 * __builtin_amdgcn_rcpf(1.0f - a);
                [[maybe_unused]] float v_depth_median = 0.0f;
                if constexpr (kMedian) {   // RasterizationEval3DBwd_kernel.cuh:433-470
                    if (active && pend_Tfar > 0.0f) {   // near member of the crossing found at the previous active splat
                        v_depth_median += pend_zgrad;
                        const float dba = ssr_log(pend_Tfar) - ssr_log(T1);
                        const float inv = (ssr_fabs(dba) > 1e-20f) ? (-1.0f / dba) : 0.0f;
                        vT1 += ((med_v * (pend_zfar - q2.y)) * inv) / T1;
                        pend_Tfar = 0.0f;
                    }
                    if (active && T0 >= 0.5f && T1 < 0.5f) {   // far member: post-splat T drops below 1/2 here
                        const float la = ssr_log(T0), d = ssr_log(T1) - la;
                        const float fr = (ssr_fabs(d) > 1e-20f) ? (-0.6931471805599453f - la) / d : 0.0f;
                        v_depth_median += fr * med_v;
                        pend_zgrad = (1.0f - fr) * med_v;
                        pend_zfar = q2.y;
                        pend_Tfar = T1;
                    }
                }
                const float cr = q1.z, cg = q1.w, cb = q2.x;
                float cdp = q2.y;
                if constexpr (kDist != SSR_DIST_NONE) cdp = s_lz[k];
                float dv = ssr_fma(cdp, vd, ssr_fma(cb, vb, ssr_fma(cg, vg, cr * vr))) - vT1;
                const float w = a * T0;
                [[maybe_unused]] float xr = 0.f, xg = 0.f, xb = 0.f, xd = 0.f;   // distortion part of the colour gradient
                if constexpr (kDist != SSR_DIST_NONE) {   // closed form D = W S - C^2 (:497-517)
                    float gsum = 0.0f;
                    const float w2 = 2.0f * w;
                    if constexpr (kDist == SSR_DIST_RGB_D) {
                        xr = ((cr * Wd - Cr) * vDr) * w2; xg = ((cg * Wd - Cg) * vDg) * w2; xb = ((cb * Wd - Cb) * vDb) * w2;
                        gsum += ((Sr + (cr * cr) * Wd) - (cr * Cr) * 2.0f) * vDr;
                        gsum += ((Sg + (cg * cg) * Wd) - (cg * Cg) * 2.0f) * vDg;
                        gsum += ((Sb + (cb * cb) * Wd) - (cb * Cb) * 2.0f) * vDb;
                    }
                    xd = ((cdp * Wd - Cd) * vDd) * w2;
                    gsum += ((Sd + (cdp * cdp) * Wd) - (cdp * Cd) * 2.0f) * vDd;
                    dv += gsum;   // v_alpha gains T0 g and v_T0 gains alpha g, exactly where dv enters
                }
                const float v_alpha = T0 * dv;   // reaches the sums through vis, which is zero where the gate is closed
                vT1 = ssr_fma(a, dv, vT1);
                T1 = T0;
                const float u = vis * v_alpha;
                const float ux = u * dx, uy = u * dy;
                const float uxx = ux * dx, uxy = ux * dy, uyy = uy * dy;
                float wr = vr * w, wg = vg * w, wb = vb * w, wd = vd * w;
                if constexpr (kDist != SSR_DIST_NONE) {
                    if constexpr (kDist == SSR_DIST_RGB_D) { wr += xr; wg += xg; wb += xb; }
                    wd = (wd + xd) * s_iz[k];
                }
                if constexpr (kMedian) wd += v_depth_median;
                // Channels 0..9 = u, ux, uy, uxx, uxy, uyy, wr, wg, wb, wd. The first two levels of the transposing
                // reduction as bank-masked DPP adds (one instruction per channel and level, against three per pair with
                // selects): lanes 0-7 of a row take the even channel of a pair, lanes 8-15 the odd one; then lane groups
                // of four likewise with the half-mirror pairing. s_nop covers the two wait states a DPP read needs
                // after a write of its source by the instruction before; inside the block the reads trail the writes.
                float r0, r1, r2, r3, r4, s0, s1, s2;
                if constexpr (kSums) {
                    // a sixth pair (map * w, w): its first level joins the others, its second shares s2's instruction
                    // slot pattern (banks 1 and 3), and the quad levels below carry it at no cost
                    const float aw = amap * w;
                    float r5;
                    asm volatile(
                        "s_nop 1\n\t"
                        "v_add_f32_dpp %0, %9, %9 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                        "v_add_f32_dpp %0, %10, %10 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                        "v_add_f32_dpp %1, %11, %11 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                        "v_add_f32_dpp %1, %12, %12 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                        "v_add_f32_dpp %2, %13, %13 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                        "v_add_f32_dpp %2, %14, %14 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                        "v_add_f32_dpp %3, %15, %15 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                        "v_add_f32_dpp %3, %16, %16 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                        "v_add_f32_dpp %4, %17, %17 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                        "v_add_f32_dpp %4, %18, %18 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                        "v_add_f32_dpp %5, %19, %19 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                        "v_add_f32_dpp %5, %20, %20 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                        "v_add_f32_dpp %6, %0, %0 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
                        "v_add_f32_dpp %6, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
                        "v_add_f32_dpp %7, %2, %2 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
                        "v_add_f32_dpp %7, %3, %3 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
                        "v_add_f32_dpp %8, %4, %4 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
                        "v_add_f32_dpp %8, %5, %5 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
                        : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(r4), "=&v"(r5), "=&v"(s0), "=&v"(s1), "=&v"(s2)
                        : "v"(u), "v"(ux), "v"(uy), "v"(uxx), "v"(uxy), "v"(uyy), "v"(wr), "v"(wg), "v"(wb), "v"(wd), "v"(aw), "v"(w));
                } else {
                asm volatile(
                    "s_nop 1\n\t"
                    "v_add_f32_dpp %0, %8, %8 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                    "v_add_f32_dpp %0, %9, %9 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                    "v_add_f32_dpp %1, %10, %10 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                    "v_add_f32_dpp %1, %11, %11 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                    "v_add_f32_dpp %2, %12, %12 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                    "v_add_f32_dpp %2, %13, %13 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                    "v_add_f32_dpp %3, %14, %14 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                    "v_add_f32_dpp %3, %15, %15 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                    "v_add_f32_dpp %4, %16, %16 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
                    "v_add_f32_dpp %4, %17, %17 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
                    "v_add_f32_dpp %5, %0, %0 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
                    "v_add_f32_dpp %5, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
                    "v_add_f32_dpp %6, %2, %2 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
                    "v_add_f32_dpp %6, %3, %3 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
                    "v_add_f32_dpp %7, %4, %4 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
                    : "=&v"(r0), "=&v"(r1), "=&v"(r2), "=&v"(r3), "=&v"(r4), "=&v"(s0), "=&v"(s1), "=&v"(s2)
                    : "v"(u), "v"(ux), "v"(uy), "v"(uxx), "v"(uxy), "v"(uyy), "v"(wr), "v"(wg), "v"(wb), "v"(wd));
                }
                const float t0 = fold_pair<kDppQuadXor2>(s0, s1, b1), t1 = s2 + dpp_full<kDppQuadXor2>(s2);
                const float fin_sum = fold_pair<kDppQuadXor1>(t0, t1, b0);
                const bool mine = (chan >= 0) & ssr_isfinite(fin_sum) & (fin_sum != 0.0f);
                const bool clash = (clash_run & 1ull) != 0;
                float* cell = reinterpret_cast<float*>(my_cells + __umul24((unsigned)k, 4u * kCh));
                if (mine) {
                    if (clash) atomicAdd(cell, fin_sum);
                    else *cell += fin_sum;
                }
                if constexpr (kAccum == SSR_ACCUM_MAX) {   // inactive lanes contribute map * 0
                    float mx = amap * w;
                    mx = ssr_max(mx, dpp_full<0x128>(mx));   // row_ror:8
                    mx = ssr_max(mx, dpp_full<0x141>(mx));   // row_half_mirror
                    mx = ssr_max(mx, dpp_full<kDppQuadXor2>(mx));
                    mx = ssr_max(mx, dpp_full<kDppQuadXor1>(mx));
                    if (l16 == 0 && mx > 0.0f) {   // non-negative floats order as their bit patterns
                        int* mc = reinterpret_cast<int*>(s_max + mt * kB + k);
                        if (clash) atomicMax(mc, __float_as_int(mx));
                        else *mc = max(*mc, __float_as_int(mx));
                    }
                }
            }
        };
        // Software pipeline, two steps per trip: list bytes run two steps ahead of their use and the fragment of the
        // next step loads while the current one computes, so that the two dependent LDS latencies hide behind
        // arithmetic; the two fragment register sets alternate, so nothing is copied between steps.
        auto list_at = [&](int st) { return (int)my_list[st]; };   // past the end: some valid slot, never used
        // slots are below 128: a 24-bit multiply (full rate) addresses the fragment, not the quarter-rate 32-bit one
        auto frag_of = [&](int k) -> const FragLds& {
            return *reinterpret_cast<const FragLds*>(reinterpret_cast<const char*>(frags) + __umul24((unsigned)k, (unsigned)sizeof(FragLds)));
        };
        auto walk = [&](auto sat_tag) {
            int k0 = list_at(0), k1 = list_at(1), k2 = list_at(2);
            float4 a0 = frag_of(k0).q0, a1 = frag_of(k0).q1, a2 = frag_of(k0).q2;
            for (int st = 0; st < n_steps; st += 2) {
                if (st == 64) clash_run = clash_hi;
                const float4 c0 = frag_of(k1).q0, c1 = frag_of(k1).q1, c2 = frag_of(k1).q2;
                const int k3 = list_at(st + 3);
                step(sat_tag, k0, a0, a1, a2);
                clash_run >>= 1;
                a0 = frag_of(k2).q0; a1 = frag_of(k2).q1; a2 = frag_of(k2).q2;
                const int k4 = list_at(st + 4);
                if (st + 1 < n_steps) step(sat_tag, k1, c0, c1, c2);
                clash_run >>= 1;
                k0 = k2; k1 = k3; k2 = k4;
            }
        };
        // (the median variants keep one instantiation, with the cap's operations: two cost them a wavefront per SIMD)
        if constexpr (kMedian) walk(std::true_type{});
        else if (sat_batch) walk(std::true_type{});
        else walk(std::false_type{});
    }
    lds_wait();   // as at the head of the loop
    __syncthreads();
    if (!first) flush();
}


template <int kDist, bool kMedian, int kAccum>
__global__ __launch_bounds__(kRasterBlock) void raster_bwd_rows_kernel(ssr_raster_bwd_params P, int tile_w, int tile_h) {
    raster_bwd_rows_body<kDist, kMedian, kAccum>(P, tile_w, tile_h);
}
// The plain average keeps one register more than five wavefronts per SIMD allow (104 against 102): hold the compiler
// to five, which it reaches without spilling; the other plain instantiations are below the limit already.
__global__ __launch_bounds__(kRasterBlock) __attribute__((amdgpu_waves_per_eu(5))) void raster_bwd_rows_avg_kernel(
    ssr_raster_bwd_params P, int tile_w, int tile_h) {
    raster_bwd_rows_body<SSR_DIST_NONE, false, SSR_ACCUM_AVG>(P, tile_w, tile_h);
}

// The plain median likewise (106 registers without the limit).
__global__ __launch_bounds__(kRasterBlock) __attribute__((amdgpu_waves_per_eu(5))) void raster_bwd_rows_median_kernel(
    ssr_raster_bwd_params P, int tile_w, int tile_h) {
    raster_bwd_rows_body<SSR_DIST_NONE, true, SSR_ACCUM_NONE>(P, tile_w, tile_h);
}

// Moves the weight sums that raster_bwd_rows_kernel left in floats 10 and 11 of the gradient rows to the weight
// arrays: row r belongs to world row accum_row(r); rows of several cameras may share one, hence the atomic.
__global__ __launch_bounds__(256) void accum_from_rows_kernel(ssr_raster_bwd_params P, int avg) {
    const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (r >= P.num_splats) return;
    const float2 ab = *reinterpret_cast<const float2*>(P.v_rows + 12 * r + 10);
    if (ab.x == 0.0f && ab.y == 0.0f) return;
    const int64_t wid = accum_row(P, (uint32_t)r);
    if (ab.x != 0.0f) atomicAdd(P.accum_weight + wid, ab.x);
    if (avg && ab.y != 0.0f) atomicAdd(P.accum_weight + P.num_world + wid, ab.y);
}

}  // namespace ssr

using namespace ssr;

extern "C" int ssr_raster_bwd(const ssr_raster_bwd_params* p, ssr_stream_t stream) {
    SSR_REQUIRE(p, "ssr_raster_bwd", "null params");
    SSR_REQUIRE(p->width > 0 && p->height > 0, "ssr_raster_bwd", "empty image");
    SSR_REQUIRE(p->n_isects >= 0 && p->n_isects < (int64_t)1 << 31, "ssr_raster_bwd", "n_isects out of range");
    SSR_REQUIRE(p->num_splats >= 0 && p->num_splats < ((int64_t)1 << 30), "ssr_raster_bwd", "num_splats must be below 2^30");
    if (p->n_isects == 0) return 0;   // nothing contributed anywhere
    SSR_REQUIRE(p->tile_offsets && p->flatten_ids, "ssr_raster_bwd", "null tile data");
    SSR_REQUIRE(p->render_T && p->last_ids && p->render_depth, "ssr_raster_bwd", "null forward output");
    SSR_REQUIRE(p->v_render_rgb && p->v_render_depth && p->v_render_T, "ssr_raster_bwd", "null output gradient");
    if (p->packed_rows) {
        SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->packed_rows) & 15) == 0, "ssr_raster_bwd", "packed_rows must be 16-byte aligned");
    } else {
        SSR_REQUIRE(p->screen.xy && p->screen.depth && p->screen.conic && p->screen.opac && p->screen.rgb,
                    "ssr_raster_bwd", "null screen buffer");
        SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->screen.xy) & 7) == 0, "ssr_raster_bwd", "screen.xy must be 8-byte aligned");
    }
    SSR_REQUIRE(p->v_rows || (p->v_screen.xy && p->v_screen.depth && p->v_screen.conic && p->v_screen.opac && p->v_screen.rgb),
                "ssr_raster_bwd", "null v_screen buffer");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->v_rows) & 15) == 0, "ssr_raster_bwd", "v_rows must be 16-byte aligned");
    // the variant kernels address a gradient row as 12 * row in 32 bits
    SSR_REQUIRE(!p->v_rows || p->num_splats <= (int64_t)(0xFFFFFFFFu / 12u), "ssr_raster_bwd", "with v_rows, num_splats must not exceed 357913941");
    SSR_REQUIRE(p->dist_type >= SSR_DIST_NONE && p->dist_type <= SSR_DIST_RGB_D, "ssr_raster_bwd",
                "dist_type must be NONE, D or RGB_D (the 3dgs pixel has no normal channel)");
    if (p->dist_type != SSR_DIST_NONE)
        SSR_REQUIRE(p->distortion_depth && p->v_distortion_depth, "ssr_raster_bwd", "null depth distortion image or cotangent");
    if (p->dist_type == SSR_DIST_RGB_D)
        SSR_REQUIRE(p->render_rgb && p->distortion_rgb && p->v_distortion_rgb, "ssr_raster_bwd", "null rgb distortion input");
    SSR_REQUIRE(p->accum_mode >= SSR_ACCUM_NONE && p->accum_mode <= SSR_ACCUM_AVG, "ssr_raster_bwd", "unknown accum_mode");
    SSR_REQUIRE(p->schedule == SSR_BWD_SCHEDULE_ROWS || p->schedule == SSR_BWD_SCHEDULE_LANES, "ssr_raster_bwd", "unknown schedule");
    if (p->accum_mode != SSR_ACCUM_NONE) {
        SSR_REQUIRE(p->accum_weight_map && p->accum_weight, "ssr_raster_bwd", "null accumulation buffer");
        SSR_REQUIRE(p->num_world > 0, "ssr_raster_bwd", "num_world must be positive");
    }
    const int tw = (int)ceil_div(p->width, kTile), th = (int)ceil_div(p->height, kTile);
    SSR_REQUIRE(p->num_images >= 0, "ssr_raster_bwd", "negative num_images");
    const int nimg = p->num_images > 1 ? p->num_images : 1;
    SSR_REQUIRE((int64_t)tw * th * nimg < (int64_t)1 << 30, "ssr_raster_bwd", "too many tiles");
    SSR_REQUIRE(nimg == 1 || p->accum_mode == SSR_ACCUM_NONE || p->gaussian_ids ||
                    (p->num_world < ((int64_t)1 << 31) && p->num_splats == nimg * p->num_world),
                "ssr_raster_bwd", "several images accumulate per world row: num_splats must be num_images * num_world (or gaussian_ids given)");
    const dim3 grid((unsigned)xcd_grid_size(tw * th * nimg)), block(kRasterBlock);
    hipStream_t st = as_stream(stream);
    const bool med = p->v_render_median != nullptr;
#define SSR_ROWS(D, M, A) hipLaunchKernelGGL((raster_bwd_rows_kernel<D, M, A>), grid, block, 0, st, *p, tw, th)
#define SSR_ROWS_A(D, M)                                          \
    switch (p->accum_mode) {                                      \
        case SSR_ACCUM_MAX: SSR_ROWS(D, M, SSR_ACCUM_MAX); break;   \
        case SSR_ACCUM_SUM: SSR_ROWS(D, M, SSR_ACCUM_SUM); break;   \
        case SSR_ACCUM_AVG: SSR_ROWS(D, M, SSR_ACCUM_AVG); break;   \
        default: SSR_ROWS(D, M, SSR_ACCUM_NONE); break;             \
    }
#define SSR_ROWS_M(D) if (med) { SSR_ROWS_A(D, true) } else { SSR_ROWS_A(D, false) }
    // the lane-per-fragment cut covers the plain backward and, where the gradient rows carry them out, the weight sums
    const bool sums = p->accum_mode == SSR_ACCUM_SUM || p->accum_mode == SSR_ACCUM_AVG;
    if (p->schedule == SSR_BWD_SCHEDULE_LANES && p->dist_type == SSR_DIST_NONE && !med &&
        (p->accum_mode == SSR_ACCUM_NONE || (sums && p->v_rows)))
        launch_raster_bwd_lanes(*p, tw, th, nimg, st);
    else if (p->dist_type == SSR_DIST_NONE && !med && p->accum_mode == SSR_ACCUM_AVG)
        hipLaunchKernelGGL(raster_bwd_rows_avg_kernel, grid, block, 0, st, *p, tw, th);
    else if (p->dist_type == SSR_DIST_NONE && med && p->accum_mode == SSR_ACCUM_NONE)
        hipLaunchKernelGGL(raster_bwd_rows_median_kernel, grid, block, 0, st, *p, tw, th);
    else switch (p->dist_type) {
        case SSR_DIST_D: SSR_ROWS_M(SSR_DIST_D); break;
        case SSR_DIST_RGB_D: SSR_ROWS_M(SSR_DIST_RGB_D); break;
        default: SSR_ROWS_M(SSR_DIST_NONE); break;
    }
#undef SSR_ROWS_M
#undef SSR_ROWS_A
#undef SSR_ROWS
    if (p->v_rows && (p->accum_mode == SSR_ACCUM_SUM || p->accum_mode == SSR_ACCUM_AVG))
        hipLaunchKernelGGL(accum_from_rows_kernel, dim3((unsigned)ceil_div(p->num_splats, 256)), dim3(256), 0, st, *p,
                           p->accum_mode == SSR_ACCUM_AVG ? 1 : 0);
    SSR_CHECK_LAUNCH("ssr_raster_bwd");
    return 0;
}
