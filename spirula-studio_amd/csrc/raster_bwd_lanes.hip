// raster_bwd_lanes.hip -- K8 without distortion or median (plain, or with the loss-map weight sums of
// accum_mode SUM / AVG, RasterizationEval3DBwd_kernel.cuh:520-538), with one LANE PER FRAGMENT: the same sums as raster_bwd.hip (rasterize_to_pixels_bwd_kernel,
// src/kernels/raster/RasterizationEval3DBwd_kernel.cuh:423-494 with the fragment VJPs of
// src/primitives/Primitive3DGS.cuh:262-300), cut differently.
//
// raster_bwd.hip gives a 16-lane row one fragment and sixteen pixels a step and then has to add ten values over
// those sixteen lanes, every step. Here a row holds SIXTEEN CONSECUTIVE FRAGMENTS of a 4x4-pixel block's list, one a
// lane, and the four rows of the wavefront hold the block's four pixel rows: lane (r, f) takes fragment f against
// pixels (r, 0..3), one after the other. Per pixel the recursions along the list become scans over the row's lanes:
//   T before fragment f   = T_behind / prod_{j <= f} (1 - alpha_j)                 (inclusive product scan)
//   v_T after fragment f  = (1 - alpha_f) v_T(f - 1) + alpha_f (c_f . v_c)          (affine scan, same products)
// both as DPP row shifts (four levels), the block's pixel state (T, v_T per pixel) travelling from chunk to chunk as a
// broadcast of lane 15. The ten sums of a fragment then accumulate in the lane's own registers over its four pixels;
// what is left of the reduction is the sum over the four rows, once per sixteen fragments, by a transposing
// exchange (v_permlane16_swap / v_permlane32_swap) that leaves every lane one finished channel of its own fragment.
// A wavefront walks the four blocks of its 8x8 sub-tile one after the other; pixel state rests in LDS in between.
//
// Decisions are the forward's: sigma is formed by the forward's own operations, and a lane whose sigma is within
// 8e-6 of ln(255 opac) (or whose alpha is within 4e-5 of 0.999) makes the wavefront re-evaluate that pixel with the
// bit-defined exponential; everywhere else alpha > 1/255 is decided by comparing sigma, and exp comes from the
// hardware.
#include <type_traits>

#include "raster_device.h"

namespace ssr {

constexpr int kChunk = 16;         // fragments per row and chunk

// kLB fragments staged per batch; kLCh channels per fragment: u, u dx, u dy, u dx^2, u dx dy, u dy^2, w_r, w_g, w_b,
// w_d and, with the weight sums, map * w and w. The sums' two channels are paid for with a shorter batch, so that four
// workgroups still share a compute unit's LDS.
template <int kLB, int kLCh, bool kSums>
struct LanesShared {
    FragLds frags[kLB + 1];        // the last one is the blank fragment behind every list
    int32_t ids[kLB];
    float acc[(4 * kLB + 1) * kLCh];   // per wavefront and slot; the last row takes what blank fragments add (zeros)
    uint8_t bits[2 * kLB];
    __attribute__((aligned(16))) uint8_t list[kBlocksPerTile * kLB];
    // pixel state, index = 16 * block + 4 * row + column = thread id of the pixel's owner at set-up
    __attribute__((aligned(16))) float T[256];
    __attribute__((aligned(16))) float vT[256];
    __attribute__((aligned(16))) int32_t last[256];
    float4 v[256];                 // v_r, v_g, v_b, v_depth / W
    float amap[kSums ? 256 : 1];   // the loss map's pixels (weight sums)
    int wave_max[4];
    int cnt[kBlocksPerTile];       // list lengths of the batch
    int next;                      // next block to hand out
};

template <bool kSums>
__global__ __launch_bounds__(kRasterBlock) __attribute__((amdgpu_waves_per_eu(4, 4))) void raster_bwd_lanes_kernel(ssr_raster_bwd_params P, int tile_w, int tile_h) {
    constexpr int kLB = kSums ? 112 : 128, kLCh = kSums ? 12 : 10;
    static_assert(kLB % kChunk == 0 && 2 * kLB <= kRasterBlock && kLB <= 255, "two staging threads per slot; slot numbers and the blank's are bytes");
    __shared__ LanesShared<kLB, kLCh, kSums> S;
    const int n_tiles = tile_w * tile_h * (P.num_images > 1 ? P.num_images : 1);
    const int tile = tile_of_workgroup(P.tile_order, blockIdx.x, n_tiles);
    if (tile < 0 || tile >= n_tiles) return;
    const int tid = threadIdx.x, lane = tid & 63, mt = tid >> 6, row = lane >> 4, l16 = lane & 15;
    const int gy = tile / tile_w, tx = tile - gy * tile_w;
    const int img = gy / tile_h, ty = gy - img * tile_h;
    const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);
    // the tile's range is asked for here, with the pixel state: behind the barrier below it would be one more memory
    // round trip in the chain order -> range -> ids -> rows that every tile starts with
    const int32_t range_start = P.tile_offsets[tile];
    const int32_t range_end = (tile == n_tiles - 1 && !P.tile_offsets_closed) ? (int32_t)P.n_isects : P.tile_offsets[tile + 1];
    int wave_last;
    int blk_last[4];
    {   // set-up: thread = pixel (block `row` of sub-tile mt, pixel l16 of the block), as in raster_bwd.hip
        const int j = tx * kTile + (mt & 1) * kMicro + (row & 1) * kBlock + (l16 & 3);
        const int i = ty * kTile + (mt >> 1) * kMicro + (row >> 1) * kBlock + (l16 >> 2);
        const bool inside = (uint32_t)i < P.height && (uint32_t)j < P.width;
        const int64_t pid = ((int64_t)img * P.height + i) * P.width + j;
        const int32_t bin_final = inside ? P.last_ids[pid] : -1;
        const float T1 = inside ? P.render_T[pid] : 0.0f;
        float vT1 = inside ? P.v_render_T[pid] : 0.0f;
        float vr = 0.f, vg = 0.f, vb = 0.f, vd = 0.f;
        if (inside) {
            const float* v = P.v_render_rgb + 3 * pid;
            vr = v[0]; vg = v[1]; vb = v[2];
            vd = P.v_render_depth[pid];
        }
        const float inv_alpha = 1.0f / ssr_max(1.0f - T1, 1e-10f);
        const float out_depth = inside ? P.render_depth[pid] : 0.0f;
        vT1 = vT1 + (out_depth * vd) * inv_alpha;
        vd = vd * inv_alpha;
        S.T[tid] = T1; S.vT[tid] = vT1; S.last[tid] = bin_final; S.v[tid] = make_float4(vr, vg, vb, vd);
        if constexpr (kSums) S.amap[tid] = inside ? P.accum_weight_map[pid] : 0.0f;
        int row_last = bin_final;
#pragma unroll
        for (int d = 8; d >= 1; d >>= 1) row_last = max(row_last, __shfl_xor(row_last, d, 16));
        blk_last[0] = __builtin_amdgcn_readlane(row_last, 0); blk_last[1] = __builtin_amdgcn_readlane(row_last, 16);
        blk_last[2] = __builtin_amdgcn_readlane(row_last, 32); blk_last[3] = __builtin_amdgcn_readlane(row_last, 48);
        wave_last = max(max(blk_last[0], blk_last[1]), max(blk_last[2], blk_last[3]));
        if (lane == 0) S.wave_max[mt] = wave_last;
    }
    for (int e = tid; e < (4 * kLB + 1) * kLCh; e += kRasterBlock) S.acc[e] = 0.0f;
    if (tid == 0) {
        const float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
        S.frags[kLB].q0 = z; S.frags[kLB].q1 = z; S.frags[kLB].q2 = z;
    }
    __syncthreads();
    const int tile_last = max(max(S.wave_max[0], S.wave_max[1]), max(S.wave_max[2], S.wave_max[3]));

    // Thread pairs own a slot: they add up the four wavefronts' sums, turn moments into the ten gradient channels
    // (x, y, depth, conic[3], opac, rgb[3]) and leave them in the first copy; then all threads move the batch to
    // global memory in the order of the destination rows (raster_bwd.hip does the same).
    auto flush = [&]() {
        if ((tid >> 1) < kLB) {
            const int slot = tid >> 1;
            const bool geom = (tid & 1) == 0;
            float m[6] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            const int c0 = geom ? 0 : 6, nc = geom ? 6 : kLCh - 6;
#pragma unroll
            for (int w = 0; w < 4; w++)
#pragma unroll
                for (int c = 0; c < 6; c++)
                    if (c < nc) m[c] += S.acc[(w * kLB + slot) * kLCh + c0 + c];
#pragma unroll
            for (int w = 1; w < 4; w++)
#pragma unroll
                for (int c = 0; c < 6; c++)
                    if (c < nc) S.acc[(w * kLB + slot) * kLCh + c0 + c] = 0.0f;
            float o[6];
            if (geom) {
                const float4 q0 = S.frags[slot].q0, q1 = S.frags[slot].q1;
                const float k = -q1.y;                       // v_sigma = -(opac vis) v_alpha = k u
                const float sx = k * m[1], sy = k * m[2];
                o[0] = ssr_fma(q0.z + q0.z, sx, q0.w * sy);
                o[1] = ssr_fma(q0.w, sx, (q1.x + q1.x) * sy);
                o[2] = (0.5f * k) * m[3]; o[3] = k * m[4]; o[4] = (0.5f * k) * m[5];
                o[5] = m[0];
            } else {
                o[0] = m[3]; o[1] = m[0]; o[2] = m[1]; o[3] = m[2]; o[4] = 0.f; o[5] = 0.f;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");   // the pair's reads above before its writes below
            __builtin_amdgcn_wave_barrier();
            float* dst = S.acc + slot * kLCh;
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
        lds_barrier();
        if (P.v_rows) {
            for (int e = tid; e < kLB * kLCh; e += kRasterBlock) {
                const int slot = e / kLCh, ch = e - slot * kLCh;
                const float x = S.acc[e];
                if (x != 0.0f) {
                    S.acc[e] = 0.0f;
                    atomicAdd(P.v_rows + (int64_t)12 * S.ids[slot] + ch, x);
                }
            }
        } else if (tid < kLB) {
            float v[10];
            bool any = false;
#pragma unroll
            for (int c = 0; c < 10; c++) { v[c] = S.acc[tid * kLCh + c]; any |= v[c] != 0.0f; }
            if (any) {
#pragma unroll
                for (int c = 0; c < 10; c++) S.acc[tid * kLCh + c] = 0.0f;
                const int64_t g = S.ids[tid];
                auto add = [](float* p, float x) { if (x != 0.0f) atomicAdd(p, x); };
                add(P.v_screen.xy + 2 * g, v[0]); add(P.v_screen.xy + 2 * g + 1, v[1]);
                add(P.v_screen.depth + g, v[2]);
                add(P.v_screen.conic + 3 * g, v[3]); add(P.v_screen.conic + 3 * g + 1, v[4]); add(P.v_screen.conic + 3 * g + 2, v[5]);
                add(P.v_screen.opac + g, v[6]);
                add(P.v_screen.rgb + 3 * g, v[7]); add(P.v_screen.rgb + 3 * g + 1, v[8]); add(P.v_screen.rgb + 3 * g + 2, v[9]);
            }
        }
        lds_barrier();
    };

    float* const my_acc = S.acc + mt * (kLB * kLCh);
    float* const dump = S.acc + 4 * kLB * kLCh;
    bool first = true;
    int32_t g_ahead = 0;
    {
        const int32_t idx0 = min(range_end - 1, tile_last) - (tid >= kLB ? tid - kLB : tid);
        if (idx0 >= range_start && tid < 2 * kLB) g_ahead = P.flatten_ids[idx0];
    }
    for (int32_t hi = min(range_end - 1, tile_last); hi >= range_start; hi -= kLB) {
        lds_wait();
        __syncthreads();   // previous batch fully consumed (and, this once per batch, memory operations complete)
        if (!first) flush();
        first = false;
        if (tid == 0) S.next = 0;
        if (tid < 2 * kLB) {
            const int half = tid >= kLB ? 1 : 0, slot = tid - half * kLB;
            const int32_t idx = hi - slot;
            uint32_t bits8 = 0;
            if (idx >= range_start) {
                const int32_t g = g_ahead;
                const FragLds f = stage_fragment_half(P.screen, P.packed_rows, g, tile_x0, tile_y0, half, bits8, P.block_masks ? P.block_masks + idx : nullptr);
                if (half == 0) { S.ids[slot] = g; S.frags[slot] = f; }
            }
            S.bits[half * kLB + slot] = (uint8_t)bits8;
            if (idx - kLB >= range_start) g_ahead = P.flatten_ids[idx - kLB];
        }
        lds_barrier();
        const int n_batch = min(kLB, hi - range_start + 1);
        int cnt[4] = {0, 0, 0, 0};
        if (lane < 4 * kLB / 8)   // 8-byte stores blank the wavefront's four lists
            reinterpret_cast<uint64_t*>(S.list + 4 * mt * kLB)[lane] = 0x0101010101010101ull * (uint64_t)kLB;
        for (int c = 0; c * 64 < n_batch; c++) {
            const int slot = c * 64 + lane;
            const uint32_t bits = slot < kLB ? (uint32_t)S.bits[(mt >> 1) * kLB + slot] >> (4 * (mt & 1)) : 0u;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const bool in = ((bits >> r) & 1u) != 0 && hi - slot <= blk_last[r];
                const uint64_t bal = __ballot(in);
                if (in) S.list[(4 * mt + r) * kLB + cnt[r] + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0u))] = (uint8_t)slot;
                cnt[r] += __builtin_popcountll(bal);
            }
        }
        if (lane < 4) S.cnt[4 * mt + lane] = lane == 0 ? cnt[0] : lane == 1 ? cnt[1] : lane == 2 ? cnt[2] : cnt[3];
        lds_barrier();   // every list of the tile is built

        // ---- the walk: the sixteen blocks are dealt to the wavefronts as they become free (a sub-tile's four blocks
        // can hold most of a tile's work); this lane = (pixel row `row` of the block, list position l16) ----
        for (;;) {
            int blk = 0;
            if (lane == 0) blk = atomicAdd(&S.next, 1);
            blk = __builtin_amdgcn_readfirstlane(blk);
            if (blk >= kBlocksPerTile) break;
            const int n_list = S.cnt[blk];
            if (n_list == 0) continue;
            const int bm = blk >> 2, q = blk & 3;   // sub-tile and quadrant of the block
            const int blk_pix = blk * 16;
            const int pix0 = blk_pix + 4 * row;                // this lane's four pixels: pix0 + 0..3
            float4 Tq = *reinterpret_cast<const float4*>(S.T + pix0);
            float4 vTq = *reinterpret_cast<const float4*>(S.vT + pix0);
            const int4 lastq = *reinterpret_cast<const int4*>(S.last + pix0);
            float Tc[4] = {Tq.x, Tq.y, Tq.z, Tq.w}, vTc[4] = {vTq.x, vTq.y, vTq.z, vTq.w};
            const int lastc[4] = {lastq.x, lastq.y, lastq.z, lastq.w};
            const float4 vc[4] = {S.v[pix0], S.v[pix0 + 1], S.v[pix0 + 2], S.v[pix0 + 3]};
            [[maybe_unused]] float4 am = make_float4(0.f, 0.f, 0.f, 0.f);
            if constexpr (kSums) am = *reinterpret_cast<const float4*>(S.amap + pix0);
            const float px0 = tile_x0 + (float)((bm & 1) * kMicro + (q & 1) * kBlock) + 0.5f;
            const float py = tile_y0 + (float)((bm >> 1) * kMicro + (q >> 1) * kBlock + row) + 0.5f;
            const uint8_t* lst = S.list + blk * kLB + l16;
#pragma unroll 1
            for (int ch = 0; ch < n_list; ch += kChunk) {
                const int slot = (int)lst[ch];
                const char* fp = reinterpret_cast<const char*>(S.frags) + __umul24((unsigned)slot, (unsigned)sizeof(FragLds));
                const FragLds& F = *reinterpret_cast<const FragLds*>(fp);
                const float4 q0 = F.q0, q1 = F.q1;
                const float2 q2 = make_float2(F.q2.x, F.q2.y);
                const float cz = q1.x, opac = q1.y, cut = F.q2.w;
                const int idx = hi - slot;
                // alpha > 1/255 <=> sigma < ln(255 opac) = cut - 1e-3 (fragment_constants); the band around it in
                // which the exponential's rounding could decide is +-8e-6
                const uint32_t lo_bits = __float_as_uint(ssr_max(cut - 1.008e-3f, 0.0f));
                const float hi_thr = cut - 0.992e-3f;
                const bool sat_possible = __builtin_amdgcn_ballot_w64(opac >= 0.9989f) != 0ull;
                // kSat: some fragment of the chunk can reach alpha = 0.999, where alpha is capped and the gradient of
                // the exponent gated (Primitive3DGS.cuh:258,273); chunks without one leave those operations out
                auto chunk = [&](auto sat_tag) {
                constexpr bool kSat = decltype(sat_tag)::value;
                const float dy = q0.y - py;
                const float ty2 = cz * dy;
                float gq[4];   // c_f . v_c
#pragma unroll
                for (int c = 0; c < 4; c++)
                    gq[c] = ssr_fma(q2.y, vc[c].w, ssr_fma(q2.x, vc[c].z, ssr_fma(q1.w, vc[c].y, q1.z * vc[c].x)));
                float a[4], visu[4], dx[4], om[4], bk[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    dx[c] = q0.x - (px0 + (float)c);
                    const float sigma = ssr_fma(q0.z * dx[c], dx[c], ssr_fma(ty2, dy, (q0.w * dx[c]) * dy));
                    const float e = __builtin_amdgcn_exp2f(sigma * -1.44269504088896341f);
                    const uint64_t m_in = __builtin_amdgcn_ballot_w64(idx <= lastc[c]);
                    const uint64_t m_lo = __builtin_amdgcn_ballot_w64(__float_as_uint(sigma) < lo_bits);   // 0 <= sigma < ln(255 opac) - band
                    const uint64_t m_off = __builtin_amdgcn_ballot_w64(sigma > hi_thr);                    // beyond the band, or no opacity
                    uint64_t unsure = m_in & ~(m_lo | m_off);
                    float vis = ((idx <= lastc[c]) & (__float_as_uint(sigma) < lo_bits)) ? e : 0.0f;
                    float al = opac * vis;
                    if constexpr (kSat) unsure |= __builtin_amdgcn_ballot_w64(ssr_fabs(al - 0.999f) <= 4e-5f);
                    if (unsure != 0ull) {   // decide exactly as the forward did
                        const bool in_range = (idx <= lastc[c]) & !(sigma < 0.f || sigma > cut);
                        const float ve = in_range ? exp_neg_small(-sigma) : 0.0f;
                        const float ov = opac * ve;
                        float amin;
                        asm("v_min_f32 %0, %1, %2" : "=v"(amin) : "s"(0.999f), "v"(ov));
                        const bool act = amin > kAlphaThreshold;
                        al = act ? amin : 0.0f;
                        vis = (act & (ov <= 0.999f)) ? ve : 0.0f;   // evaluate_alpha_vjp gate (Primitive3DGS.cuh:273)
                    } else if constexpr (kSat) {
                        const float ov = al;
                        asm("v_min_f32 %0, %1, %2" : "=v"(al) : "s"(0.999f), "v"(ov));
                        vis = ov <= 0.999f ? vis : 0.0f;
                    }
                    a[c] = al; visu[c] = vis;
                    om[c] = 1.0f - al;
                    bk[c] = al * gq[c];
                }
                // inclusive scans along the row: om -> products P, bk -> B with v_T(f) = P(f) v_T(behind) + B(f)
                asm volatile(
                    "s_nop 1\n\t"
#define SSR_SCAN_LEVEL(S_)                                                                 \
                    "v_fmac_f32_dpp %4, %4, %0 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t" \
                    "v_mul_f32_dpp %0, %0, %0 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t"  \
                    "v_fmac_f32_dpp %5, %5, %1 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t" \
                    "v_mul_f32_dpp %1, %1, %1 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t"  \
                    "v_fmac_f32_dpp %6, %6, %2 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t" \
                    "v_mul_f32_dpp %2, %2, %2 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t"  \
                    "v_fmac_f32_dpp %7, %7, %3 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t" \
                    "v_mul_f32_dpp %3, %3, %3 row_shr:" #S_ " row_mask:0xf bank_mask:0xf\n\t"
                    SSR_SCAN_LEVEL(1) SSR_SCAN_LEVEL(2) SSR_SCAN_LEVEL(4) SSR_SCAN_LEVEL(8)
#undef SSR_SCAN_LEVEL
                    : "+v"(om[0]), "+v"(om[1]), "+v"(om[2]), "+v"(om[3]), "+v"(bk[0]), "+v"(bk[1]), "+v"(bk[2]), "+v"(bk[3]));
                float vT0[4], vT1[4], T0[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    vT0[c] = ssr_fma(om[c], vTc[c], bk[c]);
                    vT1[c] = vTc[c];
                    T0[c] = Tc[c] * __builtin_amdgcn_rcpf(om[c]);
                }
                // v_T in front of this lane's fragment = v_T behind its neighbour's; the pixel state for the next chunk
                // = lane 15's
                asm volatile(
                    "s_nop 1\n\t"
                    "v_mov_b32_dpp %0, %4 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %1, %5 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %2, %6 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %3, %7 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
                    : "+v"(vT1[0]), "+v"(vT1[1]), "+v"(vT1[2]), "+v"(vT1[3])
                    : "v"(vT0[0]), "v"(vT0[1]), "v"(vT0[2]), "v"(vT0[3]));
                asm volatile(
                    "s_nop 1\n\t"
                    "v_mov_b32_dpp %0, %8 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %1, %9 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %2, %10 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %3, %11 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %4, %12 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %5, %13 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %6, %14 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    "v_mov_b32_dpp %7, %15 row_newbcast:15 row_mask:0xf bank_mask:0xf\n\t"
                    : "=&v"(Tc[0]), "=&v"(Tc[1]), "=&v"(Tc[2]), "=&v"(Tc[3]), "=&v"(vTc[0]), "=&v"(vTc[1]), "=&v"(vTc[2]), "=&v"(vTc[3])
                    : "v"(T0[0]), "v"(T0[1]), "v"(T0[2]), "v"(T0[3]), "v"(vT0[0]), "v"(vT0[1]), "v"(vT0[2]), "v"(vT0[3]));
                // per-lane sums over the four pixels of the row (the colour sums go through the matrix unit pixel by pixel)
                float u[4], ux[4], w[4];
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const float dv = gq[c] - vT1[c];
                    u[c] = visu[c] * (T0[c] * dv);
                    ux[c] = u[c] * dx[c];
                    w[c] = a[c] * T0[c];
                }
                const float U = (u[0] + u[1]) + (u[2] + u[3]), V1 = (ux[0] + ux[1]) + (ux[2] + ux[3]);
                const float V2 = ssr_fma(ux[3], dx[3], ssr_fma(ux[2], dx[2], ssr_fma(ux[1], dx[1], ux[0] * dx[0])));
                const float Wr = ssr_fma(vc[3].x, w[3], ssr_fma(vc[2].x, w[2], ssr_fma(vc[1].x, w[1], vc[0].x * w[0])));
                const float Wg = ssr_fma(vc[3].y, w[3], ssr_fma(vc[2].y, w[2], ssr_fma(vc[1].y, w[1], vc[0].y * w[0])));
                const float Wb = ssr_fma(vc[3].z, w[3], ssr_fma(vc[2].z, w[2], ssr_fma(vc[1].z, w[1], vc[0].z * w[0])));
                const float Wd = ssr_fma(vc[3].w, w[3], ssr_fma(vc[2].w, w[2], ssr_fma(vc[1].w, w[1], vc[0].w * w[0])));
                const float Uy = U * dy;
                // the sum over the four pixel rows: channels in pairs through v_permlane16_swap (rows 0<->1, 2<->3), the
                // pair sums in pairs through v_permlane32_swap; row r of R0 / R1 / R2 then holds channel r / 4 + r / 8 + r
                auto fold16 = [](float x, float y) {
                    const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(y), false, false);
                    return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
                };
                auto fold32 = [](float x, float y) {
                    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(y), false, false);
                    return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
                };
                const float R0 = fold32(fold16(U, V1), fold16(Uy, V2));                 // u, u dx, u dy, u dx^2
                const float R1 = fold32(fold16(V1 * dy, Uy * dy), fold16(Wr, Wg));      // u dx dy, u dy^2, w_r, w_g
                float* cell = (slot < kLB ? my_acc + __umul24((unsigned)slot, (unsigned)kLCh) : dump) + row;
                if constexpr (kSums) {   // rows 2 and 3 of the third register carry the weight sums: map * w and w
                    const float Wa = ssr_fma(am.w, w[3], ssr_fma(am.z, w[2], ssr_fma(am.y, w[1], am.x * w[0])));
                    const float Ww = (w[0] + w[1]) + (w[2] + w[3]);
                    const float R2 = fold32(fold16(Wb, Wd), fold16(Wa, Ww));
                    cell[0] += R0; cell[4] += R1; cell[8] += R2;
                } else {
                    const float R2 = fold32(fold16(Wb, Wd), 0.0f);                      // w_b, w_d (rows 0, 1)
                    cell[0] += R0; cell[4] += R1;
                    if (row < 2) cell[8] += R2;
                }
                };
                if (sat_possible) chunk(std::true_type{}); else chunk(std::false_type{});
            }
            // lane 0 of each row returns the block's pixel state
            if (l16 == 0) {
                *reinterpret_cast<float4*>(S.T + pix0) = make_float4(Tc[0], Tc[1], Tc[2], Tc[3]);
                *reinterpret_cast<float4*>(S.vT + pix0) = make_float4(vTc[0], vTc[1], vTc[2], vTc[3]);
            }
        }
    }
    lds_wait();
    __syncthreads();
    if (!first) flush();
}

int launch_raster_bwd_lanes(const ssr_raster_bwd_params& p, int tw, int th, int nimg, hipStream_t st) {
    const dim3 grid((unsigned)xcd_grid_size(tw * th * nimg)), block(kRasterBlock);
    if (p.accum_mode == SSR_ACCUM_SUM || p.accum_mode == SSR_ACCUM_AVG)
        hipLaunchKernelGGL(raster_bwd_lanes_kernel<true>, grid, block, 0, st, p, tw, th);
    else
        hipLaunchKernelGGL(raster_bwd_lanes_kernel<false>, grid, block, 0, st, p, tw, th);
    return 0;
}

}  // namespace ssr
