// raster_fwd.hip -- K7: per-tile front-to-back alpha compositing.
//
// Follows rasterize_to_pixels_fwd_kernel with IS_EVAL3D=0, dist_type=None, no median
// (src/kernels/raster/RasterizationEval3DFwd_kernel.cuh:48-313): per pixel, for each splat of the
// tile's sorted range whose footprint reaches the pixel's 8x8 sub-tile: alpha = min(0.999,
// opac*exp(-sigma)); skip alpha <= 1/255; T' = T(1-alpha); if T' <= 1e-4 the pixel is finished
// WITHOUT adding this splat; else accumulate rgb*alpha*T, depth*alpha*T and remember the sorted
// index. Outputs rgb, depth / max(1-T, 1e-10), T and last_id.
#include "raster_device.h"

namespace ssr {

// One workgroup per 16x16 tile, a wavefront per 8x8 sub-tile; each 16-lane row of a wavefront holds one 4x4-pixel
// block and walks its own list of the staged fragments whose block bit is set (raster_device.h), so that lanes do
// not visit fragments that only reach other parts of the sub-tile. Lists are built per batch by the wavefront that
// walks them (ballot + rank, slot numbers as bytes). kDist (SSR_DIST_*) and kMedian select the variants
// (RasterizationEval3DFwd_kernel.cuh:143-148,245-307): per-lane accumulators only.
template <int kDist, bool kMedian>
__global__ __launch_bounds__(kRasterBlock) void raster_fwd_rows_kernel(ssr_raster_fwd_params P, int tile_w, int tile_h) {
    // slot kBatch is a fragment of opacity zero: a list is padded with it up to the wavefront's step count, so that
    // a step needs no test of its own for the end of its list
    __shared__ FragLds frags[kBatch + 1];
    // distortion composites ln(max(z, 1e-6)): a per-splat value, taken once when the fragment is staged (kept at the
    // fragments' pitch, so that a list entry addresses it without a division)
    [[maybe_unused]] __shared__ float s_lz[kDist != SSR_DIST_NONE ? (kBatch + 1) * 12 : 1];
    // list entries are the fragments' byte offsets in `frags` (slot * 48 fits sixteen bits)
    __shared__ uint16_t s_list[kBlocksPerTile * kBatch + 16];
    static_assert(sizeof(FragLds) == 48 && kBatch * 48 < 65536, "list entries are 16-bit byte offsets of 48-byte fragments");
    constexpr uint32_t kPadEntry = kBatch * 48;
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

    const int32_t range_start = P.tile_offsets[tile];
    const int32_t range_end = (tile == n_tiles - 1 && !P.tile_offsets_closed) ? (int32_t)P.n_isects : P.tile_offsets[tile + 1];
    // The pixel's transmittance twice: T is the value that goes out; Tl is the same while the pixel composites and 0
    // once it has stopped (or lies outside the image). A step then needs no flag: from Tl = 0 every product is 0,
    // nothing passes the transmittance test and nothing is added.
    float T = 1.0f, Tl = inside ? 1.0f : 0.0f, cr = 0.f, cg = 0.f, cb = 0.f, cd = 0.f;
    [[maybe_unused]] float s2r = 0.f, s2g = 0.f, s2b = 0.f, s2d = 0.f;           // second moments (distortion)
    [[maybe_unused]] float median = 0.f, med_prev_z = 0.f, med_prev_T = 1.0f;   // median depth
    uint32_t cur_idx = 0;
    const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);
    const uint16_t* my_list = s_list + (4 * mt + row) * kBatch;
    // list entries are read a few steps ahead without asking whether the list reaches that far: every entry is a valid
    // offset from the start (the first barrier of the batch loop orders this with the first reads)
    for (int e = tid; e < (int)(sizeof(s_list) / sizeof(s_list[0])); e += kRasterBlock) s_list[e] = 0;
    if (tid < 3) (&frags[kBatch].q0)[tid] = make_float4(0.f, 0.f, 0.f, 0.f);
    if constexpr (kDist != SSR_DIST_NONE) { if (tid == 0) s_lz[kBatch * 12] = 0.0f; }

    // the splat id a thread stages next is read one batch ahead: the fragment gather of the next batch then waits for
    // one memory round trip, not two in a row
    int32_t g_ahead = range_start + tid < range_end ? P.flatten_ids[range_start + tid] : 0;
    for (int32_t batch_start = range_start; batch_start < range_end; batch_start += kBatch) {
        // all pixels of the tile finished: stop (this barrier also fences reuse of the LDS batch)
        if (__syncthreads_count(Tl == 0.0f) >= kRasterBlock) break;
        const int32_t idx = batch_start + tid;
        if (idx < range_end) {
            float kk;
            FragLds f = stage_fragment(P.screen, P.packed_rows, g_ahead, tile_x0, tile_y0, &kk);
            add_block_mask(f, kk, tile_x0, tile_y0);
            frags[tid] = f;
            if (P.block_masks) P.block_masks[idx] = (uint16_t)(__float_as_uint(f.q2.z) >> 16);   // for the backward
            if constexpr (kDist != SSR_DIST_NONE) s_lz[tid * 12] = ssr_log(ssr_max(f.q2.y, 1e-6f));
        } else {
            frags[tid].q2 = make_float4(0.f, 0.f, 0.f, 0.f);   // empty masks
        }
        if (idx + kBatch < range_end) g_ahead = P.flatten_ids[idx + kBatch];
        __syncthreads();
        const int n_batch = min(kBatch, range_end - batch_start);
        // a row whose sixteen pixels are finished needs no list
        const uint64_t live = __ballot(Tl != 0.0f);
        const bool row_live[4] = {(live & 0xFFFFull) != 0, (live & 0xFFFF0000ull) != 0, (live & 0xFFFF00000000ull) != 0,
                                  (live & 0xFFFF000000000000ull) != 0};
        int cnt[4] = {0, 0, 0, 0};
        if (live != 0ull) {
            for (int c = 0; c * 64 < n_batch; c++) {
                const int slot = c * 64 + lane;
                const uint32_t bits = __float_as_uint(frags[slot].q2.z) >> (16 + 4 * mt);
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    if (!row_live[r]) continue;
                    const bool in = ((bits >> r) & 1u) != 0;
                    const uint64_t bal = __ballot(in);
                    if (in) s_list[(4 * mt + r) * kBatch + cnt[r] + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(bal >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bal, 0u))] = (uint16_t)(slot * 48);
                    cnt[r] += __builtin_popcountll(bal);
                }
            }
        }
        // steps come in pairs: every list is padded to the even step count of the longest with the empty fragment
        const int n_steps = (max(max(cnt[0], cnt[1]), max(cnt[2], cnt[3])) + 1) & ~1;
#pragma unroll
        for (int r = 0; r < 4; r++)
            for (int e = cnt[r] + lane; e < n_steps; e += 64) s_list[(4 * mt + r) * kBatch + e] = (uint16_t)kPadEntry;
        // the lists are written and read by this wavefront only: order its LDS accesses, no workgroup barrier
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        __builtin_amdgcn_wave_barrier();
        uint32_t last_off = 0xFFFFFFFFu;   // offset of the last fragment this batch composited into the pixel
        // One step of a row: the fragment at byte offset `off` (registers q*) against the row's sixteen pixels,
        // branch-free. The same values as: hit = compositing && alpha > 1/255; keep = hit && T(1-alpha) > 1e-4;
        // a kept fragment is added and T updated; a hit that is not kept ends the pixel.
        auto step = [&](uint32_t off, const float4& q0, const float4& q1, const float2& q2, float cut) {
            float dx, dy, vis, sigma;
            const float alpha = eval_alpha_fast(q0, q1, cut, px, py, dx, dy, vis, sigma);
            const float a = alpha > kAlphaThreshold ? alpha : 0.0f;   // a skipped fragment: T (1 - 0) = T exactly
            const float next_T = Tl * (1.0f - a);
            if constexpr (kMedian) {   // before the early-out, so a splat that ends the pixel still counts
                const bool hit = (a > 0.0f) & (Tl > 0.0f);
                const bool cross = hit & (med_prev_T >= 0.5f) & (next_T < 0.5f);
                if (__builtin_amdgcn_ballot_w64(cross) != 0ull) {   // once per pixel: rarely any lane
                    const float la = ssr_log(med_prev_T), lb = ssr_log(next_T), d = lb - la;
                    const float fr = (ssr_fabs(d) > 1e-20f) ? (-0.6931471805599453f - la) / d : 0.0f;
                    median = cross ? med_prev_z + (q2.y - med_prev_z) * fr : median;
                }
                med_prev_T = hit ? next_T : med_prev_T;
                med_prev_z = hit ? q2.y : med_prev_z;
            }
            // a compositing pixel has Tl > 1e-4, so a skipped fragment keeps it; a stopped one has next_T = 0
            const bool keep = next_T > kTransmitThreshold;
            const float w = keep ? a * Tl : 0.0f;   // a fragment that is not composited adds zero
            float zd = q2.y;
            if constexpr (kDist != SSR_DIST_NONE) {
                zd = s_lz[off >> 2];
                if constexpr (kDist == SSR_DIST_RGB_D) {
                    s2r = ssr_fma(q1.z * q1.z, w, s2r); s2g = ssr_fma(q1.w * q1.w, w, s2g);
                    s2b = ssr_fma(q2.x * q2.x, w, s2b);
                }
                s2d = ssr_fma(zd * zd, w, s2d);
            }
            cr = ssr_fma(q1.z, w, cr); cg = ssr_fma(q1.w, w, cg); cb = ssr_fma(q2.x, w, cb);
            cd = ssr_fma(zd, w, cd);
            last_off = w > 0.0f ? off : last_off;   // w > 0 exactly when the fragment was hit and kept (a > 1/255, Tl > 1e-4)
            T = keep ? next_T : T;
            Tl = keep ? next_T : 0.0f;
        };
        // Software pipeline, two steps per trip: list entries run two steps ahead of their use and the fragment of the
        // next step loads while the current one computes, so that the two dependent LDS latencies hide behind
        // arithmetic; the two fragment register sets alternate, so nothing is copied between steps.
        auto list_at = [&](int st) { return (uint32_t)my_list[st]; };   // past the padding: some valid offset, never used
        auto frag_of = [&](uint32_t off) -> const FragLds& {
            return *reinterpret_cast<const FragLds*>(reinterpret_cast<const char*>(frags) + off);
        };
        uint32_t k0 = list_at(0), k1 = list_at(1), k2 = list_at(2);
        float4 a0 = frag_of(k0).q0, a1 = frag_of(k0).q1;
        float2 a2 = make_float2(frag_of(k0).q2.x, frag_of(k0).q2.y);
        float aw = frag_of(k0).q2.w;
        int st = 0;
        if (n_steps > 0 && live != 0ull) do {
            const float4 c0 = frag_of(k1).q0, c1 = frag_of(k1).q1;
            const float2 c2 = make_float2(frag_of(k1).q2.x, frag_of(k1).q2.y);
            const float cw = frag_of(k1).q2.w;
            const uint32_t k3 = list_at(st + 3);
            step(k0, a0, a1, a2, aw);
            a0 = frag_of(k2).q0; a1 = frag_of(k2).q1;
            a2 = make_float2(frag_of(k2).q2.x, frag_of(k2).q2.y);
            aw = frag_of(k2).q2.w;
            const uint32_t k4 = list_at(st + 4);
            step(k1, c0, c1, c2, cw);
            k0 = k2; k1 = k3; k2 = k4;
            st += 2;
        } while (st < n_steps && __builtin_amdgcn_ballot_w64(Tl != 0.0f) != 0ull);   // until this sub-tile is finished
        if (last_off != 0xFFFFFFFFu) cur_idx = (uint32_t)batch_start + last_off / 48u;
    }
    if (inside) {
        const int64_t pid = ((int64_t)img * P.height + i) * P.width + j;
        P.render_T[pid] = T;
        const float invW = 1.0f / ssr_max(1.0f - T, 1e-10f);
        float* o = P.render_rgb + 3 * pid;
        o[0] = cr; o[1] = cg; o[2] = cb;
        if constexpr (kMedian) P.render_median[pid] = median;
        if constexpr (kDist != SSR_DIST_NONE) {   // D = W S - C^2 on the raw accumulators
            const float W = 1.0f - T;
            if constexpr (kDist == SSR_DIST_RGB_D) {
                float* d = P.distortion_rgb + 3 * pid;
                d[0] = s2r * W - cr * cr; d[1] = s2g * W - cg * cg; d[2] = s2b * W - cb * cb;
            }
            P.distortion_depth[pid] = s2d * W - cd * cd;
            P.render_depth[pid] = ssr_exp(cd * invW);
        } else {
            P.render_depth[pid] = cd * invW;
        }
        P.last_ids[pid] = (int32_t)cur_idx;
    }
}

}  // namespace ssr

using namespace ssr;

extern "C" int ssr_raster_fwd(const ssr_raster_fwd_params* p, ssr_stream_t stream) {
    SSR_REQUIRE(p, "ssr_raster_fwd", "null params");
    SSR_REQUIRE(p->width > 0 && p->height > 0, "ssr_raster_fwd", "empty image");
    SSR_REQUIRE(p->n_isects >= 0 && p->n_isects < (int64_t)1 << 31, "ssr_raster_fwd", "n_isects out of range");
    SSR_REQUIRE(p->render_rgb && p->render_depth && p->render_T && p->last_ids, "ssr_raster_fwd", "null output");
    SSR_REQUIRE(p->tile_offsets, "ssr_raster_fwd", "null tile offsets");
    if (p->n_isects > 0) {
        SSR_REQUIRE(p->flatten_ids, "ssr_raster_fwd", "null flatten_ids");
        if (p->packed_rows) {
            SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->packed_rows) & 15) == 0, "ssr_raster_fwd", "packed_rows must be 16-byte aligned");
        } else {
            SSR_REQUIRE(p->screen.xy && p->screen.depth && p->screen.conic && p->screen.opac && p->screen.rgb,
                        "ssr_raster_fwd", "null screen buffer");
            SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->screen.xy) & 7) == 0, "ssr_raster_fwd", "screen.xy must be 8-byte aligned");
        }
    }
    SSR_REQUIRE(p->dist_type >= SSR_DIST_NONE && p->dist_type <= SSR_DIST_RGB_D, "ssr_raster_fwd",
                "dist_type must be NONE, D or RGB_D (the 3dgs pixel has no normal channel)");
    SSR_REQUIRE(p->dist_type == SSR_DIST_NONE || p->distortion_depth, "ssr_raster_fwd", "null distortion_depth");
    SSR_REQUIRE(p->dist_type != SSR_DIST_RGB_D || p->distortion_rgb, "ssr_raster_fwd", "null distortion_rgb");
    const int tw = (int)ceil_div(p->width, kTile), th = (int)ceil_div(p->height, kTile);
    SSR_REQUIRE(p->num_images >= 0, "ssr_raster_fwd", "negative num_images");
    const int nimg = p->num_images > 1 ? p->num_images : 1;
    SSR_REQUIRE((int64_t)tw * th * nimg < (int64_t)1 << 30, "ssr_raster_fwd", "too many tiles");
    const dim3 grid((unsigned)xcd_grid_size(tw * th * nimg)), block(kRasterBlock);
    hipStream_t s = as_stream(stream);
    const bool med = p->render_median != nullptr;
#define SSR_FWD_ROWS(D, M) hipLaunchKernelGGL((raster_fwd_rows_kernel<D, M>), grid, block, 0, s, *p, tw, th)
    switch (p->dist_type) {
        case SSR_DIST_D: if (med) SSR_FWD_ROWS(SSR_DIST_D, true); else SSR_FWD_ROWS(SSR_DIST_D, false); break;
        case SSR_DIST_RGB_D: if (med) SSR_FWD_ROWS(SSR_DIST_RGB_D, true); else SSR_FWD_ROWS(SSR_DIST_RGB_D, false); break;
        default: if (med) SSR_FWD_ROWS(SSR_DIST_NONE, true); else SSR_FWD_ROWS(SSR_DIST_NONE, false); break;
    }
#undef SSR_FWD_ROWS
    SSR_CHECK_LAUNCH("ssr_raster_fwd");
    return 0;
}
