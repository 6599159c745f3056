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

__global__ __launch_bounds__(kRasterBlock) void raster_fwd_kernel(ssr_raster_fwd_params P, int tile_w, int tile_h) {
    __shared__ FragLds frags[kBatch];
    const int n_tiles = tile_w * tile_h;
    const int tile = xcd_tile_of(blockIdx.x, n_tiles);
    if (tile >= n_tiles) return;   // whole workgroup leaves together
    const int tid = threadIdx.x, lane = tid & 63, mt = tid >> 6;
    const int ty = tile / tile_w, tx = tile - ty * tile_w;
    const int j = tx * kTile + (mt & 1) * kMicro + (lane & 7);
    const int i = ty * kTile + (mt >> 1) * kMicro + (lane >> 3);
    const float px = (float)j + 0.5f, py = (float)i + 0.5f;
    const bool inside = (uint32_t)i < P.height && (uint32_t)j < P.width;
    bool done = !inside;

    const int32_t range_start = P.tile_offsets[tile];
    const int32_t range_end = (tile == n_tiles - 1) ? (int32_t)P.n_isects : P.tile_offsets[tile + 1];

    float T = 1.0f, cr = 0.f, cg = 0.f, cb = 0.f, cd = 0.f;
    uint32_t cur_idx = 0;
    const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);

    for (int32_t batch_start = range_start; batch_start < range_end; batch_start += kBatch) {
        // all pixels of the tile finished: stop (this barrier also fences reuse of the LDS batch)
        if (__syncthreads_count(done) >= kRasterBlock) break;
        const int32_t idx = batch_start + tid;
        if (idx < range_end) {
            frags[tid] = stage_fragment(P.screen, P.packed_rows, P.flatten_ids[idx], tile_x0, tile_y0);
        } else {
            frags[tid].q2 = make_float4(0.f, 0.f, 0.f, 0.f);   // empty footprint mask
        }
        __syncthreads();
        const int n_batch = min(kBatch, range_end - batch_start);
        for (int c = 0; c * 64 < n_batch; c++) {
            if (__ballot(!done) == 0ull) break;   // this sub-tile is finished
            const uint32_t my_hits = __float_as_uint(frags[c * 64 + lane].q2.z);
            uint64_t m = __ballot((my_hits >> mt) & 1u);
            while (m) {
                const int t = __builtin_ctzll(m);
                m &= m - 1;
                const int k = c * 64 + t;
                const float4 q0 = frags[k].q0, q1 = frags[k].q1, q2 = frags[k].q2;
                float dx, dy, vis, sigma;
                const float alpha = eval_alpha_fast(q0, q1, q2.w, px, py, dx, dy, vis, sigma);
                if (!done && alpha > kAlphaThreshold) {
                    const float next_T = T * (1.0f - alpha);
                    if (next_T > kTransmitThreshold) {
                        const float w = alpha * T;
                        cr = ssr_fma(q1.z, w, cr); cg = ssr_fma(q1.w, w, cg); cb = ssr_fma(q2.x, w, cb);
                        cd = ssr_fma(q2.y, w, cd);
                        cur_idx = (uint32_t)(batch_start + k);
                        T = next_T;
                    } else {
                        done = true;
                    }
                }
            }
        }
    }
    if (inside) {
        const int64_t pid = (int64_t)i * P.width + j;
        P.render_T[pid] = T;
        const float invW = 1.0f / ssr_max(1.0f - T, 1e-10f);
        float* o = P.render_rgb + 3 * pid;
        o[0] = cr; o[1] = cg; o[2] = cb;
        P.render_depth[pid] = cd * invW;
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
    const int tw = (int)ceil_div(p->width, kTile), th = (int)ceil_div(p->height, kTile);
    hipLaunchKernelGGL(raster_fwd_kernel, dim3((unsigned)xcd_grid_size(tw * th)), dim3(kRasterBlock), 0, as_stream(stream),
                       *p, tw, th);
    SSR_CHECK_LAUNCH("ssr_raster_fwd");
    return 0;
}
