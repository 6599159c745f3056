// tiles.hip -- K2 (tiles per splat), K3 (int64 inclusive scan), K4 (key write), K6 (tile offsets).
//
// K2/K4 follow intersect_tile_kernel<count, ellipse=true> (src/kernels/tile/IntersectTile.cu:104-267),
// K6 follows intersect_offset_kernel (:271-307). Keys are (tile_id << 32) | depth bits with
// depth bits = bits(|sorting depth|) ^ 0x80000000 (:190-196); values are flat splat indices.
#include "projection_device.h"
#include <mutex>

namespace ssr {

constexpr int kTileBlock = 256;

__global__ __launch_bounds__(kTileBlock) void tile_count_kernel(
    int64_t n, const float4* __restrict__ aabb, const float2* __restrict__ xy,
    const float* __restrict__ conic, const float* __restrict__ opac, int tile_w, int tile_h,
    const int32_t* __restrict__ live, int64_t* __restrict__ tiles_per_splat, uint32_t rows_per_image,
    const int32_t* __restrict__ image_ids) {
    const int64_t g = (int64_t)blockIdx.x * kTileBlock + threadIdx.x;
    if (g >= n) return;
    const float4 a = aabb[g];
    if (a.z <= a.x || a.w <= a.y) { tiles_per_splat[g] = 0; return; }
    // several images: row g belongs to image image_ids[g] (packed rows) or g / rows_per_image, and the
    // tile-skip map holds one [tile_h, tile_w] block per image
    if (live) live += (int64_t)(image_ids ? image_ids[g] : (rows_per_image ? (int)((uint32_t)g / rows_per_image) : 0)) * (tile_w * tile_h);
    const float bb[4] = {a.x, a.y, a.z, a.w};
    const float2 c = xy[g];
    const float cxy[2] = {c.x, c.y};
    const float cn[3] = {conic[3 * g], conic[3 * g + 1], conic[3 * g + 2]};
    TileGeomD tg;
    tile_geom(bb, cxy, cn, opac[g], tile_w, tile_h, tg);
    tiles_per_splat[g] = live ? count_tiles_masked(tg, live, tile_w) : count_tiles(tg);
}

// tile_active_kernel (src/kernels/tile/IntersectTile.cu:316-347): a tile is live when any pixel of
// it, grown by one pixel (the depth-to-normal stencil of the loss reads one pixel past its own),
// is unmasked; the mask is sampled at the nearest source pixel (src/core/Interpolation.cuh:108-120).
__global__ __launch_bounds__(kTileBlock) void tile_active_kernel(const uint8_t* __restrict__ mask, int h_mask, int w_mask,
                                                                 int width, int height, int tile_w, int tile_h,
                                                                 int32_t* __restrict__ tile_active) {
    const int t = blockIdx.x * kTileBlock + threadIdx.x;
    if (t >= tile_w * tile_h) return;
    const int tx = t % tile_w, ty = t / tile_w;
    constexpr int kPad = 1;
    bool live = false;
    for (int dy = -kPad; dy < kTile + kPad && !live; ++dy) {
        const int y = ty * kTile + dy;
        if (y >= height) break;
        if (y < 0) continue;
        for (int dx = -kPad; dx < kTile + kPad; ++dx) {
            const int x = tx * kTile + dx;
            if (x >= width) break;
            if (x < 0) continue;
            const float u = (((float)x + 0.5f) * (float)w_mask) / (float)width - 0.5f;
            const float v = (((float)y + 0.5f) * (float)h_mask) / (float)height - 0.5f;
            const int sx = max(0, min(w_mask - 1, ssr_f2i_sat(ssr_floor(u + 0.5f))));
            const int sy = max(0, min(h_mask - 1, ssr_f2i_sat(ssr_floor(v + 0.5f))));
            if (mask[(size_t)sy * w_mask + sx]) { live = true; break; }
        }
    }
    tile_active[t] = live ? 1 : 0;
}

// Splats that touch more than kCoopTiles tiles (a splat close to the camera can cover thousands)
// are not written by their own thread: the wavefront takes them one at a time, 64 bands per step,
// with a wavefront scan placing each band's run of keys, so no lane loops over thousands of tiles
// while the other 63 wait.
constexpr int kCoopTiles = 96;

__device__ __forceinline__ int wave_inclusive_scan_i32(int v, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}

struct TileWriteArgs {
    const float4* __restrict__ aabb; const float* __restrict__ sort_depth; const float2* __restrict__ xy;
    const float* __restrict__ conic; const float* __restrict__ opac; const int64_t* __restrict__ cum;
    int tile_w, tile_h;
    int64_t* __restrict__ isect_ids; int32_t* __restrict__ flatten_ids;
    const int32_t* __restrict__ visible_ids; const int32_t* __restrict__ live_all;
    uint32_t rows_per_image; const int32_t* __restrict__ image_ids;
};

// Keys of work item i (row i, or the row visible_ids[i]); the whole wavefront calls this together. kCapped: no
// key is written at or beyond position `capacity`.
template <bool kCapped>
__device__ __forceinline__ void tile_write_row(const TileWriteArgs& A, int64_t i, bool in_range, int64_t capacity) {
    const float4* __restrict__ aabb = A.aabb; const float* __restrict__ sort_depth = A.sort_depth;
    const float2* __restrict__ xy = A.xy; const float* __restrict__ conic = A.conic; const float* __restrict__ opac = A.opac;
    const int64_t* __restrict__ cum = A.cum; const int tile_w = A.tile_w, tile_h = A.tile_h;
    int64_t* __restrict__ isect_ids = A.isect_ids; int32_t* __restrict__ flatten_ids = A.flatten_ids;
    const int32_t* __restrict__ visible_ids = A.visible_ids; const int32_t* __restrict__ live_all = A.live_all;
    const uint32_t rows_per_image = A.rows_per_image; const int32_t* __restrict__ image_ids = A.image_ids;
    const int lane = threadIdx.x & 63;
    const int64_t g = in_range ? (visible_ids ? (int64_t)visible_ids[i] : i) : 0;
    int64_t cur = 0, end = 0;
    TileGeomD tg;
    uint32_t du = 0;
    bool visible = false;
    // several images in one launch: row g belongs to image image_ids[g] (packed rows) or g / rows_per_image;
    // its tiles follow the earlier images' in the key space, and its block of the tile-skip map is its own
    const int image = (in_range && image_ids) ? image_ids[g] : (rows_per_image ? (int)((uint32_t)g / rows_per_image) : 0);
    const int tile_base = image * (tile_w * tile_h);
    const int32_t* live = live_all ? live_all + tile_base : nullptr;
    if (in_range) {
        cur = g == 0 ? 0 : cum[g - 1];
        end = cum[g];
        if (kCapped) { cur = min(cur, capacity); end = min(end, capacity); }
        const float4 a = aabb[g];
        visible = !(a.z <= a.x || a.w <= a.y);
        if (visible) {
            const float bb[4] = {a.x, a.y, a.z, a.w};
            const float2 c = xy[g];
            const float cxy[2] = {c.x, c.y};
            const float cn[3] = {conic[3 * g], conic[3 * g + 1], conic[3 * g + 2]};
            tile_geom(bb, cxy, cn, opac[g], tile_w, tile_h, tg);
            du = ssr_f2u(ssr_fabs(sort_depth[g]));
            du = (du >> 31) ? ~du : (du ^ 0x80000000u);
        }
    }
    const bool coop = visible && (end - cur) > kCoopTiles;
    if (visible && !coop) {
        for_each_tile(tg, [&](int lo, int hi, int fixed, bool rows) {
            for (int v = lo; v < hi && cur < end; v++) {
                if (live && !tile_is_live(live, tile_w, fixed, v, rows)) continue;
                const int64_t tile_id = tile_base + (rows ? ((int64_t)fixed * tile_w + v) : ((int64_t)v * tile_w + fixed));
                isect_ids[cur] = (int64_t)(((uint64_t)tile_id << 32) | (uint64_t)du);
                flatten_ids[cur] = (int32_t)g;
                ++cur;
            }
        });
    }
    if (in_range && !coop) {
        while (cur < end) {   // IntersectTile.cu:261-266; unreachable when count and write agree
            isect_ids[cur] = (int64_t)0xffffffffull;
            flatten_ids[cur] = (int32_t)g;
            ++cur;
        }
    }
    // cooperative part: the whole wavefront stays converged here
    uint64_t todo = __ballot(coop);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        TileGeomD sg;
        sg.xy[0] = __shfl(tg.xy[0], src, 64); sg.xy[1] = __shfl(tg.xy[1], src, 64);
        sg.ic[0] = __shfl(tg.ic[0], src, 64); sg.ic[1] = __shfl(tg.ic[1], src, 64); sg.ic[2] = __shfl(tg.ic[2], src, 64);
        sg.xmin = __shfl(tg.xmin, src, 64); sg.xmax = __shfl(tg.xmax, src, 64);
        sg.ymin = __shfl(tg.ymin, src, 64); sg.ymax = __shfl(tg.ymax, src, 64);
        sg.by_rows = __shfl((int)tg.by_rows, src, 64) != 0;
        const uint32_t sdu = (uint32_t)__shfl((int)du, src, 64);
        const int32_t sgid = (int32_t)__shfl((int)g, src, 64);
        const int sbase = __shfl(tile_base, src, 64);
        const int32_t* slive = live_all ? live_all + sbase : nullptr;
        int64_t scur = ((int64_t)__shfl((int)(cur >> 32), src, 64) << 32) | (uint32_t)__shfl((int)(uint32_t)cur, src, 64);
        const int64_t send = ((int64_t)__shfl((int)(end >> 32), src, 64) << 32) | (uint32_t)__shfl((int)(uint32_t)end, src, 64);
        const int b0 = sg.by_rows ? sg.ymin : sg.xmin, b1 = sg.by_rows ? sg.ymax : sg.xmax;
        for (int base = b0; base < b1; base += 64) {
            const int r = base + lane;
            int lo = 0, hi = 0;
            if (r < b1) tile_band_interval(sg, r, lo, hi);
            const int c = slive ? count_live(slive, tile_w, lo, hi, r, sg.by_rows) : max(hi - lo, 0);
            const int inc = wave_inclusive_scan_i32(c, lane);
            int64_t pos = scur + (inc - c);
            for (int v = lo; v < hi && pos < send; v++) {
                if (slive && !tile_is_live(slive, tile_w, r, v, sg.by_rows)) continue;
                const int64_t tile_id = sbase + (sg.by_rows ? ((int64_t)r * tile_w + v) : ((int64_t)v * tile_w + r));
                isect_ids[pos] = (int64_t)(((uint64_t)tile_id << 32) | (uint64_t)sdu);
                flatten_ids[pos] = sgid;
                pos++;
            }
            scur += __shfl(inc, 63, 64);
        }
        for (int64_t pos = scur + lane; pos < send; pos += 64) {   // pad keys, as above
            isect_ids[pos] = (int64_t)0xffffffffull;
            flatten_ids[pos] = sgid;
        }
    }
}

__global__ __launch_bounds__(kTileBlock) void tile_write_kernel(int64_t n, TileWriteArgs A) {
    const int64_t i = (int64_t)blockIdx.x * kTileBlock + threadIdx.x;
    tile_write_row<false>(A, i, i < n, 0);
}

// The key write when the host does not know the counts: the arrays hold `capacity` entries, and the work list's
// length, when there is a list, is *n_visible (device): the launch covers all n rows and the threads behind the
// list's end leave at once. No key is written at or beyond `capacity`.
__global__ __launch_bounds__(kTileBlock) void tile_write_capped_kernel(int64_t n, TileWriteArgs A, int64_t capacity,
                                                                       const int64_t* __restrict__ n_visible) {
    const int64_t i = (int64_t)blockIdx.x * kTileBlock + threadIdx.x;
    const int64_t work = (A.visible_ids && n_visible) ? min(*n_visible, n) : n;
    if ((int64_t)blockIdx.x * kTileBlock >= work) return;
    tile_write_row<true>(A, i, i < work, capacity);
}

// ---- int64 inclusive scan: per-block reduce, single-block scan of the block sums, downsweep ----

constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanBlock * kScanItems;

__device__ __forceinline__ int64_t wave_inclusive_scan(int64_t v, int lane) {
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int64_t o = __shfl_up(v, d, 64);
        if (lane >= d) v += o;
    }
    return v;
}

// Exclusive prefix of `v` over the block plus the block total; 4 wavefronts.
__device__ __forceinline__ int64_t block_exclusive_scan(int64_t v, int64_t& total, int64_t* lds /* [4] */) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t inc = wave_inclusive_scan(v, lane);
    if (lane == 63) lds[wave] = inc;
    __syncthreads();
    int64_t base = 0;
#pragma unroll
    for (int w = 0; w < kScanBlock / 64; w++) { if (w < wave) base += lds[w]; }
    total = lds[0] + lds[1] + lds[2] + lds[3];
    __syncthreads();
    return base + inc - v;
}

// Item layout of the two passes over the data: a wavefront owns 8 x 64 consecutive items and reads them in eight
// rounds, lane l taking item 64 r + l of its run, so that every load and store instruction covers one contiguous
// 512 bytes (eight consecutive items per THREAD made each instruction touch 64 cache lines).
__global__ __launch_bounds__(kScanBlock) void scan_reduce_kernel(const int64_t* __restrict__ in, int64_t n,
                                                                 int64_t* __restrict__ block_sums) {
    __shared__ int64_t lds[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)wave * (64 * kScanItems) + lane;
    int64_t s = 0;
#pragma unroll
    for (int r = 0; r < kScanItems; r++) { if (base + 64 * r < n) s += in[base + 64 * r]; }
    int64_t total;
    block_exclusive_scan(s, total, lds);
    if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}

__global__ __launch_bounds__(kScanBlock) void scan_spine_kernel(int64_t* __restrict__ block_sums, int64_t n_blocks) {
    __shared__ int64_t lds[4];
    int64_t carry = 0;
    for (int64_t start = 0; start < n_blocks; start += kScanBlock) {
        const int64_t i = start + threadIdx.x;
        const int64_t v = i < n_blocks ? block_sums[i] : 0;
        int64_t total;
        const int64_t ex = block_exclusive_scan(v, total, lds);
        if (i < n_blocks) block_sums[i] = carry + ex;   // exclusive prefix
        carry += total;
    }
}

// kSumTotals: block_prefix holds the workgroups' totals as scan_reduce_kernel left them, and every workgroup adds
// up the ones before it for itself (a few loads per thread up to kScanSumBlocks workgroups): the spine kernel
// between the two passes, a launch of four wavefronts, is then not needed.
constexpr int64_t kScanSumBlocks = 4096;
template <bool kSumTotals>
__global__ __launch_bounds__(kScanBlock) void scan_down_kernel(const int64_t* __restrict__ in, int64_t n,
                                                               const int64_t* __restrict__ block_prefix,
                                                               int64_t* __restrict__ out, int64_t* __restrict__ total_out) {
    __shared__ int64_t lds[4];
    [[maybe_unused]] __shared__ int64_t lds_before[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    [[maybe_unused]] int64_t before = 0;
    if constexpr (kSumTotals) {
        for (int64_t b = threadIdx.x; b < (int64_t)blockIdx.x; b += kScanBlock) before += block_prefix[b];
    }
    const int64_t base = (int64_t)blockIdx.x * kScanTile + (int64_t)wave * (64 * kScanItems) + lane;
    int64_t v[kScanItems];
    int64_t s = 0;
#pragma unroll
    for (int r = 0; r < kScanItems; r++) { v[r] = base + 64 * r < n ? in[base + 64 * r] : 0; s += v[r]; }
    // what lies before this wavefront's run: the workgroup's prefix and the wavefronts before it
    int64_t w = s;
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) w += __shfl_xor(w, d, 64);
    if constexpr (kSumTotals) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) before += __shfl_xor(before, d, 64);
        if (lane == 0) lds_before[wave] = before;
    }
    if (lane == 0) lds[wave] = w;
    __syncthreads();
    int64_t carry;
    if constexpr (kSumTotals) carry = (lds_before[0] + lds_before[1]) + (lds_before[2] + lds_before[3]);
    else carry = block_prefix[blockIdx.x];
#pragma unroll
    for (int k = 0; k < kScanBlock / 64; k++) { if (k < wave) carry += lds[k]; }
    // the run itself: an inclusive scan of each round of 64 items on top of the rounds before it
#pragma unroll
    for (int r = 0; r < kScanItems; r++) {
        const int64_t inc = carry + wave_inclusive_scan(v[r], lane);
        if (base + 64 * r < n) {
            out[base + 64 * r] = inc;
            if (total_out && base + 64 * r == n - 1) *total_out = inc;
        }
        carry = __shfl(inc, 63, 64);
    }
}

// ---- scan workspace held by the library itself (ssr_inclusive_sum_i64_static) ----

// Block sums of the largest scan the allocation-free entry point accepts: 65 536 blocks of 2048
// elements = 2^27 elements, 512 KiB. Every GPU the library runs on holds its own copy of this array
// at its own address for the life of the process. The name below is only the host-side handle of
// the symbol; host code uses the address hipGetSymbolAddress returns for the current device.
constexpr int64_t kStaticScanBlocks = 65536;
static __device__ __align__(256) int64_t scan_static_scratch[kStaticScanBlocks];

constexpr int kMaxDevices = 64;
static int64_t* g_static_scan_ptr[kMaxDevices];   // per device, null until resolved
static std::mutex g_static_scan_mutex;

// Resolves (once per device, with that device current) the device address of the array above.
static int static_scan_pointer(int64_t** out) {
    int dev = -1;
    int e = check_hip(hipGetDevice(&dev), "ssr_inclusive_sum_i64_static/hipGetDevice");
    if (e) return e;
    if (dev < 0 || dev >= kMaxDevices) return fail("ssr_inclusive_sum_i64_static", "device index out of range");
    std::lock_guard<std::mutex> lock(g_static_scan_mutex);
    if (!g_static_scan_ptr[dev]) {
        void* p = nullptr;
        e = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scan_static_scratch)), "ssr_inclusive_sum_i64_static/hipGetSymbolAddress");
        if (e) return e;
        if (!p) return fail("ssr_inclusive_sum_i64_static", "the scan workspace has no device address");
        g_static_scan_ptr[dev] = static_cast<int64_t*>(p);
    }
    *out = g_static_scan_ptr[dev];
    return 0;
}

int warm_static_scan() {
    int64_t* p = nullptr;
    return static_scan_pointer(&p);
}

// ---- K6 ----

// n_dev (optional): the real number of keys, on the device, where the host only knows an upper bound n_isects.
__global__ __launch_bounds__(kTileBlock) void tile_offsets_kernel(int64_t n_isects, const int64_t* __restrict__ n_dev,
                                                                  const int64_t* __restrict__ ids, int64_t n_tiles,
                                                                  int32_t* __restrict__ offsets) {
    const int64_t idx = (int64_t)blockIdx.x * kTileBlock + threadIdx.x;
    if (n_dev) n_isects = min(n_isects, *n_dev);
    // The tiles up to the first key's and those behind the last key's can be half the image (a scene that covers
    // its middle): the first workgroup and the one that holds the last key fill them together, not one thread each.
    if (blockIdx.x == 0) {
        const int64_t upto = n_isects > 0 ? min((int64_t)(ids[0] >> 32) + 1, n_tiles) : (n_dev ? n_tiles : 0);   // no key: nobody below writes anything
        for (int64_t i = threadIdx.x; i < upto; i += kTileBlock) offsets[i] = 0;
    }
    if (n_isects > 0 && (int64_t)blockIdx.x == (n_isects - 1) / kTileBlock) {
        const int64_t from = (ids[n_isects - 1] >> 32) + 1;
        for (int64_t i = from + threadIdx.x; i < n_tiles; i += kTileBlock) offsets[i] = (int32_t)n_isects;
    }
    if (idx >= n_isects) return;
    const int64_t tile = ids[idx] >> 32;
    if (idx > 0) {
        const int64_t prev = ids[idx - 1] >> 32;
        if (prev != tile)
            for (int64_t i = prev + 1; i < tile + 1 && i < n_tiles; ++i) offsets[i] = (int32_t)idx;
    }
}

// Launch order of the compositing workgroups: all tiles by descending fragment count. Workgroups are dispatched in
// index order as compute units free up, and dealt round-robin to the eight XCDs, so with this order the long tiles
// of a clustered scene start at once instead of forming the tail of the launch, and every XCD receives the same
// mix of loads (contiguous bands of tiles per XCD, which keep a band's splat rows in one L2, left whole XCDs idle
// at the end: measured, the balance is worth far more than the locality). A counting sort in 256 classes of 32
// fragments: workgroups of 1024 tiles count their classes into a table; a second kernel turns the table into
// positions and scatters. The order inside a class does not matter.
constexpr int kOrderBlock = 1024;
__device__ __forceinline__ uint32_t tile_class(const int32_t* __restrict__ offsets, uint32_t t, uint32_t n_tiles, int64_t n_isects) {
    const int64_t e = (t + 1 < n_tiles || n_isects < 0) ? (int64_t)offsets[t + 1] : n_isects;   // < 0: one entry more
    const int64_t len = e - offsets[t];
    return 255u - (uint32_t)min((int64_t)255, len >> 5);   // class 0 holds the longest tiles
}
// The lanes of this wavefront that hold the same class as this lane (live lanes only).
__device__ __forceinline__ uint64_t wave_peers_u8(uint32_t cls, bool live) {
    uint64_t peers = __ballot(live);
#pragma unroll
    for (int b = 0; b < 8; b++) {
        const bool own = ((cls >> b) & 1u) != 0;
        const uint64_t vote = __ballot(own);
        peers &= own ? vote : ~vote;
    }
    return peers;
}
// Tiles of one class are many (most tiles of an image hold similar numbers of fragments): a wavefront adds once per
// class it holds, not once per tile.
// counts[block][256]: how many tiles of each class the workgroup's 1024 tiles hold
__global__ __launch_bounds__(kOrderBlock) void tile_order_count_kernel(const int32_t* __restrict__ offsets, uint32_t n_tiles,
                                                                       int64_t n_isects, uint32_t* __restrict__ counts) {
    __shared__ uint32_t s_count[256];
    if (threadIdx.x < 256) s_count[threadIdx.x] = 0;
    __syncthreads();
    const uint32_t t = blockIdx.x * kOrderBlock + threadIdx.x;
    {
        const bool live = t < n_tiles;
        const uint32_t cls = live ? tile_class(offsets, t, n_tiles, n_isects) : 0u;
        const uint64_t peers = wave_peers_u8(cls, live);
        if (live && (peers & ((1ull << (threadIdx.x & 63)) - 1ull)) == 0) atomicAdd(&s_count[cls], (uint32_t)__popcll(peers));
    }
    __syncthreads();
    if (threadIdx.x < 256) counts[blockIdx.x * 256 + threadIdx.x] = s_count[threadIdx.x];
}
// Every workgroup sums the table for itself (a few dozen rows): the size of each class and what the workgroups
// before it hold of it give, after a scan over the classes, where its own tiles of that class go.
__global__ __launch_bounds__(kOrderBlock) void tile_order_scatter_kernel(const int32_t* __restrict__ offsets, uint32_t n_tiles,
                                                                         int64_t n_isects, const uint32_t* __restrict__ counts,
                                                                         int32_t* __restrict__ order) {
    __shared__ uint32_t s_next[256];
    __shared__ uint32_t s_wave[4];
    if (threadIdx.x < 256) {
        uint32_t total = 0, before = 0;
#pragma unroll 8
        for (uint32_t b = 0; b < gridDim.x; b++) {   // (unrolled: the rows' loads in flight together)
            const uint32_t c = counts[b * 256 + threadIdx.x];
            total += c;
            if (b < blockIdx.x) before += c;
        }
        uint32_t incl = total;   // exclusive scan over the 256 classes: four wavefronts, then their totals
        const int lane = threadIdx.x & 63;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d, 64);
            if (lane >= d) incl += up;
        }
        if (lane == 63) s_wave[threadIdx.x >> 6] = incl;
        s_next[threadIdx.x] = incl - total + before;
    }
    __syncthreads();
    if (threadIdx.x < 256) {
        uint32_t add = 0;
        for (uint32_t w = 0; w < (threadIdx.x >> 6); w++) add += s_wave[w];
        s_next[threadIdx.x] += add;
    }
    __syncthreads();
    const uint32_t t = blockIdx.x * kOrderBlock + threadIdx.x;
    const bool live = t < n_tiles;
    const int lane = threadIdx.x & 63;
    const uint32_t cls = live ? tile_class(offsets, t, n_tiles, n_isects) : 0u;
    const uint64_t peers = wave_peers_u8(cls, live);
    const uint32_t rank = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
    uint32_t base = 0;
    if (live && rank == 0) base = atomicAdd(&s_next[cls], (uint32_t)__popcll(peers));
    base = __shfl(base, peers ? __ffsll((long long)peers) - 1 : 0, 64);   // from the class's first lane
    if (live) order[base + rank] = (int32_t)t;
}

// The same order from one launch when the tiles are few enough for one workgroup to hold their classes in registers
// (four per thread): count into LDS, scan the 256 classes, scatter. Measured: 2500 tiles 12.8 -> 9.0 us against the two
// launches; at 8160 tiles one compute unit alone is the slower way (10 -> 17.7 us), hence the limit.
constexpr int kOrderOnePer = 4;
__global__ __launch_bounds__(kOrderBlock) void tile_order_one_kernel(const int32_t* __restrict__ offsets, uint32_t n_tiles,
                                                                     int64_t n_isects, int32_t* __restrict__ order) {
    __shared__ uint32_t s_next[256];
    __shared__ uint32_t s_wave[4];
    if (threadIdx.x < 256) s_next[threadIdx.x] = 0;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    uint32_t cls[kOrderOnePer];
#pragma unroll
    for (int k = 0; k < kOrderOnePer; k++) {
        const uint32_t t = (uint32_t)k * kOrderBlock + threadIdx.x;
        cls[k] = t < n_tiles ? tile_class(offsets, t, n_tiles, n_isects) : 0u;
    }
#pragma unroll
    for (int k = 0; k < kOrderOnePer; k++) {
        if ((uint32_t)k * kOrderBlock >= n_tiles) break;   // the same for every thread
        const bool live = (uint32_t)k * kOrderBlock + threadIdx.x < n_tiles;
        const uint64_t peers = wave_peers_u8(cls[k], live);
        if (live && (peers & ((1ull << lane) - 1ull)) == 0) atomicAdd(&s_next[cls[k]], (uint32_t)__popcll(peers));
    }
    __syncthreads();
    uint32_t total = 0, incl = 0;
    if (threadIdx.x < 256) {   // exclusive scan over the classes: four wavefronts, then their totals
        total = incl = s_next[threadIdx.x];
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t up = __shfl_up(incl, d, 64);
            if (lane >= d) incl += up;
        }
        if (lane == 63) s_wave[threadIdx.x >> 6] = incl;
    }
    __syncthreads();
    if (threadIdx.x < 256) {
        uint32_t add = 0;
        for (uint32_t w = 0; w < (threadIdx.x >> 6); w++) add += s_wave[w];
        s_next[threadIdx.x] = incl - total + add;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kOrderOnePer; k++) {
        if ((uint32_t)k * kOrderBlock >= n_tiles) break;
        const uint32_t t = (uint32_t)k * kOrderBlock + threadIdx.x;
        const bool live = t < n_tiles;
        const uint64_t peers = wave_peers_u8(cls[k], live);
        const uint32_t rank = (uint32_t)__popcll(peers & ((1ull << lane) - 1ull));
        uint32_t base = 0;
        if (live && rank == 0) base = atomicAdd(&s_next[cls[k]], (uint32_t)__popcll(peers));
        base = __shfl(base, peers ? __ffsll((long long)peers) - 1 : 0, 64);   // from the class's first lane
        if (live) order[base + rank] = (int32_t)t;
    }
}

}  // namespace ssr

using namespace ssr;

extern "C" {

int ssr_compute_tile_active(const uint8_t* mask, int32_t mask_height, int32_t mask_width, uint32_t width, uint32_t height,
                            int32_t* tile_active, ssr_stream_t stream) {
    SSR_REQUIRE(mask && tile_active, "ssr_compute_tile_active", "null pointer");
    SSR_REQUIRE(mask_height > 0 && mask_width > 0 && width > 0 && height > 0, "ssr_compute_tile_active", "empty mask or image");
    SSR_REQUIRE(width < (1u << 30) && height < (1u << 30), "ssr_compute_tile_active", "image too large");
    const int tw = (int)ceil_div(width, kTile), th = (int)ceil_div(height, kTile);
    hipLaunchKernelGGL(tile_active_kernel, dim3((unsigned)ceil_div((int64_t)tw * th, kTileBlock)), dim3(kTileBlock), 0,
                       as_stream(stream), mask, mask_height, mask_width, (int)width, (int)height, tw, th, tile_active);
    SSR_CHECK_LAUNCH("ssr_compute_tile_active");
    return 0;
}

int ssr_tile_count(int64_t n, const float* aabb, const float* xy, const float* conic, const float* opac,
                   uint32_t width, uint32_t height, const int32_t* tile_active, int64_t* tiles_per_splat,
                   ssr_stream_t stream) {
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, "ssr_tile_count", "count out of range");
    if (n == 0) return 0;
    SSR_REQUIRE(aabb && xy && conic && opac && tiles_per_splat, "ssr_tile_count", "null pointer");
    SSR_REQUIRE(width > 0 && height > 0, "ssr_tile_count", "empty image");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(aabb) & 15) == 0 && (reinterpret_cast<uintptr_t>(xy) & 7) == 0,
                "ssr_tile_count", "aabb must be 16-byte and xy 8-byte aligned");
    const int tw = (int)ceil_div(width, kTile), th = (int)ceil_div(height, kTile);
    hipLaunchKernelGGL(tile_count_kernel, dim3((unsigned)ceil_div(n, kTileBlock)), dim3(kTileBlock), 0, as_stream(stream),
                       n, reinterpret_cast<const float4*>(aabb), reinterpret_cast<const float2*>(xy), conic, opac, tw, th,
                       tile_active, tiles_per_splat, 0u, (const int32_t*)nullptr);
    SSR_CHECK_LAUNCH("ssr_tile_count");
    return 0;
}

int ssr_tile_count_images(int64_t n, int64_t rows_per_image, const int32_t* image_ids, int32_t num_images, const float* aabb,
                          const float* xy, const float* conic, const float* opac, uint32_t width, uint32_t height,
                          const int32_t* tile_active, int64_t* tiles_per_splat, ssr_stream_t stream) {
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, "ssr_tile_count_images", "count out of range");
    if (n == 0) return 0;
    SSR_REQUIRE(num_images >= 1, "ssr_tile_count_images", "num_images must be at least 1");
    SSR_REQUIRE(image_ids || (rows_per_image > 0 && rows_per_image * num_images == n), "ssr_tile_count_images",
                "without image_ids, n must be num_images * rows_per_image");
    SSR_REQUIRE(aabb && xy && conic && opac && tiles_per_splat, "ssr_tile_count_images", "null pointer");
    SSR_REQUIRE(width > 0 && height > 0, "ssr_tile_count_images", "empty image");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(aabb) & 15) == 0 && (reinterpret_cast<uintptr_t>(xy) & 7) == 0,
                "ssr_tile_count_images", "aabb must be 16-byte and xy 8-byte aligned");
    const int tw = (int)ceil_div(width, kTile), th = (int)ceil_div(height, kTile);
    SSR_REQUIRE((int64_t)num_images * tw * th < (int64_t)1 << 31, "ssr_tile_count_images", "tile ids of all images must fit 31 bits");
    hipLaunchKernelGGL(tile_count_kernel, dim3((unsigned)ceil_div(n, kTileBlock)), dim3(kTileBlock), 0, as_stream(stream),
                       n, reinterpret_cast<const float4*>(aabb), reinterpret_cast<const float2*>(xy), conic, opac, tw, th,
                       tile_active, tiles_per_splat, image_ids ? 0u : (uint32_t)rows_per_image, image_ids);
    SSR_CHECK_LAUNCH("ssr_tile_count_images");
    return 0;
}

size_t ssr_scan_scratch_bytes(int64_t n) {
    if (n <= 0) return 0;
    return (size_t)ceil_div(n, kScanTile) * sizeof(int64_t);
}

int ssr_inclusive_sum_i64(const int64_t* in, int64_t* out, int64_t n, int64_t* total_out, void* scratch,
                          size_t scratch_bytes, ssr_stream_t stream) {
    SSR_REQUIRE(n >= 0, "ssr_inclusive_sum_i64", "negative count");
    if (n == 0) return 0;
    SSR_REQUIRE(in && out, "ssr_inclusive_sum_i64", "null pointer");
    SSR_REQUIRE(scratch && scratch_bytes >= ssr_scan_scratch_bytes(n), "ssr_inclusive_sum_i64", "scratch too small");
    const int64_t nb = ceil_div(n, kScanTile);
    int64_t* sums = reinterpret_cast<int64_t*>(scratch);
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(scan_reduce_kernel, dim3((unsigned)nb), dim3(kScanBlock), 0, s, in, n, sums);
    if (nb <= kScanSumBlocks) {
        hipLaunchKernelGGL(scan_down_kernel<true>, dim3((unsigned)nb), dim3(kScanBlock), 0, s, in, n, sums, out, total_out);
    } else {
        hipLaunchKernelGGL(scan_spine_kernel, dim3(1), dim3(kScanBlock), 0, s, sums, nb);
        hipLaunchKernelGGL(scan_down_kernel<false>, dim3((unsigned)nb), dim3(kScanBlock), 0, s, in, n, sums, out, total_out);
    }
    SSR_CHECK_LAUNCH("ssr_inclusive_sum_i64");
    return 0;
}

int ssr_inclusive_sum_i64_static(const int64_t* in, int64_t* out, int64_t n, int64_t* total_out, ssr_stream_t stream) {
    SSR_REQUIRE(n >= 0, "ssr_inclusive_sum_i64_static", "negative count");
    SSR_REQUIRE(n <= kStaticScanBlocks * (int64_t)kScanTile, "ssr_inclusive_sum_i64_static",
                "count exceeds the built-in workspace (2^27 elements); use ssr_inclusive_sum_i64 with caller scratch");
    if (n == 0) return 0;
    SSR_REQUIRE(in && out, "ssr_inclusive_sum_i64_static", "null pointer");
    int64_t* sums = nullptr;
    const int e = static_scan_pointer(&sums);
    if (e) return e;
    // Nothing to clear: the first kernel writes every block sum the other two read.
    const int64_t nb = ceil_div(n, kScanTile);
    hipStream_t s = as_stream(stream);
    hipLaunchKernelGGL(scan_reduce_kernel, dim3((unsigned)nb), dim3(kScanBlock), 0, s, in, n, sums);
    if (nb <= kScanSumBlocks) {
        hipLaunchKernelGGL(scan_down_kernel<true>, dim3((unsigned)nb), dim3(kScanBlock), 0, s, in, n, sums, out, total_out);
    } else {
        hipLaunchKernelGGL(scan_spine_kernel, dim3(1), dim3(kScanBlock), 0, s, sums, nb);
        hipLaunchKernelGGL(scan_down_kernel<false>, dim3((unsigned)nb), dim3(kScanBlock), 0, s, in, n, sums, out, total_out);
    }
    SSR_CHECK_LAUNCH("ssr_inclusive_sum_i64_static");
    return 0;
}

int ssr_tile_write(int64_t n, const float* aabb, const float* sort_depth, const float* xy, const float* conic,
                   const float* opac, const int64_t* cum_tiles, uint32_t width, uint32_t height, int64_t* isect_ids,
                   int32_t* flatten_ids, const int32_t* visible_ids, int64_t n_visible, const int32_t* tile_active,
                   ssr_stream_t stream) {
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, "ssr_tile_write", "count out of range");
    if (visible_ids) {
        SSR_REQUIRE(n_visible >= 0 && n_visible <= n, "ssr_tile_write", "visible count out of range");
        if (n_visible == 0) return 0;
    }
    if (n == 0) return 0;
    SSR_REQUIRE(aabb && sort_depth && xy && conic && opac && cum_tiles, "ssr_tile_write", "null pointer");
    SSR_REQUIRE(isect_ids && flatten_ids, "ssr_tile_write", "null output (n_isects == 0 needs no call)");
    SSR_REQUIRE(width > 0 && height > 0, "ssr_tile_write", "empty image");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(aabb) & 15) == 0 && (reinterpret_cast<uintptr_t>(xy) & 7) == 0,
                "ssr_tile_write", "aabb must be 16-byte and xy 8-byte aligned");
    const int tw = (int)ceil_div(width, kTile), th = (int)ceil_div(height, kTile);
    const int64_t work = visible_ids ? n_visible : n;
    const TileWriteArgs A = {reinterpret_cast<const float4*>(aabb), sort_depth, reinterpret_cast<const float2*>(xy), conic, opac,
                             cum_tiles, tw, th, isect_ids, flatten_ids, visible_ids, tile_active, 0u, nullptr};
    hipLaunchKernelGGL(tile_write_kernel, dim3((unsigned)ceil_div(work, kTileBlock)), dim3(kTileBlock), 0, as_stream(stream),
                       work, A);
    SSR_CHECK_LAUNCH("ssr_tile_write");
    return 0;
}

int ssr_tile_write_images(int64_t n, int64_t rows_per_image, const int32_t* image_ids, int32_t num_images,
                          const float* aabb, const float* sort_depth, const float* xy, const float* conic, const float* opac,
                          const int64_t* cum_tiles, uint32_t width, uint32_t height, int64_t* isect_ids, int32_t* flatten_ids,
                          const int32_t* tile_active, ssr_stream_t stream) {
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, "ssr_tile_write_images", "count out of range");
    if (n == 0) return 0;
    SSR_REQUIRE(num_images >= 1, "ssr_tile_write_images", "num_images must be at least 1");
    SSR_REQUIRE(image_ids || (rows_per_image > 0 && rows_per_image * num_images == n), "ssr_tile_write_images",
                "without image_ids, n must be num_images * rows_per_image");
    SSR_REQUIRE(aabb && sort_depth && xy && conic && opac && cum_tiles, "ssr_tile_write_images", "null pointer");
    SSR_REQUIRE(isect_ids && flatten_ids, "ssr_tile_write_images", "null output (n_isects == 0 needs no call)");
    SSR_REQUIRE(width > 0 && height > 0, "ssr_tile_write_images", "empty image");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(aabb) & 15) == 0 && (reinterpret_cast<uintptr_t>(xy) & 7) == 0,
                "ssr_tile_write_images", "aabb must be 16-byte and xy 8-byte aligned");
    const int tw = (int)ceil_div(width, kTile), th = (int)ceil_div(height, kTile);
    SSR_REQUIRE((int64_t)num_images * tw * th < (int64_t)1 << 31, "ssr_tile_write_images",
                "tile ids of all images must fit 31 bits");
    const TileWriteArgs A = {reinterpret_cast<const float4*>(aabb), sort_depth, reinterpret_cast<const float2*>(xy), conic, opac,
                             cum_tiles, tw, th, isect_ids, flatten_ids, nullptr, tile_active,
                             image_ids ? 0u : (uint32_t)rows_per_image, image_ids};
    hipLaunchKernelGGL(tile_write_kernel, dim3((unsigned)ceil_div(n, kTileBlock)), dim3(kTileBlock), 0, as_stream(stream), n, A);
    SSR_CHECK_LAUNCH("ssr_tile_write_images");
    return 0;
}

int ssr_tile_write_capped(const ssr_tile_write_capped_params* p, ssr_stream_t stream) {
    SSR_REQUIRE(p, "ssr_tile_write_capped", "null params");
    SSR_REQUIRE(p->n >= 0 && p->n < (int64_t)1 << 31, "ssr_tile_write_capped", "count out of range");
    SSR_REQUIRE(p->capacity >= 0 && p->capacity < (int64_t)1 << 31, "ssr_tile_write_capped", "capacity out of range");
    if (p->n == 0 || p->capacity == 0) return 0;
    SSR_REQUIRE(p->num_images >= 1, "ssr_tile_write_capped", "num_images must be at least 1");
    SSR_REQUIRE(p->num_images == 1 || p->image_ids || (p->rows_per_image > 0 && p->rows_per_image * p->num_images == p->n),
                "ssr_tile_write_capped", "without image_ids, n must be num_images * rows_per_image");
    SSR_REQUIRE(p->num_images == 1 || !p->visible_ids, "ssr_tile_write_capped", "the work list is for one image");
    SSR_REQUIRE(p->aabb && p->sort_depth && p->xy && p->conic && p->opac && p->cum_tiles, "ssr_tile_write_capped", "null pointer");
    SSR_REQUIRE(p->isect_ids && p->flatten_ids, "ssr_tile_write_capped", "null output");
    SSR_REQUIRE(!p->visible_ids || p->n_visible, "ssr_tile_write_capped", "a work list needs its device count");
    SSR_REQUIRE(p->width > 0 && p->height > 0, "ssr_tile_write_capped", "empty image");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->aabb) & 15) == 0 && (reinterpret_cast<uintptr_t>(p->xy) & 7) == 0,
                "ssr_tile_write_capped", "aabb must be 16-byte and xy 8-byte aligned");
    const int tw = (int)ceil_div(p->width, kTile), th = (int)ceil_div(p->height, kTile);
    SSR_REQUIRE((int64_t)p->num_images * tw * th < (int64_t)1 << 31, "ssr_tile_write_capped",
                "tile ids of all images must fit 31 bits");
    const bool images = p->num_images > 1;
    const TileWriteArgs A = {reinterpret_cast<const float4*>(p->aabb), p->sort_depth, reinterpret_cast<const float2*>(p->xy),
                             p->conic, p->opac, p->cum_tiles, tw, th, p->isect_ids, p->flatten_ids, p->visible_ids,
                             p->tile_active, (images && !p->image_ids) ? (uint32_t)p->rows_per_image : 0u,
                             images ? p->image_ids : nullptr};
    hipLaunchKernelGGL(tile_write_capped_kernel, dim3((unsigned)ceil_div(p->n, kTileBlock)), dim3(kTileBlock), 0,
                       as_stream(stream), p->n, A, p->capacity, p->n_visible);
    SSR_CHECK_LAUNCH("ssr_tile_write_capped");
    return 0;
}

int ssr_sort_end_bit(uint32_t n_tiles) {
    int b = 0;
    while (b < 32 && (1u << b) <= n_tiles) ++b;   // src/kernels/tile/IntersectTile.cu:489-490
    return 32 + b;
}

int ssr_tile_offsets(int64_t n_isects, const int64_t* sorted_ids, uint32_t n_tiles, int32_t* offsets,
                     ssr_stream_t stream) {
    SSR_REQUIRE(n_isects >= 0 && n_isects < (int64_t)1 << 31, "ssr_tile_offsets", "n_isects out of range");
    if (n_tiles == 0) return 0;
    SSR_REQUIRE(offsets, "ssr_tile_offsets", "null offsets");
    if (n_isects == 0) return ssr_fill_u32(offsets, 0u, n_tiles, stream);   // IntersectTile.cu:448-451
    SSR_REQUIRE(sorted_ids, "ssr_tile_offsets", "null keys");
    hipLaunchKernelGGL(tile_offsets_kernel, dim3((unsigned)ceil_div(n_isects, kTileBlock)), dim3(kTileBlock), 0,
                       as_stream(stream), n_isects, (const int64_t*)nullptr, sorted_ids, (int64_t)n_tiles, offsets);
    SSR_CHECK_LAUNCH("ssr_tile_offsets");
    return 0;
}

int ssr_tile_offsets_capped(int64_t capacity, const int64_t* n_isects, const int64_t* sorted_ids, uint32_t n_tiles,
                            int32_t* offsets, ssr_stream_t stream) {
    SSR_REQUIRE(capacity > 0 && capacity < (int64_t)1 << 31, "ssr_tile_offsets_capped", "capacity out of range");
    SSR_REQUIRE(n_tiles > 0 && n_tiles < 0x7fffffffu, "ssr_tile_offsets_capped", "tile count out of range");
    SSR_REQUIRE(offsets && sorted_ids && n_isects, "ssr_tile_offsets_capped", "null pointer");
    hipLaunchKernelGGL(tile_offsets_kernel, dim3((unsigned)ceil_div(capacity, kTileBlock)), dim3(kTileBlock), 0,
                       as_stream(stream), capacity, n_isects, sorted_ids, (int64_t)n_tiles + 1, offsets);
    SSR_CHECK_LAUNCH("ssr_tile_offsets_capped");
    return 0;
}

size_t ssr_tile_order_scratch_bytes(uint32_t n_tiles) {
    return 256 * (size_t)ceil_div((int64_t)n_tiles, kOrderBlock) * sizeof(uint32_t);
}

int ssr_tile_order(const int32_t* tile_offsets, uint32_t n_tiles, int64_t n_isects, int32_t* order, void* scratch,
                   size_t scratch_bytes, ssr_stream_t stream) {
    SSR_REQUIRE(n_tiles < (1u << 30), "ssr_tile_order", "too many tiles");
    if (n_tiles == 0) return 0;
    SSR_REQUIRE(tile_offsets && order, "ssr_tile_order", "null pointer");
    SSR_REQUIRE(scratch && scratch_bytes >= ssr_tile_order_scratch_bytes(n_tiles), "ssr_tile_order", "scratch too small");
    if (n_tiles <= (uint32_t)(kOrderOnePer * kOrderBlock)) {
        hipLaunchKernelGGL(tile_order_one_kernel, dim3(1), dim3(kOrderBlock), 0, as_stream(stream), tile_offsets, n_tiles, n_isects,
                           order);
        SSR_CHECK_LAUNCH("ssr_tile_order");
        return 0;
    }
    uint32_t* counts = static_cast<uint32_t*>(scratch);
    const dim3 grid((unsigned)ceil_div((int64_t)n_tiles, kOrderBlock)), block(kOrderBlock);
    hipLaunchKernelGGL(tile_order_count_kernel, grid, block, 0, as_stream(stream), tile_offsets, n_tiles, n_isects, counts);
    hipLaunchKernelGGL(tile_order_scatter_kernel, grid, block, 0, as_stream(stream), tile_offsets, n_tiles, n_isects,
                       (const uint32_t*)counts, order);
    SSR_CHECK_LAUNCH("ssr_tile_order");
    return 0;
}

}  // extern "C"
