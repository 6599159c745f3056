// sort.hip -- K5: stable LSD radix sort of (uint64 key, int32 value) pairs on a bit range.
//
// Contract: sort_pairs<int64,int32> with double-buffer semantics
// (src/backend/common/SortScan.h:42-56; call site src/kernels/tile/IntersectTile.cu:486-493, where
// the CUDA backend calls cub::DeviceRadixSort::SortPairs and the Vulkan backend its own
// 8-bit-digit sort, src/backend/vulkan/SortScanVulkan.cpp:84-146). The result is the unique
// stable order on the masked key, so any correct stable sort is bit-identical to either.
//
// Per 8-bit digit pass: (1) per-workgroup digit histogram, (2) per-digit scan across workgroups,
// (3) stable scatter (which first scans the 256 digit totals for itself). In (3) each wavefront owns a contiguous
// run of keys and ranks them 64 at a time with ballot-based digit matching (wave64: one 64-bit
// ballot per digit bit), so order inside a workgroup is wave, round, lane = input order.
#include "common.h"

namespace ssr {

constexpr int kSortBlock = 256;                         // 4 wavefronts
constexpr int kSortWaves = kSortBlock / 64;
constexpr int kSortRounds = 16;                         // keys per lane
constexpr int kSortTile = kSortBlock * kSortRounds;     // 4096 keys per workgroup
constexpr int kRadix = 256;

__device__ __forceinline__ uint32_t digit_of(uint64_t key, int shift, uint32_t mask) {
    return (uint32_t)(key >> shift) & mask;
}

// hist[d * n_blocks + block]
__global__ __launch_bounds__(kSortBlock) void sort_hist_kernel(const uint64_t* __restrict__ keys, int64_t n, int shift,
                                                               uint32_t mask, uint32_t n_blocks,
                                                               uint32_t* __restrict__ hist) {
    __shared__ uint32_t lh[kRadix];
    lh[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kSortTile;
#pragma unroll 4
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = base + r * kSortBlock + threadIdx.x;
        if (i < n) atomicAdd(&lh[digit_of(keys[i], shift, mask)], 1u);
    }
    __syncthreads();
    hist[(size_t)threadIdx.x * n_blocks + blockIdx.x] = lh[threadIdx.x];
}

// One workgroup per digit: exclusive scan of its row of per-workgroup counts; row total out.
__global__ __launch_bounds__(kSortBlock) void sort_scan_rows_kernel(uint32_t* __restrict__ hist, uint32_t n_blocks,
                                                                    uint32_t* __restrict__ totals) {
    __shared__ uint32_t ws[kSortWaves];
    uint32_t* row = hist + (size_t)blockIdx.x * n_blocks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t carry = 0;
    for (uint32_t start = 0; start < n_blocks; start += kSortBlock) {
        const uint32_t i = start + threadIdx.x;
        const uint32_t v = i < n_blocks ? row[i] : 0;
        uint32_t inc = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = __shfl_up(inc, d, 64);
            if (lane >= d) inc += o;
        }
        if (lane == 63) ws[wave] = inc;
        __syncthreads();
        uint32_t base = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) { if (w < wave) base += ws[w]; total += ws[w]; }
        if (i < n_blocks) row[i] = carry + base + inc - v;
        carry += total;
        __syncthreads();
    }
    if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

__global__ __launch_bounds__(kSortBlock) void sort_scatter_kernel(
    const uint64_t* __restrict__ keys_in, const int32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
    int32_t* __restrict__ vals_out, int64_t n, int shift, uint32_t mask, int n_bits, uint32_t n_blocks,
    const uint32_t* __restrict__ hist, const uint32_t* __restrict__ totals) {
    __shared__ uint32_t wcount[kSortWaves][kRadix];   // per-wave running digit counts, then bases
    __shared__ uint32_t ws[kSortWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int w = 0; w < kSortWaves; w++) wcount[w][threadIdx.x] = 0;
    // exclusive scan of the 256 digit totals, done by every workgroup for itself (a kernel of its own
    // for these 1 KB would cost a launch per pass): thread t ends up with the first position of digit t
    uint32_t digit_base;
    {
        const uint32_t v = totals[threadIdx.x];
        uint32_t inc = v;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = __shfl_up(inc, d, 64);
            if (lane >= d) inc += o;
        }
        if (lane == 63) ws[wave] = inc;
        __syncthreads();
        uint32_t base = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) { if (w < wave) base += ws[w]; }
        digit_base = base + inc - v;
    }

    const int64_t wave_base = (int64_t)blockIdx.x * kSortTile + (int64_t)wave * (kSortRounds * 64);
    uint64_t key[kSortRounds];
    int32_t val[kSortRounds];
    uint32_t off[kSortRounds];
    const uint64_t lt_mask = (1ull << lane) - 1ull;
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = wave_base + r * 64 + lane;
        const bool live = i < n;
        key[r] = live ? keys_in[i] : 0;
        val[r] = live ? vals_in[i] : 0;
        const uint32_t d = digit_of(key[r], shift, mask);
        // lanes holding the same digit (and alive): intersect one ballot per digit bit
        uint64_t peers = __ballot(live);
        for (int b = 0; b < n_bits; b++) {
            const uint64_t vote = __ballot((d >> b) & 1u);
            peers &= ((d >> b) & 1u) ? vote : ~vote;
        }
        uint32_t prev = 0;
        if (live) {
            prev = wcount[wave][d];          // count from earlier rounds of this wave
        }
        // every peer has read before the leader updates: same wavefront, program order on LDS
        __builtin_amdgcn_wave_barrier();
        if (live && (peers & lt_mask) == 0) wcount[wave][d] = prev + (uint32_t)__popcll(peers);
        __builtin_amdgcn_wave_barrier();
        off[r] = prev + (uint32_t)__popcll(peers & lt_mask);
    }
    __syncthreads();
    {   // thread t owns digit t: turn per-wave counts into global positions of each wave's first key
        const uint32_t d = threadIdx.x;
        uint32_t run = digit_base + hist[(size_t)d * n_blocks + blockIdx.x];
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) {
            const uint32_t c = wcount[w][d];
            wcount[w][d] = run;
            run += c;
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = wave_base + r * 64 + lane;
        if (i < n) {
            const uint32_t pos = wcount[wave][digit_of(key[r], shift, mask)] + off[r];
            keys_out[pos] = key[r];
            vals_out[pos] = val[r];
        }
    }
}

}  // namespace ssr

using namespace ssr;

extern "C" {

size_t ssr_sort_scratch_bytes(int64_t n) {
    if (n <= 0) return 0;
    const size_t nb = (size_t)ceil_div(n, kSortTile);
    return (nb * kRadix + kRadix) * sizeof(uint32_t);
}

int ssr_sort_pairs_u64_i32(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b, int64_t n,
                           int begin_bit, int end_bit, int* selector, void* scratch, size_t scratch_bytes,
                           ssr_stream_t stream) {
    SSR_REQUIRE(selector, "ssr_sort_pairs_u64_i32", "null selector");
    *selector = 0;
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, "ssr_sort_pairs_u64_i32", "count out of range");
    SSR_REQUIRE(begin_bit >= 0 && end_bit <= 64 && begin_bit <= end_bit, "ssr_sort_pairs_u64_i32", "bad bit range");
    if (n == 0 || begin_bit == end_bit) return 0;
    SSR_REQUIRE(keys_a && keys_b && vals_a && vals_b, "ssr_sort_pairs_u64_i32", "null buffer");
    SSR_REQUIRE(scratch && scratch_bytes >= ssr_sort_scratch_bytes(n), "ssr_sort_pairs_u64_i32", "scratch too small");
    const uint32_t nb = (uint32_t)ceil_div(n, kSortTile);
    uint32_t* hist = reinterpret_cast<uint32_t*>(scratch);
    uint32_t* totals = hist + (size_t)nb * kRadix;
    hipStream_t s = as_stream(stream);
    uint64_t* k[2] = {reinterpret_cast<uint64_t*>(keys_a), reinterpret_cast<uint64_t*>(keys_b)};
    int32_t* v[2] = {vals_a, vals_b};
    int cur = 0;
    for (int shift = begin_bit; shift < end_bit; shift += 8) {
        const int bits = end_bit - shift < 8 ? end_bit - shift : 8;
        const uint32_t mask = (1u << bits) - 1u;
        hipLaunchKernelGGL(sort_hist_kernel, dim3(nb), dim3(kSortBlock), 0, s, k[cur], n, shift, mask, nb, hist);
        hipLaunchKernelGGL(sort_scan_rows_kernel, dim3(kRadix), dim3(kSortBlock), 0, s, hist, nb, totals);
        hipLaunchKernelGGL(sort_scatter_kernel, dim3(nb), dim3(kSortBlock), 0, s, k[cur], v[cur], k[cur ^ 1], v[cur ^ 1], n,
                           shift, mask, bits, nb, hist, totals);
        cur ^= 1;
    }
    SSR_CHECK_LAUNCH("ssr_sort_pairs_u64_i32");
    *selector = cur;
    return 0;
}

}  // extern "C"
