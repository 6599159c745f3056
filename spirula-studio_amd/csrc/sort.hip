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
constexpr int kSortRounds = 8;                          // keys per lane
constexpr int kSortTile = kSortBlock * kSortRounds;     // 2048 keys per workgroup
constexpr int kRadix = 256;

__device__ __forceinline__ uint32_t digit_of(uint64_t key, int shift, uint32_t mask) {
    return (uint32_t)(key >> shift) & mask;
}

// For each lane: the number of live lanes below it that hold the same 8-bit digit (its rank among its
// peers), and the size of that peer group. One ballot per digit bit set in `varying` (the caller knows
// the other bits to be the same in every live lane); a lane differs from this one when any bit's vote
// disagrees with its own bit (vote XOR own bit, OR-ed over the bits).
template <int kBits = 8>
__device__ __forceinline__ void wave_match_digit(uint32_t d, uint32_t varying, bool live, uint32_t& rank, uint32_t& group) {
    uint32_t differ_lo = 0, differ_hi = 0;
#pragma unroll
    for (int b = 0; b < kBits; b++) {
        if ((varying >> b) & 1u) {
            const uint32_t own = (uint32_t)__builtin_amdgcn_sbfe((int)d, (uint32_t)b, 1u);   // 0 or ~0
            const uint64_t vote = __ballot(own != 0u);
            differ_lo |= (uint32_t)vote ^ own;
            differ_hi |= (uint32_t)(vote >> 32) ^ own;
        }
    }
    const uint64_t alive = __ballot(live);
    const uint32_t peers_lo = ~differ_lo & (uint32_t)alive, peers_hi = ~differ_hi & (uint32_t)(alive >> 32);
    rank = __builtin_amdgcn_mbcnt_hi(peers_hi, __builtin_amdgcn_mbcnt_lo(peers_lo, 0u));
    group = (uint32_t)__popc(peers_lo) + (uint32_t)__popc(peers_hi);
}

// hist[d * n_blocks + block]
// n_dev (optional): the real number of keys, on the device, where the host only knows an upper bound n; workgroups
// behind it leave at once.
__global__ __launch_bounds__(kSortBlock) void sort_hist_kernel(const uint64_t* __restrict__ keys, int64_t n,
                                                               const int64_t* __restrict__ n_dev, int shift,
                                                               uint32_t mask, uint32_t n_blocks,
                                                               uint32_t* __restrict__ hist, uint32_t* clear4) {
    __shared__ uint32_t lh[kRadix];
    if (n_dev) n = min(n, *n_dev);
    if (clear4 && blockIdx.x == 0 && threadIdx.x < 4) clear4[threadIdx.x] = 0;   // counters of a later kernel on this stream
    if ((int64_t)blockIdx.x * kSortTile >= n) return;   // behind the keys: its column is never read (sort_scan_rows_kernel)
    lh[threadIdx.x] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kSortTile;
    uint64_t k[kSortRounds];   // all loads ahead of the counting
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = base + r * kSortBlock + threadIdx.x;
        k[r] = i < n ? keys[i] : 0;
    }
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = base + r * kSortBlock + threadIdx.x;
        if (i < n) atomicAdd(&lh[digit_of(k[r], shift, mask)], 1u);
    }
    __syncthreads();
    hist[(size_t)threadIdx.x * n_blocks + blockIdx.x] = lh[threadIdx.x];
}

// One workgroup per digit: exclusive scan of its row of per-workgroup counts; row total out.
// (rows of n_blocks columns; only the columns of workgroups that hold keys were written: the first n_used)
__global__ __launch_bounds__(kSortBlock) void sort_scan_rows_kernel(uint32_t* __restrict__ hist, uint32_t n_blocks,
                                                                    uint32_t* __restrict__ totals, int64_t n,
                                                                    const int64_t* __restrict__ n_dev) {
    __shared__ uint32_t ws[2][kSortWaves];   // two sets in turn: one barrier a chunk is enough
    uint32_t* row = hist + (size_t)blockIdx.x * n_blocks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t carry = 0;
    if (n_dev) n = min(n, *n_dev);
    const uint32_t n_used = (uint32_t)((n + kSortTile - 1) / kSortTile);
    n_blocks = min(n_blocks, n_used);
    // a row is a few thousand counts and this kernel nothing but their latency: eight chunks of 256 are loaded
    // together, then scanned one after the other
    constexpr int kAhead = 8;
    int flip = 0;
    for (uint32_t start = 0; start < n_blocks; start += kSortBlock * kAhead) {
        uint32_t v[kAhead];
#pragma unroll
        for (int k = 0; k < kAhead; k++) {
            const uint32_t i = start + k * kSortBlock + threadIdx.x;
            v[k] = i < n_blocks ? row[i] : 0;
        }
#pragma unroll
        for (int k = 0; k < kAhead; k++) {
            if (start + k * kSortBlock >= n_blocks) break;   // the same for the whole workgroup
            const uint32_t i = start + k * kSortBlock + threadIdx.x;
            uint32_t inc = v[k];
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const uint32_t o = __shfl_up(inc, d, 64);
                if (lane >= d) inc += o;
            }
            if (lane == 63) ws[flip][wave] = inc;
            __syncthreads();
            uint32_t base = 0, total = 0;
#pragma unroll
            for (int w = 0; w < kSortWaves; w++) { if (w < wave) base += ws[flip][w]; total += ws[flip][w]; }
            if (i < n_blocks) row[i] = carry + base + inc - v[k];
            carry += total;
            flip ^= 1;
        }
    }
    if (threadIdx.x == 0) totals[blockIdx.x] = carry;
}

__global__ __launch_bounds__(kSortBlock) void sort_scatter_kernel(
    const uint64_t* __restrict__ keys_in, const int32_t* __restrict__ vals_in, uint64_t* __restrict__ keys_out,
    int32_t* __restrict__ vals_out, int64_t n, const int64_t* __restrict__ n_dev, int shift, uint32_t mask, uint32_t n_blocks,
    const uint32_t* __restrict__ hist, const uint32_t* __restrict__ totals) {
    if (n_dev) n = min(n, *n_dev);
    if ((int64_t)blockIdx.x * kSortTile >= n) return;   // nothing of this workgroup's is real (the whole workgroup leaves)
    __shared__ uint32_t wcount[kSortWaves][kRadix];   // per-wave running digit counts, then bases
    __shared__ uint32_t ws[kSortWaves], ws2[kSortWaves];
    __shared__ uint32_t s_shift[kRadix];
    // The pairs pass through LDS in digit order, keys first and the values after them through the same 16 KB:
    // 21 KB a workgroup leave room for seven of them on a compute unit (29 KB for five), which is one round of
    // workgroups instead of two for the 3.4 M keys of the 1080p benchmark scene.
    __shared__ uint64_t s_key[kSortTile];
    int32_t* s_val = reinterpret_cast<int32_t*>(s_key);
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
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = wave_base + r * 64 + lane;
        const bool live = i < n;
        key[r] = live ? keys_in[i] : 0;
        val[r] = live ? vals_in[i] : 0;
        const uint32_t d = digit_of(key[r], shift, mask);
        uint32_t rank, group;
        wave_match_digit(d, mask, live, rank, group);
        uint32_t prev = 0;
        if (live) {
            prev = wcount[wave][d];          // count from earlier rounds of this wave
        }
        // every peer has read before the leader updates: same wavefront, program order on LDS
        __builtin_amdgcn_wave_barrier();
        if (live && rank == 0) wcount[wave][d] = prev + group;
        __builtin_amdgcn_wave_barrier();
        off[r] = prev + rank;
    }
    __syncthreads();
    {   // thread t owns digit t: per-wave counts become positions, inside this workgroup's keys in digit
        // order, of each wave's first key of the digit; s_shift[t] = where the digit's run goes in the output
        // minus where it starts in that order
        const uint32_t d = threadIdx.x;
        uint32_t c[kSortWaves], block_count = 0;
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) { c[w] = wcount[w][d]; block_count += c[w]; }
        uint32_t inc = block_count;
#pragma unroll
        for (int k = 1; k < 64; k <<= 1) {
            const uint32_t o = __shfl_up(inc, k, 64);
            if (lane >= k) inc += o;
        }
        if (lane == 63) ws2[wave] = inc;
        __syncthreads();
        uint32_t local = inc - block_count;
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) { if (w < wave) local += ws2[w]; }
        s_shift[d] = digit_base + hist[(size_t)d * n_blocks + blockIdx.x] - local;
        uint32_t run = local;
#pragma unroll
        for (int w = 0; w < kSortWaves; w++) { wcount[w][d] = run; run += c[w]; }
    }
    __syncthreads();
    // stage the pairs in digit order, then write them out in that order: neighbouring lanes write
    // neighbouring addresses wherever a digit's run is longer than one key
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = wave_base + r * 64 + lane;
        if (i < n) {
            off[r] = wcount[wave][digit_of(key[r], shift, mask)] + off[r];   // the pair's place in digit order
            s_key[off[r]] = key[r];
        }
    }
    __syncthreads();
    const int64_t block_base = (int64_t)blockIdx.x * kSortTile;
    const int block_n = (int)(n - block_base < kSortTile ? n - block_base : kSortTile);
    uint32_t dst[kSortRounds];
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int j = r * kSortBlock + threadIdx.x;
        if (j < block_n) {
            const uint64_t k = s_key[j];
            dst[r] = s_shift[digit_of(k, shift, mask)] + (uint32_t)j;
            keys_out[dst[r]] = k;
        }
    }
    __syncthreads();   // the keys are out of LDS
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int64_t i = wave_base + r * 64 + lane;
        if (i < n) s_val[off[r]] = val[r];
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kSortRounds; r++) {
        const int j = r * kSortBlock + threadIdx.x;
        if (j < block_n) vals_out[dst[r]] = s_val[j];
    }
}

// ---- Tile-segmented variant ---------------------------------------------------------------------
// Keys are (tile id << 32) | depth bits. A stable sort on the tile bits alone leaves every tile's
// entries contiguous and in input order; a stable sort of each such segment on the depth bits then
// gives the same order as a stable sort on the whole key. Only the tile-bit passes stream the whole
// key array through HBM; a segment is sorted by one workgroup, in LDS when it fits.

// Ranks the wave's 64 keys of one round by `d` (8 bits): returns the number of earlier keys of this wave
// with the same digit, and advances the wave's running count (wcount_row = this wave's 256 counters).
template <int kBits = 8>
__device__ __forceinline__ uint32_t seg_rank_round(uint32_t d, uint32_t varying, bool live, uint32_t* wcount_row) {
    uint32_t rank, group;
    wave_match_digit<kBits>(d, varying, live, rank, group);
    uint32_t prev = 0;
    if (live) prev = wcount_row[d];
    __builtin_amdgcn_wave_barrier();
    if (live && rank == 0) wcount_row[d] = prev + group;
    __builtin_amdgcn_wave_barrier();
    return prev + rank;
}

// Per-wave digit counts become the segment-local position of each wave's first key of that digit. Called by the
// whole workgroup (barriers inside). With at least as many digits as threads every thread owns a run of consecutive
// digits; else threads 0..kRadixT-1 own one each.
// radix_used: the digits in use (kRadixT, or fewer with the same divisibility), the others are not touched.
template <int kWaves, int kRadixT = kRadix>
__device__ __forceinline__ void seg_digit_bases(uint32_t (*wcount)[kRadixT], uint32_t* ws, int radix_used = kRadixT) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int kThreads = kWaves * 64;
    if constexpr (kRadixT >= kThreads) {
        constexpr int kPer = kRadixT / kThreads;
        static_assert(kPer * kThreads == kRadixT && kWaves <= kRadix / 64, "whole runs of digits; ws holds one total per wavefront");
        const int per = radix_used / kThreads;   // this thread's digits: threadIdx.x * per .. + per - 1
        uint32_t c[kWaves][kPer];
        uint32_t total = 0;
#pragma unroll
        for (int j = 0; j < kPer; j++)
#pragma unroll
            for (int w = 0; w < kWaves; w++) { c[w][j] = j < per ? wcount[w][threadIdx.x * per + j] : 0u; total += c[w][j]; }
        uint32_t inc = total;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = __shfl_up(inc, d, 64);
            if (lane >= d) inc += o;
        }
        uint32_t run = inc - total;
        if constexpr (kWaves > 1) {
            if (lane == 63) ws[wave] = inc;
            __syncthreads();   // also: every count is read before any base is written
#pragma unroll
            for (int w = 0; w < kWaves; w++) { if (w < wave) run += ws[w]; }
        }
#pragma unroll
        for (int j = 0; j < kPer; j++)
#pragma unroll
            for (int w = 0; w < kWaves; w++) { if (j < per) { wcount[w][threadIdx.x * per + j] = run; run += c[w][j]; } }
        __syncthreads();
        return;
    }
    const bool owner = threadIdx.x < kRadixT;
    uint32_t total = 0, inc = 0;
    if (owner) {
#pragma unroll
        for (int w = 0; w < kWaves; w++) total += wcount[w][threadIdx.x];
        inc = total;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const uint32_t o = __shfl_up(inc, d, 64);
            if (lane >= d) inc += o;
        }
        if (lane == 63) ws[wave] = inc;
    }
    __syncthreads();
    if (owner) {
        uint32_t run = inc - total;
#pragma unroll
        for (int w = 0; w < kRadixT / 64; w++) { if (w < wave) run += ws[w]; }
#pragma unroll
        for (int w = 0; w < kWaves; w++) {
            const uint32_t c = wcount[w][threadIdx.x];
            wcount[w][threadIdx.x] = run;
            run += c;
        }
    }
    __syncthreads();
}

// OR over the workgroup of `x` (the key bits that differ inside the segment): a digit whose bits are
// all clear in it is the same for every key, and its pass moves nothing.
template <int kWaves>
__device__ __forceinline__ uint32_t seg_or_all(uint32_t x, uint32_t* wor) {
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) x |= __shfl_xor(x, d, 64);
    if ((threadIdx.x & 63) == 0) wor[threadIdx.x >> 6] = x;
    __syncthreads();
    uint32_t all = 0;
#pragma unroll
    for (int w = 0; w < kWaves; w++) all |= wor[w];
    return all;
}

constexpr int kSegWideFrom = 192;   // keys from which a segment takes the wider digits
// The workgroup (kWaves wavefronts) sorts keys[s, s + len), len <= 64 * kWaves * kRounds, in place on the
// low 32 key bits: keys in registers, one LDS round trip per digit pass. Digits are 8 bits at bits 0, 8, 16, 24;
// with kDigitBits = 9 (512 counters a wavefront) a segment of kSegWideFrom keys or more whose differing bits fit
// fewer 9-bit digits takes those, cut evenly over the span (25 depth bits differ across a tile of the 1080p
// benchmark scene: four 8-bit passes, three 9-bit ones).
template <int kWaves, int kRounds, int kDigitBits = 8>
__device__ __forceinline__ void seg_sort_lds(uint64_t* keys, int32_t* vals, int64_t s, int len,
                                             uint32_t (*wcount)[1 << kDigitBits], uint32_t* ws, uint32_t* wor, uint2* buf) {
    constexpr int kRadixT = 1 << kDigitBits;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_wave = ((len + kWaves - 1) / kWaves + 63) & ~63;   // contiguous run per wave
    const int rounds = per_wave >> 6;
    const int first = wave * per_wave + lane;
    const uint64_t key0 = keys[s];
    const uint32_t hi = (uint32_t)(key0 >> 32);

    uint32_t key[kRounds], off[kRounds];
    int32_t val[kRounds];
    uint32_t differ = 0;
#pragma unroll
    for (int r = 0; r < kRounds; r++) {
        const int i = first + r * 64;
        const bool live = r < rounds && i < len;
        key[r] = live ? (uint32_t)keys[s + i] : (uint32_t)key0;
        val[r] = live ? vals[s + i] : 0;
        differ |= key[r] ^ (uint32_t)key0;
    }
    differ = seg_or_all<kWaves>(differ, wor);
    if (differ == 0) return;   // all keys equal: already in order
    // 8-bit digits at bits 0, 8, 16, 24, those that are the same in every key skipped; or, where the counters allow
    // wider digits and that saves a pass on a segment long enough to feel it, equal digits over the span
    int lsb = 0, width = 8;
    if constexpr (kDigitBits > 8) {
        const int lo = __ffs((int)differ) - 1, span = 32 - __clz((int)differ) - lo;
        const int wide = (span + kDigitBits - 1) / kDigitBits;
        const int bytes = ((differ & 0xffu) != 0) + ((differ & 0xff00u) != 0) + ((differ & 0xff0000u) != 0) + ((differ >> 24) != 0);
        if (len >= kSegWideFrom && wide < bytes) { lsb = lo; width = (span + wide - 1) / wide; }
    }
    const uint32_t mask = (1u << width) - 1u;
    const int radix_used = width > 8 ? kRadixT : kRadix;
    int last_shift = lsb;   // the last pass that moves anything writes straight to the output
    for (int shift = lsb; shift < 32; shift += width) { if ((differ >> shift) & mask) last_shift = shift; }
#pragma unroll 1
    for (int shift = lsb; shift <= last_shift; shift += width) {
        if (((differ >> shift) & mask) == 0) continue;
#pragma unroll
        for (int e = 0; e < kRadixT / 64; e++) { if (64 * e < radix_used) wcount[wave][lane + 64 * e] = 0; }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < kRounds; r++) {
            if (r < rounds) {
                const bool live = first + r * 64 < len;
                off[r] = seg_rank_round<kDigitBits>((key[r] >> shift) & mask, (differ >> shift) & mask, live, wcount[wave]);
            }
        }
        __syncthreads();
        seg_digit_bases<kWaves, kRadixT>(wcount, ws, radix_used);
        if (shift == last_shift) {
#pragma unroll
            for (int r = 0; r < kRounds; r++) {
                if (r < rounds && first + r * 64 < len) {
                    const uint32_t pos = wcount[wave][(key[r] >> shift) & mask] + off[r];
                    keys[s + pos] = ((uint64_t)hi << 32) | key[r];
                    vals[s + pos] = val[r];
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < kRounds; r++) {
                if (r < rounds && first + r * 64 < len) {
                    const uint32_t pos = wcount[wave][(key[r] >> shift) & mask] + off[r];
                    buf[pos] = make_uint2(key[r], (uint32_t)val[r]);
                }
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < kRounds; r++) {
                if (r < rounds && first + r * 64 < len) {
                    const uint2 kv = buf[first + r * 64];
                    key[r] = kv.x;
                    val[r] = (int32_t)kv.y;
                }
            }
            // the barrier after the next pass's clearing of wcount also orders these reads of buf before
            // that pass's writes to it
        }
    }
}

// Work lists of the tiles whose segments are too long for the direct kernel, by size class:
// counts[c] entries in list[c]; class 0 up to kSegCap0 keys, class 1 up to kSegCap1, class 2 beyond.
struct SegLists { uint32_t* counts; uint32_t* list[3]; bool has_class0; };
constexpr int kSegCap0 = 4 * 64 * 8;           // four wavefronts, 8 keys per lane
constexpr int kSegCap1 = 16 * 64 * 8;          // sixteen wavefronts, 8 keys per lane

// End of tile `tile`'s segment. n < 0: the offsets hold one entry more, which ends the last tile (the host does
// not know the number of keys).
__device__ __forceinline__ int64_t seg_end(const int32_t* __restrict__ tile_offsets, uint32_t tile, uint32_t n_tiles, int64_t n) {
    return (tile + 1 < n_tiles || n < 0) ? (int64_t)tile_offsets[tile + 1] : n;
}

// Digit width of a segment sort: a lone wavefront sorts a segment of several rounds faster in three 9-bit passes than
// in four 8-bit ones (config 5, 336 keys a tile: 105 -> 83 us); four wavefronts, whose passes are mostly barriers,
// and short segments do not (measured: +1.5 us on configs 1 and 3, +3.5 on config 4's 100-key tiles).
template <int kWaves> constexpr int seg_digit_bits() { return kWaves == 1 ? 9 : 8; }
// One workgroup of kWaves wavefronts per tile: sorts segments of 2..64*kWaves*kRounds keys, lists the
// longer ones. These kernels are bound by instruction issue: one wavefront per tile executes the fewest
// instructions per key, but its tiles take long, so it pays only when there are several rounds of
// workgroups to balance the compute units; four wavefronts per tile otherwise.
template <int kWaves, int kRounds>
__global__ __launch_bounds__(kWaves * 64) void sort_segments_direct_kernel(uint64_t* keys, int32_t* vals,
                                                                           const int32_t* __restrict__ tile_offsets,
                                                                           uint32_t n_tiles, int64_t n, SegLists lists) {
    constexpr int kCap = kWaves * 64 * kRounds;
    static_assert(kCap <= kSegCap0, "class 0 starts above the direct kernel's capacity");
    __shared__ __attribute__((aligned(16))) uint32_t wcount[kWaves][1 << seg_digit_bits<kWaves>()];
    __shared__ uint32_t ws[kRadix / 64];
    __shared__ uint32_t wor[kWaves];
    __shared__ uint2 buf[kCap];
    const uint32_t tile = blockIdx.x;
    const int64_t s = tile_offsets[tile];
    const int64_t e = seg_end(tile_offsets, tile, n_tiles, n);
    const int len = (int)(e - s);
    if (len <= 1) return;
    if (len > kCap) {
        if (threadIdx.x == 0) {
            // class 0 exists only where a kernel for it follows: otherwise everything up to kSegCap1 is class 1
            const int c = len > kSegCap1 ? 2 : (len > kSegCap0 || !lists.has_class0) ? 1 : 0;
            lists.list[c][atomicAdd(&lists.counts[c], 1u)] = tile;
        }
        return;
    }
    seg_sort_lds<kWaves, kRounds, seg_digit_bits<kWaves>()>(keys, vals, s, len, wcount, ws, wor, buf);
}

// Workgroups of four wavefronts take the listed segments of class 0 in turn.
__global__ __launch_bounds__(256) void sort_segments_small_kernel(uint64_t* keys, int32_t* vals,
                                                                  const int32_t* __restrict__ tile_offsets, uint32_t n_tiles,
                                                                  int64_t n, SegLists lists) {
    __shared__ uint32_t wcount[4][kRadix];
    __shared__ uint32_t ws[kRadix / 64];
    __shared__ uint32_t wor[4];
    __shared__ uint2 buf[kSegCap0];
    static_assert(kSegCap0 == 4 * 64 * 8, "class 0 is sorted by four wavefronts with 8 keys per lane");
    const uint32_t count = lists.counts[0];
    for (uint32_t idx = blockIdx.x; idx < count; idx += gridDim.x) {
        const uint32_t tile = lists.list[0][idx];
        const int64_t s = tile_offsets[tile];
        const int64_t e = seg_end(tile_offsets, tile, n_tiles, n);
        seg_sort_lds<4, 8>(keys, vals, s, (int)(e - s), wcount, ws, wor, buf);
        __syncthreads();   // LDS is reused by the next segment
    }
}

// The workgroup (16 wavefronts) sorts keys[s, s + len) of any length on the low 32 key bits: four digit
// passes through global memory, between that range of (keys, vals) and the same range of the second
// buffer pair; the result ends where it started.
constexpr int kSegGlobalWaves = 16;
__device__ __forceinline__ void seg_sort_global(uint64_t* keys, int32_t* vals, uint64_t* keys_alt, int32_t* vals_alt, int64_t s,
                                                int len, uint32_t (*wcount)[kRadix], uint32_t* ws) {
    constexpr int kWaves = kSegGlobalWaves;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int per_wave = ((len + kWaves - 1) / kWaves + 63) & ~63;
    const int w_begin = wave * per_wave;
    const int w_end = min(len, w_begin + per_wave);
    uint64_t* k_src = keys + s; uint64_t* k_dst = keys_alt + s;
    int32_t* v_src = vals + s; int32_t* v_dst = vals_alt + s;
#pragma unroll 1
    for (int shift = 0; shift < 32; shift += 8) {
        wcount[wave][lane] = wcount[wave][lane + 64] = wcount[wave][lane + 128] = wcount[wave][lane + 192] = 0;
        __syncthreads();
#pragma unroll 4
        for (int i = w_begin + lane; i < w_end; i += 64) {
            const uint64_t k = __hip_atomic_load(k_src + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            atomicAdd(&wcount[wave][(uint32_t)(k >> shift) & 255u], 1u);
        }
        __syncthreads();
        seg_digit_bases<kWaves>(wcount, ws);
        // wcount[wave][d] now runs: the next free position of digit d for this wave
        uint64_t k_next = 0; int32_t v_next = 0;
        if (w_begin + lane < w_end) {
            k_next = __hip_atomic_load(k_src + w_begin + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            v_next = __hip_atomic_load(v_src + w_begin + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
        for (int i0 = w_begin; i0 < w_end; i0 += 64) {
            const uint64_t k = k_next; const int32_t v = v_next;
            const bool live = i0 + lane < w_end;
            const int j = i0 + 64 + lane;   // the next round's pair is in flight while this one is ranked
            if (j < w_end) {
                k_next = __hip_atomic_load(k_src + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                v_next = __hip_atomic_load(v_src + j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
            const uint32_t pos = seg_rank_round((uint32_t)(k >> shift) & 255u, 255u, live, wcount[wave]);
            if (live) {
                __hip_atomic_store(k_dst + pos, k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                __hip_atomic_store(v_dst + pos, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
        __syncthreads();   // workgroup-scope release/acquire: the next pass reads what this one wrote
        uint64_t* tk = k_src; k_src = k_dst; k_dst = tk;
        int32_t* tv = v_src; v_src = v_dst; v_dst = tv;
    }
}

// Workgroups of sixteen wavefronts take the listed segments of class 2 (through global memory), then of class 1
// (in LDS), longest class first, each workgroup drawing its next segment from a shared cursor when it has
// finished one (segment lengths differ eightfold, so a fixed assignment leaves workgroups idle at the end).
// lists.counts[3] is the cursor: zero at launch.
__global__ __launch_bounds__(kSegGlobalWaves * 64) void sort_segments_long_kernel(
    uint64_t* keys, int32_t* vals, uint64_t* keys_alt, int32_t* vals_alt, const int32_t* __restrict__ tile_offsets,
    uint32_t n_tiles, int64_t n, SegLists lists) {
    __shared__ uint32_t wcount[kSegGlobalWaves][kRadix];
    __shared__ uint32_t ws[kRadix / 64];
    __shared__ uint32_t wor[kSegGlobalWaves];
    __shared__ uint2 buf[kSegCap1];
    __shared__ uint32_t s_next;
    static_assert(kSegCap1 == kSegGlobalWaves * 64 * 8, "class 1 is sorted by sixteen wavefronts with 8 keys per lane");
    const uint32_t count1 = lists.counts[1], count2 = lists.counts[2];
    if (count1 + count2 == 0) return;   // nothing listed: no workgroup touches the cursor
    for (;;) {
        if (threadIdx.x == 0) s_next = atomicAdd(&lists.counts[3], 1u);
        __syncthreads();
        const uint32_t idx = s_next;
        if (idx >= count1 + count2) break;   // the same value in every thread: the workgroup leaves together
        const uint32_t tile = idx < count2 ? lists.list[2][idx] : lists.list[1][idx - count2];
        const int64_t s = tile_offsets[tile];
        const int64_t e = seg_end(tile_offsets, tile, n_tiles, n);
        if (idx < count2) seg_sort_global(keys, vals, keys_alt, vals_alt, s, (int)(e - s), wcount, ws);
        else seg_sort_lds<kSegGlobalWaves, 8>(keys, vals, s, (int)(e - s), wcount, ws, wor, buf);
        __syncthreads();   // LDS, s_next included, is reused by the next segment
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

size_t ssr_sort_tile_scratch_bytes(int64_t n, uint32_t n_tiles) {
    if (n <= 0) return 0;
    return ((ssr_sort_scratch_bytes(n) + 15) & ~(size_t)15) + (4 + 3 * (size_t)n_tiles) * sizeof(uint32_t);
}

// clear4 (optional): four counters that the first kernel launched here sets to zero
static int sort_pairs_impl(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b, int64_t n, int begin_bit,
                           int end_bit, int* selector, void* scratch, size_t scratch_bytes, ssr_stream_t stream,
                           uint32_t* clear4, const int64_t* n_dev = nullptr) {
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
    // as few passes as 8-bit digits allow, the bits spread evenly over them (13 tile bits: 7 + 6, not 8 + 5): the
    // scatter of a narrower digit writes longer runs, and no pass is left with the short runs of a full 256-way split
    int passes = (end_bit - begin_bit + 7) / 8;
    for (int shift = begin_bit, bits = 0; shift < end_bit; shift += bits, passes--) {
        bits = (end_bit - shift + passes - 1) / passes;
        const uint32_t mask = (1u << bits) - 1u;
        hipLaunchKernelGGL(sort_hist_kernel, dim3(nb), dim3(kSortBlock), 0, s, k[cur], n, n_dev, shift, mask, nb, hist,
                           shift == begin_bit ? clear4 : nullptr);
        hipLaunchKernelGGL(sort_scan_rows_kernel, dim3(kRadix), dim3(kSortBlock), 0, s, hist, nb, totals, n, n_dev);
        hipLaunchKernelGGL(sort_scatter_kernel, dim3(nb), dim3(kSortBlock), 0, s, k[cur], v[cur], k[cur ^ 1], v[cur ^ 1], n,
                           n_dev, shift, mask, nb, hist, totals);
        cur ^= 1;
    }
    SSR_CHECK_LAUNCH("ssr_sort_pairs_u64_i32");
    *selector = cur;
    return 0;
}

int ssr_sort_pairs_u64_i32(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b, int64_t n,
                           int begin_bit, int end_bit, int* selector, void* scratch, size_t scratch_bytes,
                           ssr_stream_t stream) {
    return sort_pairs_impl(keys_a, keys_b, vals_a, vals_b, n, begin_bit, end_bit, selector, scratch, scratch_bytes, stream,
                           nullptr);
}

// n_dev: only the first *n_dev (device) of the n entries are keys; tile_offsets then has n_tiles + 1 entries
static int sort_tile_pairs_impl(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b, int64_t n,
                                uint32_t n_tiles, int32_t* tile_offsets, int* selector, void* scratch, size_t scratch_bytes,
                                ssr_stream_t stream, const int64_t* n_dev) {
    const bool closed = n_dev != nullptr;
    SSR_REQUIRE(selector, "ssr_sort_tile_pairs", "null selector");
    *selector = 0;
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, "ssr_sort_tile_pairs", "count out of range");
    if (n_tiles == 0) return 0;
    SSR_REQUIRE(tile_offsets, "ssr_sort_tile_pairs", "null offsets");
    SSR_REQUIRE(n == 0 || (scratch && scratch_bytes >= ssr_sort_tile_scratch_bytes(n, n_tiles)), "ssr_sort_tile_pairs",
                "scratch too small");
    SegLists lists = {};
    if (n > 0) {
        lists.counts = reinterpret_cast<uint32_t*>(static_cast<char*>(scratch) + ((ssr_sort_scratch_bytes(n) + 15) & ~(size_t)15));
        for (int c = 0; c < 3; c++) lists.list[c] = lists.counts + 4 + (size_t)c * n_tiles;
    }
    const int end_bit = ssr_sort_end_bit(n_tiles);
    if (n > 0 && end_bit > 32) {   // partition by tile: stable on the tile bits only
        if (sort_pairs_impl(keys_a, keys_b, vals_a, vals_b, n, 32, end_bit, selector, scratch, scratch_bytes, stream, lists.counts,
                            n_dev))
            return 1;
    } else if (n > 0) {
        SSR_REQUIRE(keys_a && keys_b && vals_a && vals_b, "ssr_sort_tile_pairs", "null buffer");
        if (ssr_fill_u32(lists.counts, 0u, 4, stream)) return 1;
    }
    const int cur = *selector;
    int64_t* k[2] = {keys_a, keys_b};
    int32_t* v[2] = {vals_a, vals_b};
    if (closed ? ssr_tile_offsets_capped(n, n_dev, k[cur], n_tiles, tile_offsets, stream)
               : ssr_tile_offsets(n, k[cur], n_tiles, tile_offsets, stream))
        return 1;
    if (n <= 1) return 0;
    const int64_t n_host = n;   // sizes the launches
    if (closed) n = -1;         // the kernels end the last tile at tile_offsets[n_tiles]
    hipStream_t s = as_stream(stream);
    uint64_t* kc = reinterpret_cast<uint64_t*>(k[cur]);
    uint64_t* ka = reinterpret_cast<uint64_t*>(k[cur ^ 1]);
    // one wavefront per tile: at least two rounds of such workgroups on 256 compute units, and segments that mostly fit
    // its 512 keys (a mean of 336 does, config 5; a mean of 411 with a third of the tiles above 512 does not)
    const bool lone_waves = n_tiles >= 16384 && n_host / n_tiles <= 384;
    lists.has_class0 = lone_waves;
    if (lone_waves) {
        hipLaunchKernelGGL((sort_segments_direct_kernel<1, 8>), dim3(n_tiles), dim3(64), 0, s, kc, v[cur], tile_offsets, n_tiles,
                           n, lists);
    } else {
        // 8 keys per lane sort segments of up to 2048 keys directly, at the price of a slower kernel for short
        // segments: worth it where the mean segment is long
        if (n_host / n_tiles > 512)
            hipLaunchKernelGGL((sort_segments_direct_kernel<4, 8>), dim3(n_tiles), dim3(256), 0, s, kc, v[cur], tile_offsets,
                               n_tiles, n, lists);
        else
            hipLaunchKernelGGL((sort_segments_direct_kernel<4, 4>), dim3(n_tiles), dim3(256), 0, s, kc, v[cur], tile_offsets,
                               n_tiles, n, lists);
    }
    // the listed segments: fixed grids, a workgroup with no list entry ends at once
    if (lone_waves && n_host > 512)   // four wavefronts sort class 0 directly otherwise
        hipLaunchKernelGGL(sort_segments_small_kernel, dim3(n_tiles < 2048 ? n_tiles : 2048), dim3(256), 0, s, kc, v[cur],
                           tile_offsets, n_tiles, n, lists);
    if (n_host > (lone_waves ? kSegCap0 : 1024))
        hipLaunchKernelGGL(sort_segments_long_kernel, dim3(n_tiles < 512 ? n_tiles : 512), dim3(kSegGlobalWaves * 64), 0, s, kc,
                           v[cur], ka, v[cur ^ 1], tile_offsets, n_tiles, n, lists);
    SSR_CHECK_LAUNCH("ssr_sort_tile_pairs");
    return 0;
}

int ssr_sort_tile_pairs(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b, int64_t n,
                        uint32_t n_tiles, int32_t* tile_offsets, int* selector, void* scratch, size_t scratch_bytes,
                        ssr_stream_t stream) {
    return sort_tile_pairs_impl(keys_a, keys_b, vals_a, vals_b, n, n_tiles, tile_offsets, selector, scratch, scratch_bytes,
                                stream, nullptr);
}

int ssr_sort_tile_pairs_capped(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b, int64_t capacity,
                               const int64_t* n_isects, uint32_t n_tiles, int32_t* tile_offsets, int* selector, void* scratch,
                               size_t scratch_bytes, ssr_stream_t stream) {
    SSR_REQUIRE(n_tiles > 0 && n_tiles < 0x7fffffffu, "ssr_sort_tile_pairs_capped", "tile count out of range");
    SSR_REQUIRE(capacity > 0, "ssr_sort_tile_pairs_capped", "capacity must be positive");
    SSR_REQUIRE(n_isects, "ssr_sort_tile_pairs_capped", "null count");
    return sort_tile_pairs_impl(keys_a, keys_b, vals_a, vals_b, capacity, n_tiles, tile_offsets, selector, scratch, scratch_bytes,
                                stream, n_isects);
}

}  // extern "C"
