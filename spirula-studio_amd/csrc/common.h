// common.h -- shared host/device helpers of libssr_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string>

#include "../../include/ssr_backend.h"
#include "../../include/ssr_math.h"

namespace ssr {

constexpr int kTile = 16;    // binning tile: TILE_SIZE_X * MACRO_TILE_SIZE_X (src/core/Common.cuh:36-39)
constexpr int kMicro = 8;    // compositing sub-tile: TILE_SIZE_X
constexpr float kAlphaThreshold = 1.0f / 255.0f;   // src/core/Common.cuh:47
constexpr float kTransmitThreshold = 1e-4f;        // src/kernels/tile/IntersectTile.cu:25

// Per-thread sticky error (returned and cleared by ssr_last_error()).
void set_error(const std::string& msg);
int fail(const char* where, const std::string& msg);
int check_hip(hipError_t e, const char* where);

inline hipStream_t as_stream(ssr_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Resolves the current device's address of the scan workspace that ssr_inclusive_sum_i64_static
// uses (tiles.hip); ssr_init calls it so that the first scan does not pay for it.
int warm_static_scan();

#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__) && !defined(__gfx942__) && !defined(__gfx90a__)
#error "lds_wait() encodes s_waitcnt for the gfx9 family: on another target the same bits name other counters"
#endif
// Waits until every LDS (and scalar-memory) operation this wavefront has issued is complete: s_waitcnt lgkmcnt(0)
// in the gfx9 encoding (vmcnt 63, expcnt 7 left alone). Placed ahead of a workgroup barrier that follows
// non-returning LDS float atomics, whose completion the kernels here do not leave to the compiler.
__device__ __forceinline__ void lds_wait() { __builtin_amdgcn_s_waitcnt(0xc07f); }
// A workgroup barrier that orders LDS traffic only: every LDS operation of this wavefront is complete, then the
// barrier. Unlike __syncthreads() it does not wait for vector-memory operations in flight (global atomics whose
// results nobody reads, rows on their way from memory into LDS for a later batch) -- the release fence of
// __syncthreads() would, at every barrier. Neither builtin may be moved across by the compiler, nor memory accesses
// across them. Data that arrives in LDS from memory needs its own vmcnt wait ahead of the barrier that publishes it.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_s_barrier();
}
// Waits until every vector-memory operation this wavefront has issued is complete, loads into LDS included:
// s_waitcnt vmcnt(0) in the gfx9 encoding (the six vmcnt bits are [3:0] and [15:14]).
__device__ __forceinline__ void vmem_wait() { __builtin_amdgcn_s_waitcnt(0x0f70); }

}  // namespace ssr

#define SSR_CHECK_LAUNCH(where)                                       \
    do {                                                              \
        int _e = ssr::check_hip(hipGetLastError(), where);            \
        if (_e) return _e;                                            \
    } while (0)

#define SSR_REQUIRE(cond, where, msg)                                 \
    do {                                                              \
        if (!(cond)) return ssr::fail(where, msg);                    \
    } while (0)
