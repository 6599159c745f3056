// runtime.hip -- thin HIP runtime surface behind the C ABI: allocation, copies, fills, events
// and the per-thread sticky error. Mirrors the contract of the reference's backend runtime
// (src/backend/api/BackendRuntime.h:29-168); the behaviours its runtime smoke test spells out
// (src/backend/vulkan/tests/vk_runtime_smoke.cpp:44-160) are kept: malloc(0) is NULL, pinned
// host memory does not classify as a device pointer, a failing call reports once.
#include "common.h"
#include <stdlib.h>
#include <string.h>

#include <string.h>

namespace ssr {

static thread_local std::string g_error;
static thread_local std::string g_error_out;
static std::string g_device_name;

void set_error(const std::string& msg) {
    if (g_error.empty()) g_error = msg;   // first error wins until it is read
}
int fail(const char* where, const std::string& msg) {
    set_error(std::string(where) + ": " + msg);
    return 1;
}
int check_hip(hipError_t e, const char* where) {
    if (e == hipSuccess) return 0;
    set_error(std::string(where) + ": " + hipGetErrorString(e));
    return (int)e ? (int)e : 1;
}

__global__ void fill_u32_kernel(uint32_t* __restrict__ dst, uint32_t value, int64_t count) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    // 16-byte stores over the aligned body, scalar tail
    const int64_t n4 = count >> 2;
    uint4* d4 = reinterpret_cast<uint4*>(dst);
    const uint4 v4 = make_uint4(value, value, value, value);
    for (int64_t k = i; k < n4; k += stride) d4[k] = v4;
    for (int64_t k = (n4 << 2) + i; k < count; k += stride) dst[k] = value;
}

__global__ void fill_u8_kernel(uint8_t* __restrict__ dst, uint8_t value, int n) {
    int i = threadIdx.x;
    if (i < n) dst[i] = value;
}

__global__ void debug_math_kernel(int op, int64_t n, const float* a, const float* b, float* out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float r;
    switch (op) {
        case 0: r = ssr_exp(a[i]); break;
        case 1: r = ssr_log(a[i]); break;
        case 2: r = ssr_atan2(a[i], b[i]); break;
        case 4: r = ssr_adam_inv_bias1(a[i]); break;
        case 5: r = ssr_adam_inv_bias2(a[i]); break;
        default: r = ssr_sigmoid(a[i]); break;
    }
    out[i] = r;
}

}  // namespace ssr

using namespace ssr;

extern "C" {

const char* ssr_last_error(void) {
    g_error_out.swap(g_error);
    g_error.clear();
    return g_error_out.c_str();
}

int ssr_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) { (void)hipGetLastError(); return 0; }
    return n;
}

int ssr_init(int device) {
    int n = ssr_device_count();
    SSR_REQUIRE(n > 0, "ssr_init", "no HIP device visible");
    SSR_REQUIRE(device >= 0 && device < n, "ssr_init", "device index out of range");
    int e = check_hip(hipSetDevice(device), "ssr_init/hipSetDevice");
    if (e) return e;
    hipDeviceProp_t prop;
    e = check_hip(hipGetDeviceProperties(&prop, device), "ssr_init/hipGetDeviceProperties");
    if (e) return e;
    g_device_name = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    e = check_hip(hipFree(nullptr), "ssr_init/context");
    if (e) return e;
    return warm_static_scan();
}

const char* ssr_device_name(void) { return g_device_name.c_str(); }

void* ssr_device_malloc(size_t bytes) {
    if (bytes == 0) return nullptr;
    void* p = nullptr;
    if (check_hip(hipMalloc(&p, bytes), "ssr_device_malloc")) return nullptr;
    return p;
}

int ssr_device_free(void* ptr) {
    if (!ptr) return 0;
    int e = check_hip(hipDeviceSynchronize(), "ssr_device_free/sync");   // drain in-flight work first
    if (e) return e;
    return check_hip(hipFree(ptr), "ssr_device_free");
}

void* ssr_host_malloc_pinned(size_t bytes) {
    if (bytes == 0) return nullptr;
    void* p = nullptr;
    if (check_hip(hipHostMalloc(&p, bytes, hipHostMallocDefault), "ssr_host_malloc_pinned")) return nullptr;
    return p;
}

int ssr_host_free_pinned(void* ptr) {
    if (!ptr) return 0;
    return check_hip(hipHostFree(ptr), "ssr_host_free_pinned");
}

int ssr_is_device_pointer(const void* ptr) {
    if (!ptr) return 0;
    hipPointerAttribute_t attr;
    memset(&attr, 0, sizeof(attr));
    if (hipPointerGetAttributes(&attr, ptr) != hipSuccess) {
        (void)hipGetLastError();   // an unknown host pointer is not an error of ours
        return 0;
    }
    return attr.type == hipMemoryTypeDevice ? 1 : 0;
}

int ssr_memcpy(void* dst, const void* src, size_t bytes, int kind, ssr_stream_t stream, int async) {
    if (bytes == 0) return 0;
    SSR_REQUIRE(dst && src, "ssr_memcpy", "null pointer");
    if (kind == SSR_MEMCPY_AUTO) {
        const int d = ssr_is_device_pointer(dst), s = ssr_is_device_pointer(src);
        kind = d ? (s ? SSR_MEMCPY_D2D : SSR_MEMCPY_H2D) : (s ? SSR_MEMCPY_D2H : SSR_MEMCPY_H2H);
    }
    hipMemcpyKind k;
    switch (kind) {
        case SSR_MEMCPY_H2D: k = hipMemcpyHostToDevice; break;
        case SSR_MEMCPY_D2H: k = hipMemcpyDeviceToHost; break;
        case SSR_MEMCPY_D2D: k = hipMemcpyDeviceToDevice; break;
        case SSR_MEMCPY_H2H: k = hipMemcpyHostToHost; break;
        default: return fail("ssr_memcpy", "unknown copy kind");
    }
    int e = check_hip(hipMemcpyAsync(dst, src, bytes, k, as_stream(stream)), "ssr_memcpy");
    if (e || async) return e;
    return check_hip(hipStreamSynchronize(as_stream(stream)), "ssr_memcpy/sync");
}

int ssr_fill_u32(void* dst, uint32_t value, int64_t count, ssr_stream_t stream) {
    if (count <= 0) return 0;
    SSR_REQUIRE(dst, "ssr_fill_u32", "null pointer");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(dst) & 3) == 0, "ssr_fill_u32", "destination not 4-byte aligned");
    uint32_t* d = reinterpret_cast<uint32_t*>(dst);
    // peel to 16-byte alignment on the host side of the launch
    int64_t head = (int64_t)(((16 - (reinterpret_cast<uintptr_t>(d) & 15)) & 15) >> 2);
    if (head > count) head = count;
    if (head) {
        hipLaunchKernelGGL(fill_u32_kernel, dim3(1), dim3(64), 0, as_stream(stream), d, value, head);
        SSR_CHECK_LAUNCH("ssr_fill_u32");
        d += head; count -= head;
    }
    if (count) {
        const int block = 256;
        int64_t blocks = ceil_div(ceil_div(count, 4), block);
        if (blocks > 4096) blocks = 4096;
        if (blocks < 1) blocks = 1;
        hipLaunchKernelGGL(fill_u32_kernel, dim3((unsigned)blocks), dim3(block), 0, as_stream(stream), d, value, count);
        SSR_CHECK_LAUNCH("ssr_fill_u32");
    }
    return 0;
}

int ssr_memset(void* dst, int byte_value, size_t bytes, ssr_stream_t stream, int async) {
    if (bytes == 0) return 0;
    SSR_REQUIRE(dst, "ssr_memset", "null pointer");
    // Fill kernels rather than hipMemsetAsync, so that callers may capture this into a graph.
    uint8_t bv = (uint8_t)byte_value;
    uint32_t word = 0x01010101u * bv;
    uint8_t* p = reinterpret_cast<uint8_t*>(dst);
    size_t head = (4 - (reinterpret_cast<uintptr_t>(p) & 3)) & 3;
    if (head > bytes) head = bytes;
    int e = 0;
    if (head) {
        hipLaunchKernelGGL(fill_u8_kernel, dim3(1), dim3(64), 0, as_stream(stream), p, bv, (int)head);
        SSR_CHECK_LAUNCH("ssr_memset/head");
    }
    size_t words = (bytes - head) / 4;
    if (words) { e = ssr_fill_u32(p + head, word, (int64_t)words, stream); if (e) return e; }
    size_t tail = bytes - head - words * 4;
    if (tail) {
        hipLaunchKernelGGL(fill_u8_kernel, dim3(1), dim3(64), 0, as_stream(stream), p + head + words * 4, bv, (int)tail);
        SSR_CHECK_LAUNCH("ssr_memset/tail");
    }
    if (async) return 0;
    return check_hip(hipStreamSynchronize(as_stream(stream)), "ssr_memset/sync");
}

int ssr_device_synchronize(void) { return check_hip(hipDeviceSynchronize(), "ssr_device_synchronize"); }
int ssr_stream_synchronize(ssr_stream_t s) { return check_hip(hipStreamSynchronize(as_stream(s)), "ssr_stream_synchronize"); }

ssr_stream_t ssr_stream_create(void) {
    hipStream_t s = nullptr;
    if (check_hip(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "ssr_stream_create")) return nullptr;
    return reinterpret_cast<ssr_stream_t>(s);
}
int ssr_stream_destroy(ssr_stream_t s) {
    if (!s) return 0;
    return check_hip(hipStreamDestroy(as_stream(s)), "ssr_stream_destroy");
}

ssr_event_t ssr_event_create(void) {
    hipEvent_t e = nullptr;
    if (check_hip(hipEventCreate(&e), "ssr_event_create")) return nullptr;
    return reinterpret_cast<ssr_event_t>(e);
}
int ssr_event_record(ssr_event_t ev, ssr_stream_t s) {
    SSR_REQUIRE(ev, "ssr_event_record", "null event");
    return check_hip(hipEventRecord(reinterpret_cast<hipEvent_t>(ev), as_stream(s)), "ssr_event_record");
}
int ssr_event_synchronize(ssr_event_t ev) {
    SSR_REQUIRE(ev, "ssr_event_synchronize", "null event");
    return check_hip(hipEventSynchronize(reinterpret_cast<hipEvent_t>(ev)), "ssr_event_synchronize");
}
int ssr_event_elapsed_ms(ssr_event_t a, ssr_event_t b, float* ms) {
    SSR_REQUIRE(a && b && ms, "ssr_event_elapsed_ms", "null argument");
    int e = check_hip(hipEventSynchronize(reinterpret_cast<hipEvent_t>(b)), "ssr_event_elapsed_ms/sync");
    if (e) return e;
    return check_hip(hipEventElapsedTime(ms, reinterpret_cast<hipEvent_t>(a), reinterpret_cast<hipEvent_t>(b)),
                     "ssr_event_elapsed_ms");
}
int ssr_event_destroy(ssr_event_t ev) {
    if (!ev) return 0;
    return check_hip(hipEventDestroy(reinterpret_cast<hipEvent_t>(ev)), "ssr_event_destroy");
}

int ssr_read_i64(const int64_t* device_value, int64_t* host_value, int count, ssr_stream_t stream) {
    SSR_REQUIRE(device_value && host_value, "ssr_read_i64", "null pointer");
    SSR_REQUIRE(count > 0 && count <= 1024, "ssr_read_i64", "count out of range");
    // through a pinned staging buffer of this thread's own (kept until the process ends): a copy into pageable
    // memory goes through the runtime's bounce buffer, which for these few bytes costs 16 us more per call
    static thread_local int64_t* staging = nullptr;
    if (!staging) {
        void* p = nullptr;
        if (hipHostMalloc(&p, 1024 * sizeof(int64_t), hipHostMallocDefault) == hipSuccess) staging = static_cast<int64_t*>(p);
        else (void)hipGetLastError();
    }
    int64_t* dst = staging ? staging : host_value;
    int e = check_hip(hipMemcpyAsync(dst, device_value, sizeof(int64_t) * (size_t)count, hipMemcpyDeviceToHost, as_stream(stream)),
                      "ssr_read_i64");
    if (e) return e;
    e = check_hip(hipStreamSynchronize(as_stream(stream)), "ssr_read_i64/sync");
    if (e) return e;
    if (staging) memcpy(host_value, staging, sizeof(int64_t) * (size_t)count);
    return 0;
}

int ssr_debug_math(int op, int64_t n, const float* a, const float* b, float* out, ssr_stream_t stream) {
    if (n <= 0) return 0;
    SSR_REQUIRE(a && out, "ssr_debug_math", "null pointer");
    hipLaunchKernelGGL(debug_math_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0, as_stream(stream),
                       op, n, a, b ? b : a, out);
    SSR_CHECK_LAUNCH("ssr_debug_math");
    return 0;
}

}  // extern "C"
