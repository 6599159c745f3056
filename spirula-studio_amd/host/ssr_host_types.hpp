// ssr_host_types.hpp -- boundary types of the host layer: the non-owning device views, the
// grow-only device pool and the small enums that the reference's backend seam passes around.
//
// Same shapes and meanings as the reference's (src/core/Tensor.h:63-67 TorchTensorView,
// :140-219 DevicePool, :445-452 DeviceVector, :819-826 DeviceTensor2D/3D, :883 DeviceTensorFloatND;
// src/backend/api/BackendTypes.h:34-49 vector PODs; src/core/PoolSlots.h slot names), so that code
// written against the reference's launch functions reads the same against this backend. Only what
// the projection / tile / raster path needs is present.
#pragma once
#include <cstdint>
#include <mutex>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <variant>
#include <vector>

// ---- vector PODs with the device layout (BackendTypes.h:34-49) ----
struct float2 { float x, y; };
struct float3 { float x, y, z; };
struct alignas(16) float4 { float x, y, z, w; };
static_assert(sizeof(float3) == 12 && sizeof(float4) == 16 && alignof(float4) == 16, "device layout");

// (data_ptr, element_size, shape): host or device memory, decided by the address
typedef std::tuple<uint64_t, uint32_t, std::vector<int64_t>> TorchTensorView;

enum class DistortionType : int { None = 0, D = 1, RGB_D = 2, DN = 3, RGB_DN = 4 };   // src/primitives/Primitive.cuh:24-26
enum class DensifyAccumMode : int { None = 0, Max = 1, Sum = 2, Avg = 3 };        // src/primitives/Primitive.cuh:37-39

namespace backend {
enum class MemcpyKind { HostToDevice, DeviceToHost, DeviceToDevice, Auto };
using Stream = void*;
inline constexpr Stream kDefaultStream = nullptr;
struct Event;
int device_count();
bool device_select(int index);
void* device_malloc(size_t bytes);
void* device_malloc_checked(size_t bytes, const char* what = nullptr);
void device_free(void* ptr);
void* host_malloc_pinned(size_t bytes);
void host_free_pinned(void* ptr);
const char* last_error();
void memcpy_sync(void* dst, const void* src, size_t bytes, MemcpyKind kind);
void memcpy_async(void* dst, const void* src, size_t bytes, MemcpyKind kind, Stream stream = kDefaultStream);
void memset_sync(void* dst, int value, size_t bytes);
void memset_async(void* dst, int value, size_t bytes, Stream stream = kDefaultStream);
bool is_device_pointer(const void* ptr);
void device_synchronize();
void stream_synchronize(Stream stream = kDefaultStream);
Event* event_create(bool enable_timing);
void event_record(Event* event, Stream stream = kDefaultStream);
void event_synchronize(Event* event);
void event_destroy(Event* event);
float event_elapsed_ms(Event* start, Event* end);
}  // namespace backend

// Slots of the process-global pool that the path uses (names as in src/core/PoolSlots.h).
enum class PoolSlot : int {
    WorldMeans, WorldQuats, WorldScales, WorldOpacities, WorldFeaturesDc, WorldFeaturesSh,
    WorldShQuantPacked, WorldShQuantBounds,
    CamViewmats, CamIntrins, CamDistCoeffs,
    EngRadii,
    ProjAabb, ProjDepths, ProjScreenXy, ProjScreenDepth, ProjScreenConic, ProjScreenOpac, ProjScreenRgb,
    IsectTilesPerSplat, IsectCumTiles, IsectIdsA, IsectIdsB, IsectFlatA, IsectFlatB, IsectOffsets,
    IsectScanScratch, IsectSortScratch, SeamSortScratch, SeamScanScratch, IsectCounters, ProjVisibleIds, ProjVisibleIdsB, ProjPackedRows,
    IsectTileActive, EngTileMask, IsectTileOrder, IsectBlockMasks,
    AdamG1Means, AdamG1Quats, AdamG1Scales, AdamG1Opacities, AdamG1FeaturesDc, AdamG1FeaturesSh,
    AdamG2Means, AdamG2Quats, AdamG2Scales, AdamG2Opacities, AdamG2FeaturesDc, AdamG2FeaturesSh, EngDensifyScore, EngZeroAabb, FusedProjBwdRowOf, AdamShStatePacked, AdamShStateBounds, AdamNonShPacked, AdamNonShBounds, EngPoseGrad, ProjCameraIds, ProjGaussianIds, ProjGaussianIdsB, ProjPackedScratch, ProjPackedNnz, ProjPackedWorldRows, FusedMultiCamGrad,
    RendersRgb, RendersDepth, RenderTs, RenderLastIds, RenderDistortionRgb, RenderDistortionDepth, RenderMedian,
    RasterBwdAccumWeight, RasterBwdVRows, EngVDistRgb, EngVDistDepth, EngVMedian, EngAccumMap,
    RasterBwdVScreenXy, RasterBwdVScreenDepth, RasterBwdVScreenConic, RasterBwdVScreenOpac, RasterBwdVScreenRgb,
    EngVRgb, EngVDepth, EngVTs,
    GradMeans, GradQuats, GradScales, GradOpacities, GradFeaturesDc, GradFeaturesSh,
    Count
};

// Grow-only pool: a slot reallocates only when the request exceeds its capacity; the caller never
// frees. Guarded by a mutex because trainer and viewer threads both acquire (Tensor.h:165-167).
class DevicePool {
    struct Slot { void* ptr = nullptr; size_t cap = 0, used = 0; };
    std::vector<Slot> slots_;
    mutable std::mutex mu_;
    uint64_t generation_ = 0;
    DevicePool() : slots_((size_t)PoolSlot::Count) {}
public:
    static DevicePool& global() { static DevicePool p; return p; }
    template <typename T> T* acquire(PoolSlot slot, size_t n) {
        std::lock_guard<std::mutex> lock(mu_);
        Slot& s = slots_[(size_t)slot];
        const size_t bytes = n * sizeof(T);
        if (bytes > s.cap) {
            if (s.ptr) backend::device_free(s.ptr);
            s.ptr = nullptr; s.cap = 0;
            s.ptr = backend::device_malloc_checked(bytes);
            s.cap = bytes;
        }
        s.used = bytes;
        return static_cast<T*>(s.ptr);
    }
    size_t capacity_bytes(PoolSlot slot) const { std::lock_guard<std::mutex> l(mu_); return slots_[(size_t)slot].cap; }
    size_t total_bytes() const { std::lock_guard<std::mutex> l(mu_); size_t t = 0; for (auto& s : slots_) t += s.cap; return t; }
    void free_all() {
        std::lock_guard<std::mutex> lock(mu_);
        for (auto& s : slots_) { if (s.ptr) backend::device_free(s.ptr); s = Slot{}; }
        generation_++;
    }
    // Changes whenever the pool has given its memory back: what a caller remembers about a slot's CONTENTS (a
    // buffer it has zeroed once) holds only within one generation, whatever address the slot has afterwards.
    uint64_t generation() const { std::lock_guard<std::mutex> l(mu_); return generation_; }
};

template <typename T>
class DeviceVector {
protected:
    int64_t numel_ = 0;
    T* data_ = nullptr;
public:
    DeviceVector() = default;
    DeviceVector(T* p, int64_t n) : numel_(n), data_(p) {}
    explicit DeviceVector(const TorchTensorView& v) {
        data_ = (T*)std::get<0>(v);
        std::vector<int64_t> shape = std::get<2>(v);
        if (shape.size() == 1) shape.push_back(1);
        if (shape.size() != 2) throw std::runtime_error("Expected 2D tensor view with channel-last layout");
        if (shape[1] * std::get<1>(v) != sizeof(T)) throw std::runtime_error("Element size mismatch");
        numel_ = shape[0];
    }
    int64_t size() const { return numel_; }
    int64_t numel() const { return numel_; }
    T* data_ptr() const { return data_; }
    void resize(PoolSlot slot, int64_t n) { data_ = DevicePool::global().acquire<T>(slot, (size_t)n); numel_ = n; }
    void zero() const { if (data_ && numel_) backend::memset_async(data_, 0, (size_t)numel_ * sizeof(T)); }
};

template <typename T>
class DeviceTensor2D {
    int64_t s0_ = 0, s1_ = 0;
    T* data_ = nullptr;
public:
    DeviceTensor2D() = default;
    DeviceTensor2D(T* p, int64_t a, int64_t b) : s0_(a), s1_(b), data_(p) {}
    template <int D> int64_t size() const { return D == 0 ? s0_ : s1_; }
    int64_t numel() const { return s0_ * s1_; }
    T* data_ptr() const { return data_; }
    void resize(PoolSlot slot, int64_t a, int64_t b) { data_ = DevicePool::global().acquire<T>(slot, (size_t)(a * b)); s0_ = a; s1_ = b; }
    void zero() const { if (data_ && numel()) backend::memset_async(data_, 0, (size_t)numel() * sizeof(T)); }
};

template <typename T>
class DeviceTensor3D {
    int64_t s_[3] = {0, 0, 0};
    T* data_ = nullptr;
public:
    DeviceTensor3D() = default;
    DeviceTensor3D(T* p, int64_t a, int64_t b, int64_t c) : s_{a, b, c}, data_(p) {}
    template <int D> int64_t size() const { return s_[D]; }
    int64_t numel() const { return s_[0] * s_[1] * s_[2]; }
    T* data_ptr() const { return data_; }
    void resize(PoolSlot slot, int64_t a, int64_t b, int64_t c) {
        data_ = DevicePool::global().acquire<T>(slot, (size_t)(a * b * c)); s_[0] = a; s_[1] = b; s_[2] = c;
    }
    void zero() const { if (data_ && numel()) backend::memset_async(data_, 0, (size_t)numel() * sizeof(T)); }
};

// float tensor of any rank, channel count = product of the trailing dims
class DeviceTensorFloatND {
    std::vector<int64_t> shape_;
    float* data_ = nullptr;
public:
    DeviceTensorFloatND() = default;
    DeviceTensorFloatND(float* p, std::vector<int64_t> shape) : shape_(std::move(shape)), data_(p) {}
    explicit DeviceTensorFloatND(const TorchTensorView& v) : shape_(std::get<2>(v)), data_((float*)std::get<0>(v)) {
        if (std::get<1>(v) != sizeof(float)) throw std::runtime_error("DeviceTensorFloatND expects float32");
    }
    template <typename T> explicit DeviceTensorFloatND(const DeviceVector<T>& v)
        : shape_{v.size(), (int64_t)(sizeof(T) / sizeof(float))}, data_((float*)v.data_ptr()) {}
    template <typename T> explicit DeviceTensorFloatND(const DeviceTensor2D<T>& v)
        : shape_{v.template size<0>(), v.template size<1>(), (int64_t)(sizeof(T) / sizeof(float))}, data_((float*)v.data_ptr()) {}
    float* data_ptr() const { return data_; }
    const std::vector<int64_t>& shape() const { return shape_; }
    int64_t numel() const { int64_t n = shape_.empty() ? 0 : 1; for (auto s : shape_) n *= s; return n; }
    int64_t rows() const { return shape_.empty() ? 0 : shape_[0]; }
    int64_t channels() const { return rows() ? numel() / rows() : 0; }
};

// src/core/NonShQuantState.h:16-28: the 16-bit quantized Adam moments of the five non-SH tensors, one float4 of
// bounds per 256 splats and tensor (bounds held as plain floats here)
struct NonShQuantState {
    bool enabled = false;
    uint8_t* means_packed = nullptr;
    uint8_t* quats_packed = nullptr;
    uint8_t* scales_packed = nullptr;
    uint8_t* opacities_packed = nullptr;
    uint8_t* features_dc_packed = nullptr;
    float* means_bounds = nullptr;
    float* quats_bounds = nullptr;
    float* scales_bounds = nullptr;
    float* opacities_bounds = nullptr;
    float* features_dc_bounds = nullptr;
};

struct RenderOutput {
    // (rgb [I,H,W] float3, depth [I,H,W] float, normal -- unused by the 3dgs primitive)
    typedef std::tuple<DeviceTensor3D<float3>, DeviceTensor3D<float>, DeviceTensor3D<float3>> TensorTuple;
};
