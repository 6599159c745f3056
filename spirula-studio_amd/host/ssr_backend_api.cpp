// ssr_backend_api.cpp -- the reference-shaped launch functions and runtime, implemented on the C
// ABI of libssr_hip.so. This file contains no device code and needs no HIP headers.
#include "ssr_backend_api.hpp"

#include <cstring>

#include "../../include/ssr_backend.h"

// set for the duration of a projection_mip_* / fused_projection_bwd_optimizer_mip call (ssr_detail::AntialiasedScope)
static thread_local bool g_antialiased = false;
ssr_detail::AntialiasedScope::AntialiasedScope() { g_antialiased = true; }
ssr_detail::AntialiasedScope::~AntialiasedScope() { g_antialiased = false; }

namespace {

[[noreturn]] void throw_last(const char* where) {
    const char* e = ssr_last_error();
    throw std::runtime_error(std::string(where) + ": " + ((e && e[0]) ? e : "unknown backend error"));
}
inline void ok(int rc, const char* where) { if (rc != 0) throw_last(where); }

thread_local std::string g_sticky;   // backend::last_error(): returned once, then cleared

ssr_ext::Options g_opts;
bool g_profile = false;
ssr_ext::StageTimes g_times;
int64_t g_n_isects = 0;
int64_t g_n_visible = -1;
int64_t g_seen_visible = -1;         // the last visible count the host learned, kept over the projections that follow it
                                     // (g_n_visible starts unknown again with every projection)
bool g_counts_fused = false;         // the last projection already produced tile counts
int64_t* g_counters = nullptr;       // device [n_isects, n_visible], one readback for both: one of the two pairs of the slot
int64_t* g_counters_base = nullptr;  // the slot's two pairs; a projection with a visible list takes them in turn
int g_counters_turn = 0;
bool g_counters_clean[2] = {false, false};   // the pair's visible counter is known to be zero
int32_t* g_visible_ids = nullptr;    // device work list of the last projection (null: off)
float* g_packed_rows = nullptr;      // packed screen rows of the last projection (null: off)
const float* g_packed_for_xy = nullptr;   // the screen.xy buffer those rows mirror
float* g_world_rows = nullptr;                 // parameter rows of the last packed projection (null: off)
const int32_t* g_world_rows_for_ids = nullptr; // the gaussian_ids they follow
const float* g_world_rows_for_means = nullptr; // the means tensor they were read from
int64_t g_world_rows_count = 0;
bool g_packed_mode = false;          // the last projection was the packed form
std::vector<int64_t> g_packed_counts;   // ... and its rows per camera (rows are ordered by camera, then splat)
int g_list_toggle = 0;               // which of the two visible-list buffers the last projection used
float* g_vrows = nullptr;             // packed gradient rows of the last compositing backward (null: off)
const int32_t* g_tile_order = nullptr;       // launch order of the compositing workgroups for the offsets below (null: off)
const int32_t* g_tile_order_for = nullptr;   // the tile_offsets that order was made from
const uint16_t* g_block_masks = nullptr;     // block masks the last compositing forward left (null: none)
const int32_t* g_block_masks_for = nullptr;  // the flatten_ids they belong to
const float* g_vrows_for_xy = nullptr; // the v_screen.xy buffer they stand in for
const int32_t* g_bwd_list = nullptr; // list of the last projection backward
int64_t g_bwd_count = 0;
// Counts left on the device (Options::deferred_counts): the key arrays of the next intersection are sized from
// g_deferred_capacity (0: unknown, that call reads the count as the reference does), the counters travel to pinned
// memory behind the scan, and resolve_counts() waits for them when somebody needs the numbers.
int64_t g_deferred_capacity = 0;
int64_t g_deferred_used = 0;          // capacity of the arrays the pending counts belong to
bool g_counts_pending = false;
int64_t g_short_frames = 0;           // intersections that did not fit their arrays, counted as they are found out
int64_t* g_counts_host = nullptr;     // pinned [2]
ssr_event_t g_counts_event = nullptr;
const int32_t* g_offsets_closed = nullptr;   // tile_offsets with one more entry, the end of the last tile (null: none)

int64_t capacity_for(int64_t n_isects) { return n_isects + n_isects / 16 + 65536; }

struct StageTimer {
    ssr_event_t a = nullptr, b = nullptr;
    float* out;
    explicit StageTimer(float* o) : out(o) {
        if (!g_profile) return;
        a = ssr_event_create(); b = ssr_event_create();
        ssr_event_record(a, nullptr);
    }
    ~StageTimer() {
        if (!g_profile) return;
        ssr_event_record(b, nullptr);
        float ms = 0;
        ssr_event_elapsed_ms(a, b, &ms);
        *out = ms;
        ssr_event_destroy(a); ssr_event_destroy(b);
    }
};

// camera_model_from_name / camera_distortion_from_name (src/core/CameraModel.h:64-71,165-183), with the
// lower-case spellings this harness has always accepted
int camera_model_of(const std::string& m) {
    if (m == "PINHOLE" || m == "pinhole" || m == "SIMPLE_PINHOLE" || m == "SIMPLE_RADIAL" || m == "RADIAL" || m == "OPENCV")
        return SSR_CAM_PINHOLE;
    if (m == "FISHEYE" || m == "fisheye" || m == "SIMPLE_FISHEYE" || m == "SIMPLE_RADIAL_FISHEYE" || m == "RADIAL_FISHEYE" ||
        m == "OPENCV_FISHEYE" || m == "THIN_PRISM_FISHEYE")
        return SSR_CAM_FISHEYE;
    if (m == "EQUISOLID" || m == "equisolid") return SSR_CAM_EQUISOLID;
    if (m == "EQUIRECTANGULAR" || m == "equirectangular" || m == "EQUIRECT") return SSR_CAM_EQUIRECT;
    throw std::runtime_error("projection: unknown camera model '" + m + "'");
}
int lens_tier_of(const std::string& d) {
    if (d == "NONE" || d == "none" || d.empty()) return SSR_LENS_NONE;
    if (d == "OPENCV" || d == "opencv") return SSR_LENS_OPENCV;
    if (d == "THIN_PRISM" || d == "thin_prism") return SSR_LENS_THIN_PRISM;
    if (d == "RATIONAL" || d == "rational") return SSR_LENS_RATIONAL;
    throw std::runtime_error("projection: unknown distortion tier '" + d + "'");
}

ssr_world world_of(const std::vector<DeviceTensorFloatND>& s) {
    if (s.size() != 6) throw std::runtime_error("expected 6 world tensors (means, quats, scales, opacities, dc, sh)");
    ssr_world w;
    w.means = s[0].data_ptr(); w.quats = s[1].data_ptr(); w.log_scales = s[2].data_ptr();
    w.opacity_logits = s[3].data_ptr(); w.features_dc = s[4].data_ptr(); w.features_sh = s[5].data_ptr();
    w.sh_stride = (int32_t)s[5].channels();
    return w;
}
ssr_screen screen_of(const std::vector<DeviceTensorFloatND>& s) {
    if (s.size() != 5) throw std::runtime_error("expected 5 screen tensors (xy, depth, conic, opac, rgb)");
    ssr_screen r;
    r.xy = s[0].data_ptr(); r.depth = s[1].data_ptr(); r.conic = s[2].data_ptr(); r.opac = s[3].data_ptr();
    r.rgb = s[4].data_ptr();
    return r;
}
ssr_sh_quant sh_of(const std::optional<TorchTensorView>& packed, const std::optional<TorchTensorView>& bounds,
                   uint32_t num_sh_buffer, int bits, int64_t stride) {
    ssr_sh_quant q;
    std::memset(&q, 0, sizeof(q));
    q.codec = SSR_SH_F32;
    q.num_sh_buffer = num_sh_buffer;
    q.bounds_stride = stride;
    if (bits == 32) return q;
    if (bits != 8 && bits != 16) throw std::runtime_error("projection: sh_value_bits must be 32, 16 or 8");
    if (!packed || !bounds) throw std::runtime_error("projection: quantized SH needs packed codes and bounds");
    q.packed = (const void*)std::get<0>(*packed);
    if (g_opts.sh_int8_f16scale && bits == 8) {
        q.codec = SSR_SH_I8_F16SCALE;
        q.scale_f16 = (const uint16_t*)std::get<0>(*bounds);
    } else {
        q.codec = bits == 8 ? SSR_SH_REF_Q8 : SSR_SH_REF_Q16;
        q.bounds = (const float*)std::get<0>(*bounds);
    }
    return q;
}
ssr_camera camera_of(const std::string& model, const std::string& distortion, const TorchTensorView& dist_coeffs,
                     const TorchTensorView& viewmats, const TorchTensorView& intrins, uint32_t w, uint32_t h,
                     bool several_ok = false) {
    ssr_camera c;
    c.camera_model = camera_model_of(model);
    c.distortion = lens_tier_of(distortion);
    // camera_distortion_is_compiled, src/core/CameraModel.h:154-162
    const bool wide = c.camera_model == SSR_CAM_FISHEYE || c.camera_model == SSR_CAM_EQUISOLID;
    if ((wide && c.distortion == SSR_LENS_RATIONAL) || (c.camera_model == SSR_CAM_EQUIRECT && c.distortion != SSR_LENS_NONE))
        throw std::runtime_error("projection: camera model '" + model + "' has no '" + distortion + "' distortion tier");
    c.dist_coeffs = (const float*)std::get<0>(dist_coeffs);
    if (c.distortion != SSR_LENS_NONE) {
        const auto& ds = std::get<2>(dist_coeffs);
        if (!c.dist_coeffs || ds.size() != 2 || ds[1] != 8)
            throw std::runtime_error("projection: distortion needs a [num_cameras, 8] coefficient tensor");
    }
    const auto& shape = std::get<2>(viewmats);
    c.num_cameras = shape.empty() ? 0u : (uint32_t)shape[0];
    if (c.num_cameras < 1 || (c.num_cameras != 1 && !several_ok))
        throw std::runtime_error("this entry point runs one camera per call (got " + std::to_string(c.num_cameras) + ")");
    c.width = w; c.height = h;
    c.viewmats = (const float*)std::get<0>(viewmats);
    c.intrins = (const float*)std::get<0>(intrins);
    return c;
}
// Camera i of a [C, ...] set, as a one-camera set: the kernels take one camera per launch
ssr_camera camera_at(const ssr_camera& all, uint32_t i) {
    ssr_camera c = all;
    c.num_cameras = 1;
    c.viewmats = all.viewmats + 16 * (size_t)i;
    c.intrins = all.intrins + 4 * (size_t)i;
    if (all.dist_coeffs) c.dist_coeffs = all.dist_coeffs + 8 * (size_t)i;
    return c;
}
ssr_screen screen_rows_from(const ssr_screen& s, int64_t row) {
    ssr_screen o = s;
    if (s.xy) o.xy = s.xy + 2 * row;
    if (s.depth) o.depth = s.depth + row;
    if (s.conic) o.conic = s.conic + 3 * row;
    if (s.opac) o.opac = s.opac + row;
    if (s.rgb) o.rgb = s.rgb + 3 * row;
    return o;
}

}  // namespace

// ---------------------------------------------------------------------------------------------
namespace backend {

struct Event { ssr_event_t ev; };

int device_count() { return ssr_device_count(); }
bool device_select(int index) {
    if (ssr_init(index) != 0) { g_sticky = ssr_last_error(); return false; }
    return true;
}
void* device_malloc(size_t bytes) {
    void* p = ssr_device_malloc(bytes);
    if (!p && bytes) g_sticky = ssr_last_error();
    return p;
}
void* device_malloc_checked(size_t bytes, const char* what) {
    void* p = device_malloc(bytes);
    if (!p && bytes > 0) {
        char buf[64];
        std::snprintf(buf, sizeof buf, "%.0f MiB", (double)bytes / (1024.0 * 1024.0));
        std::string msg = std::string("GPU allocation failed: ") + last_error() + "; could not allocate " + buf;
        if (what && what[0]) { msg += " for "; msg += what; }
        msg += ". Try a smaller model (fewer splats / SH) or a lower image resolution.";
        throw std::runtime_error(msg);
    }
    return p;
}
void device_free(void* ptr) { if (ssr_device_free(ptr) != 0) g_sticky = ssr_last_error(); }
void* host_malloc_pinned(size_t bytes) {
    void* p = ssr_host_malloc_pinned(bytes);
    if (!p && bytes) g_sticky = ssr_last_error();
    return p;
}
void host_free_pinned(void* ptr) { if (ssr_host_free_pinned(ptr) != 0) g_sticky = ssr_last_error(); }
const char* last_error() {
    static thread_local std::string out;
    out.swap(g_sticky);
    g_sticky.clear();
    return out.c_str();
}
static int kind_of(MemcpyKind k) {
    switch (k) {
        case MemcpyKind::HostToDevice: return SSR_MEMCPY_H2D;
        case MemcpyKind::DeviceToHost: return SSR_MEMCPY_D2H;
        case MemcpyKind::DeviceToDevice: return SSR_MEMCPY_D2D;
        default: return SSR_MEMCPY_AUTO;
    }
}
void memcpy_sync(void* d, const void* s, size_t n, MemcpyKind k) { if (ssr_memcpy(d, s, n, kind_of(k), nullptr, 0)) g_sticky = ssr_last_error(); }
void memcpy_async(void* d, const void* s, size_t n, MemcpyKind k, Stream st) { if (ssr_memcpy(d, s, n, kind_of(k), st, 1)) g_sticky = ssr_last_error(); }
void memset_sync(void* d, int v, size_t n) { if (ssr_memset(d, v, n, nullptr, 0)) g_sticky = ssr_last_error(); }
void memset_async(void* d, int v, size_t n, Stream st) { if (ssr_memset(d, v, n, st, 1)) g_sticky = ssr_last_error(); }
bool is_device_pointer(const void* p) { return ssr_is_device_pointer(p) != 0; }
void device_synchronize() { if (ssr_device_synchronize()) g_sticky = ssr_last_error(); }
void stream_synchronize(Stream st) { if (ssr_stream_synchronize(st)) g_sticky = ssr_last_error(); }
Event* event_create(bool) { Event* e = new Event{ssr_event_create()}; return e; }
void event_record(Event* e, Stream st) { if (e && ssr_event_record(e->ev, st)) g_sticky = ssr_last_error(); }
void event_synchronize(Event* e) { if (e && ssr_event_synchronize(e->ev)) g_sticky = ssr_last_error(); }
void event_destroy(Event* e) { if (e) { ssr_event_destroy(e->ev); delete e; } }
float event_elapsed_ms(Event* a, Event* b) {
    float ms = 0;
    if (!a || !b || ssr_event_elapsed_ms(a->ev, b->ev, &ms)) g_sticky = ssr_last_error();
    return ms;
}


// ---- src/backend/common/SortScan.h:53-60, the two instantiations of the tile-intersection stage ----
template <>
void sort_pairs<int64_t, int32_t>(DoubleBuffer<int64_t>& keys, DoubleBuffer<int32_t>& values, int64_t num_items,
                                  int begin_bit, int end_bit, Stream stream) {
    if (num_items < 0) throw std::runtime_error("sort_pairs: negative num_items");
    if (num_items == 0 || end_bit <= begin_bit) return;   // nothing to order: the current buffers already hold the result
    const size_t bytes = ssr_sort_scratch_bytes(num_items);
    void* work = DevicePool::global().acquire<uint8_t>(PoolSlot::SeamSortScratch, bytes > 16 ? bytes : 16);
    int moved = 0;   // 0: the result is where the input was, 1: in the alternate pair
    if (ssr_sort_pairs_u64_i32(keys.current(), keys.alternate(), values.current(), values.alternate(), num_items, begin_bit,
                               end_bit, &moved, work, bytes, stream) != 0)
        throw std::runtime_error(std::string("sort_pairs: ") + ssr_last_error());
    keys.selector ^= moved;
    values.selector ^= moved;
}

template <>
void inclusive_sum<int64_t>(const int64_t* in, int64_t* out, int64_t num_items, Stream stream) {
    if (num_items < 0) throw std::runtime_error("inclusive_sum: negative num_items");
    if (num_items == 0) return;
    const size_t bytes = ssr_scan_scratch_bytes(num_items);
    void* work = DevicePool::global().acquire<uint8_t>(PoolSlot::SeamScanScratch, bytes > 16 ? bytes : 16);
    if (ssr_inclusive_sum_i64(in, out, num_items, nullptr, work, bytes, stream) != 0)
        throw std::runtime_error(std::string("inclusive_sum: ") + ssr_last_error());
}

}  // namespace backend

namespace ssr_ext {
Options& options() { return g_opts; }
void set_stage_profiling(bool on) { g_profile = on; }
StageTimes last_stage_times() { return g_times; }
void resolve_counts() {
    if (!g_counts_pending) return;
    g_counts_pending = false;
    ok(ssr_event_synchronize(g_counts_event), "resolve_counts");
    g_n_isects = g_counts_host[0];
    if (g_visible_ids) g_seen_visible = g_n_visible = g_counts_host[1];
    const int64_t used = g_deferred_used;
    if (g_n_isects > used) {
        g_deferred_capacity = 0;   // the next intersection reads its count and sizes from it
        // Counted and left in the sticky error as well: a caller that only renders never asks for the counts, and the
        // stages that settle them on its behalf must not lose the fact that a frame was short.
        g_short_frames++;
        g_sticky = "an intersection of " + std::to_string(g_n_isects) + " entries did not fit the " + std::to_string(used) +
                   " its arrays were sized for (deferred counts): that frame misses fragments";
        throw std::runtime_error("resolve_counts: " + std::to_string(g_n_isects) + " intersections did not fit the " +
                                 std::to_string(used) + " the arrays were sized for; the images and gradients of this "
                                 "iteration miss fragments: repeat it");
    }
    g_deferred_capacity = capacity_for(g_n_isects);
}
void set_deferred_capacity(int64_t capacity) { g_deferred_capacity = capacity < 0 ? 0 : capacity; }
int64_t deferred_capacity() { return g_deferred_capacity; }
int64_t short_frames() { return g_short_frames; }
int64_t last_n_isects() { resolve_counts(); return g_n_isects; }
int64_t last_n_visible() { resolve_counts(); return g_n_visible; }
bool backward_overwrites_all_rows(int64_t num_splats) {
    resolve_counts();
    if (!g_opts.overwrite_world_grads) return false;
    if (g_packed_mode) return false;                       // packed rows: only listed splats are written
    if (!g_visible_ids || g_n_visible < 0) return true;    // no list: every row is visited
    return g_n_visible * 2 >= num_splats;
}
const int32_t* last_backward_list(int64_t* count) { if (count) *count = g_bwd_count; return g_bwd_list; }
bool projection_stores_radii(int64_t cameras) { return cameras == 1; }
void forget_packed_world_rows() { g_world_rows = nullptr; g_world_rows_for_ids = nullptr; g_world_rows_for_means = nullptr; g_world_rows_count = 0; }
void zero_world_rows(const std::vector<DeviceTensorFloatND>& v, const int32_t* ids, int64_t n,
                     const DeviceTensor2D<float4>* aabb, const int32_t* sorted_now, int64_t n_now) {
    ssr_world w = world_of(v);
    ok(ssr_zero_world_rows(&w, ids, n, aabb ? (const float*)aabb->data_ptr() : nullptr, sorted_now, sorted_now ? n_now : 0, nullptr),
       "zero_world_rows");
}
}  // namespace ssr_ext

// The counters [n_isects, n_visible] live in one slot of two pairs, zeroed when the slot is first handed out.
// next_turn: the caller is a projection that counts visible splats into the pair and has the other pair's counter
// cleared by its kernel; otherwise the current pair is returned (only its n_isects is used).
static int64_t* counters_pair(bool next_turn) {
    int64_t* base = DevicePool::global().acquire<int64_t>(PoolSlot::IsectCounters, 4);
    static uint64_t generation = ~(uint64_t)0;
    if (base != g_counters_base || generation != DevicePool::global().generation()) {
        generation = DevicePool::global().generation();
        g_counters_base = base;
        g_counters_turn = 0;
        backend::memset_async(base, 0, 4 * sizeof(int64_t));
        g_counters_clean[0] = g_counters_clean[1] = true;
    }
    if (next_turn) {
        g_counters_turn ^= 1;
        // a projection that failed before its launch, or had no splats, has not cleared this pair
        if (!g_counters_clean[g_counters_turn]) backend::memset_async(base + 2 * g_counters_turn, 0, 2 * sizeof(int64_t));
        g_counters_clean[g_counters_turn] = false;   // about to count
    }
    return base + 2 * g_counters_turn;
}

// ---------------------------------------------------------------------------------------------
std::tuple<DeviceTensor2D<float4>, DeviceTensor2D<float>, std::vector<DeviceTensorFloatND>>
projection_3dgs_forward(const int64_t num_splats, const int max_sh_degree,
                        const std::vector<DeviceTensorFloatND>& in_splats, TorchTensorView viewmats,
                        TorchTensorView intrins, const uint32_t image_width, const uint32_t image_height,
                        const std::string camera_model, const std::string distortion, const TorchTensorView dist_coeffs,
                        DeviceVector<float> radii, const std::optional<TorchTensorView> sh_value_packed,
                        const std::optional<TorchTensorView> sh_value_bounds, const uint32_t num_sh_buffer,
                        const int sh_value_bits, const int64_t sh_bounds_stride) {
    try { ssr_ext::resolve_counts(); } catch (const std::runtime_error&) {}   // an unfinished iteration's counts; a short one stays in short_frames() / last_error()
    ssr_projection_fwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.num_splats = num_splats;
    p.sh_degree = max_sh_degree;
    p.antialiased = g_antialiased ? 1 : 0;
    p.world = world_of(in_splats);
    p.sh = sh_of(sh_value_packed, sh_value_bounds, num_sh_buffer, sh_value_bits, sh_bounds_stride);
    // Several cameras ([C,4,4] viewmats): one projection launch per camera into row block c of the
    // [C,N,...] outputs (the reference's single launch covers C*N rows, ProjectionFwd_kernel.cuh:60-110).
    const ssr_camera cameras = camera_of(camera_model, distortion, dist_coeffs, viewmats, intrins, image_width, image_height, true);
    const int64_t C = cameras.num_cameras, N = num_splats;

    DeviceTensor2D<float4> aabb; aabb.resize(PoolSlot::ProjAabb, C, N);
    DeviceTensor2D<float> depths; depths.resize(PoolSlot::ProjDepths, C, N);
    float* xy = DevicePool::global().acquire<float>(PoolSlot::ProjScreenXy, (size_t)(C * N * 2));
    float* dp = DevicePool::global().acquire<float>(PoolSlot::ProjScreenDepth, (size_t)(C * N));
    float* cn = DevicePool::global().acquire<float>(PoolSlot::ProjScreenConic, (size_t)(C * N * 3));
    float* op = DevicePool::global().acquire<float>(PoolSlot::ProjScreenOpac, (size_t)(C * N));
    float* rg = DevicePool::global().acquire<float>(PoolSlot::ProjScreenRgb, (size_t)(C * N * 3));
    p.aabb = (float*)aabb.data_ptr(); p.sort_depth = depths.data_ptr(); p.radii = radii.data_ptr();
    p.screen.xy = xy; p.screen.depth = dp; p.screen.conic = cn; p.screen.opac = op; p.screen.rgb = rg;
    g_counts_fused = false;
    g_packed_mode = false;
    g_world_rows = nullptr; g_world_rows_for_ids = nullptr; g_world_rows_for_means = nullptr; g_world_rows_count = 0;
    if (g_opts.fuse_tile_count) {
        p.tiles_per_splat = DevicePool::global().acquire<int64_t>(PoolSlot::IsectTilesPerSplat, (size_t)(C * N));
        g_counts_fused = true;
    }
    g_counters = counters_pair(false);
    g_visible_ids = nullptr;
    g_n_visible = -1;
    p.radii_store = C == 1 ? 1 : 0;   // the one writer of radii: same values as the caller's zero-fill and the maximum
    if (g_opts.visible_list && C == 1) {   // one list and one counter: a single camera's
        g_list_toggle ^= 1;
        g_visible_ids = DevicePool::global().acquire<int32_t>(
            g_list_toggle ? PoolSlot::ProjVisibleIdsB : PoolSlot::ProjVisibleIds, (size_t)(C * N));
        // the visible counter starts at zero: this projection clears the other pair's for the next one, as the
        // one before did for this one (the pairs start out zeroed), so no fill is launched per projection
        g_counters = counters_pair(true);
        p.visible_ids = g_visible_ids;
        p.visible_count = g_counters + 1;
        p.clear_count = g_counters_base + 2 * (g_counters_turn ^ 1) + 1;
    }
    g_packed_rows = nullptr;
    g_packed_for_xy = nullptr;
    if (g_opts.packed_rows) {
        g_packed_rows = DevicePool::global().acquire<float>(PoolSlot::ProjPackedRows, (size_t)(C * N * 12));
        g_packed_for_xy = xy;
        p.packed_rows = g_packed_rows;
    }
    {
        StageTimer t(&g_times.k1);
        const ssr_projection_fwd_params all = p;
        for (int64_t c = 0; c < C; c++) {
            p.camera = camera_at(cameras, (uint32_t)c);
            p.aabb = all.aabb + 4 * c * N; p.sort_depth = all.sort_depth + c * N;
            p.screen = screen_rows_from(all.screen, c * N);
            if (all.tiles_per_splat) p.tiles_per_splat = all.tiles_per_splat + c * N;
            if (all.packed_rows) p.packed_rows = all.packed_rows + 12 * c * N;
            ok(ssr_projection_fwd(&p, nullptr), "projection_3dgs_forward");
        }
        if (p.clear_count && N > 0) g_counters_clean[g_counters_turn ^ 1] = true;   // the launch went out
    }
    std::vector<DeviceTensorFloatND> screen = {
        DeviceTensorFloatND(xy, {C * N, 2}), DeviceTensorFloatND(dp, {C * N, 1}), DeviceTensorFloatND(cn, {C * N, 3}),
        DeviceTensorFloatND(op, {C * N, 1}), DeviceTensorFloatND(rg, {C * N, 3})};
    return std::make_tuple(aabb, depths, screen);
}

std::tuple<DeviceVector<int32_t>, DeviceVector<int32_t>, DeviceVector<float4>, DeviceVector<float>,
           std::vector<DeviceTensorFloatND>>
projection_3dgs_packed_forward(const int64_t num_splats, const int max_sh_degree,
                               const std::vector<DeviceTensorFloatND>& in_splats, TorchTensorView viewmats,
                               TorchTensorView intrins, const uint32_t image_width, const uint32_t image_height,
                               const std::string camera_model, const std::string distortion, const TorchTensorView dist_coeffs,
                               DeviceVector<float> radii, const std::optional<TorchTensorView> sh_value_packed,
                               const std::optional<TorchTensorView> sh_value_bounds, const uint32_t num_sh_buffer,
                               const int sh_value_bits, const int64_t sh_bounds_stride) {
    try { ssr_ext::resolve_counts(); } catch (const std::runtime_error&) {}   // an unfinished iteration's counts; a short one stays in short_frames() / last_error()
    ssr_projection_packed_params p;
    std::memset(&p, 0, sizeof(p));
    p.num_splats = num_splats;
    p.sh_degree = max_sh_degree;
    p.antialiased = g_antialiased ? 1 : 0;
    p.world = world_of(in_splats);
    p.sh = sh_of(sh_value_packed, sh_value_bounds, num_sh_buffer, sh_value_bits, sh_bounds_stride);
    // Several cameras: one mask / emit pair per camera, each camera's rows behind the previous camera's, which is
    // the (camera, splat) order the reference's single scan over C * N leaves (ProjectionPackedFwd.cu:64-158). Every
    // camera stages into its own part of the scratch slot, so that all masks run before the one readback of the
    // C row counts.
    const ssr_camera cameras = camera_of(camera_model, distortion, dist_coeffs, viewmats, intrins, image_width, image_height, true);
    const int64_t C = cameras.num_cameras;
    p.radii = radii.data_ptr();
    p.stage_world_rows = g_opts.packed_world_rows ? 1 : 0;
    p.scratch_bytes = p.stage_world_rows ? ssr_projection_packed_scratch_bytes_world_rows(num_splats)
                                         : ssr_projection_packed_scratch_bytes(num_splats);
    g_world_rows = nullptr; g_world_rows_for_ids = nullptr; g_world_rows_for_means = nullptr; g_world_rows_count = 0;
    const size_t scratch_stride = (p.scratch_bytes + 255) & ~(size_t)255;
    uint8_t* scratch = DevicePool::global().acquire<uint8_t>(PoolSlot::ProjPackedScratch, scratch_stride * (size_t)C);
    int64_t* nnz_dev = DevicePool::global().acquire<int64_t>(PoolSlot::ProjPackedNnz, (size_t)C);
    // the work list and its counters belong to the non-packed form
    g_packed_mode = true;
    g_visible_ids = nullptr; g_n_visible = -1; g_counters = nullptr;
    g_counts_fused = false; g_packed_rows = nullptr; g_packed_for_xy = nullptr;
    StageTimer t(&g_times.k1);
    for (int64_t c = 0; c < C; c++) {
        p.camera = camera_at(cameras, (uint32_t)c);
        p.scratch = scratch + scratch_stride * (size_t)c;
        p.nnz = nnz_dev + c;
        ok(ssr_projection_packed_mask(&p, nullptr), "projection_3dgs_packed_forward/mask");
    }
    std::vector<int64_t> counts((size_t)C, 0);
    if (num_splats > 0) ok(ssr_read_i64(nnz_dev, counts.data(), (int)C, nullptr), "projection_3dgs_packed_forward/readback");
    int64_t nnz = 0;
    for (int64_t v : counts) nnz += v;
    g_packed_counts = counts;
    g_n_visible = nnz;
    DeviceVector<int32_t> camera_ids, gaussian_ids;
    DeviceVector<float4> aabb;
    DeviceVector<float> depths;
    if (nnz == 0) {   // nothing visible: empty (null) views, which every later stage treats as "no work"
        std::vector<DeviceTensorFloatND> none = {
            DeviceTensorFloatND(nullptr, {0, 2}), DeviceTensorFloatND(nullptr, {0, 1}), DeviceTensorFloatND(nullptr, {0, 3}),
            DeviceTensorFloatND(nullptr, {0, 1}), DeviceTensorFloatND(nullptr, {0, 3})};
        return std::make_tuple(camera_ids, gaussian_ids, aabb, depths, none);
    }
    camera_ids.resize(PoolSlot::ProjCameraIds, nnz);
    // two id buffers alternate, so that the list a backward ran over outlives the next projection
    g_list_toggle ^= 1;
    gaussian_ids.resize(g_list_toggle ? PoolSlot::ProjGaussianIdsB : PoolSlot::ProjGaussianIds, nnz);
    aabb.resize(PoolSlot::ProjAabb, nnz);
    depths.resize(PoolSlot::ProjDepths, nnz);
    float* xy = DevicePool::global().acquire<float>(PoolSlot::ProjScreenXy, (size_t)(nnz * 2));
    float* dp = DevicePool::global().acquire<float>(PoolSlot::ProjScreenDepth, (size_t)nnz);
    float* cn = DevicePool::global().acquire<float>(PoolSlot::ProjScreenConic, (size_t)(nnz * 3));
    float* op = DevicePool::global().acquire<float>(PoolSlot::ProjScreenOpac, (size_t)nnz);
    float* rg = DevicePool::global().acquire<float>(PoolSlot::ProjScreenRgb, (size_t)(nnz * 3));
    std::vector<DeviceTensorFloatND> screen = {
        DeviceTensorFloatND(xy, {nnz, 2}), DeviceTensorFloatND(dp, {nnz, 1}), DeviceTensorFloatND(cn, {nnz, 3}),
        DeviceTensorFloatND(op, {nnz, 1}), DeviceTensorFloatND(rg, {nnz, 3})};
    int64_t* tiles = nullptr;
    if (g_opts.fuse_tile_count) {
        tiles = DevicePool::global().acquire<int64_t>(PoolSlot::IsectTilesPerSplat, (size_t)nnz);
        g_counts_fused = true;
    }
    if (g_opts.packed_rows) {
        g_packed_rows = DevicePool::global().acquire<float>(PoolSlot::ProjPackedRows, (size_t)(nnz * 12));
        g_packed_for_xy = xy;
    }
    if (p.stage_world_rows) {
        g_world_rows = DevicePool::global().acquire<float>(PoolSlot::ProjPackedWorldRows, (size_t)(nnz * 16));
        g_world_rows_for_ids = gaussian_ids.data_ptr();
        g_world_rows_for_means = p.world.means;
        g_world_rows_count = nnz;
    }
    int64_t row0 = 0;
    for (int64_t c = 0; c < C; c++) {
        const int64_t rows = counts[(size_t)c];
        if (rows > 0) {
            p.camera = camera_at(cameras, (uint32_t)c);
            p.camera_index = (int32_t)c;
            p.world_rows = g_world_rows ? g_world_rows + 4 * row0 : nullptr;   // four planes of nnz entries
            p.world_rows_stride = nnz;
            p.scratch = scratch + scratch_stride * (size_t)c;
            p.nnz = nnz_dev + c;
            p.max_rows = rows;
            p.camera_ids = camera_ids.data_ptr() + row0; p.gaussian_ids = gaussian_ids.data_ptr() + row0;
            p.aabb = (float*)aabb.data_ptr() + 4 * row0; p.sort_depth = depths.data_ptr() + row0;
            p.screen.xy = xy + 2 * row0; p.screen.depth = dp + row0; p.screen.conic = cn + 3 * row0;
            p.screen.opac = op + row0; p.screen.rgb = rg + 3 * row0;
            p.tiles_per_splat = tiles ? tiles + row0 : nullptr;
            p.packed_rows = g_packed_rows ? g_packed_rows + 12 * row0 : nullptr;
            ok(ssr_projection_packed_emit(&p, nullptr), "projection_3dgs_packed_forward/emit");
        }
        row0 += rows;
    }
    return std::make_tuple(camera_ids, gaussian_ids, aabb, depths, screen);
}

int64_t intersect_tile_count(int width, int height) {
    return (int64_t)((width + 15) / 16) * (int64_t)((height + 15) / 16);
}

void compute_tile_active(TorchTensorView mask, int I, int width, int height, int32_t* tile_active) {
    if (I < 1) throw std::runtime_error("compute_tile_active: no image");
    const auto& ms = std::get<2>(mask);
    if (ms.size() != 3 || ms[0] != I) throw std::runtime_error("compute_tile_active: mask must be [I, H_mask, W_mask]");
    const int64_t tiles = intersect_tile_count(width, height);
    for (int i = 0; i < I; i++)   // one [tile_h, tile_w] block per image (IntersectTile.cuh:18-22)
        ok(ssr_compute_tile_active((const uint8_t*)std::get<0>(mask) + (size_t)i * (size_t)(ms[1] * ms[2]), (int32_t)ms[1],
                                   (int32_t)ms[2], (uint32_t)width, (uint32_t)height, tile_active + (size_t)i * (size_t)tiles, nullptr),
           "compute_tile_active");
}

namespace {
// K4-K6 in arrays of g_deferred_used entries, the counts staying on the device: the key write stops at the capacity,
// the sort reads the count where it lies, and the offsets carry one more entry, the end of the last tile, which
// the compositing launches read instead of a host count.
std::tuple<DeviceVector<int64_t>, DeviceVector<int32_t>, DeviceTensor3D<int32_t>>
intersect_tile_deferred(DeviceTensorFloatND& aabb, DeviceTensorFloatND& depths, DeviceTensorFloatND& proj_xy,
                        DeviceTensorFloatND& proj_conic, DeviceTensorFloatND& proj_opac, uint32_t I, uint32_t image_width,
                        uint32_t image_height, const int32_t* img_ids, const int32_t* tile_active, DeviceVector<int64_t>& cum,
                        int64_t total) {
    const uint32_t tile_w = (image_width + 15) / 16, tile_h = (image_height + 15) / 16;
    const uint32_t n_tiles = tile_w * tile_h * I;
    const int64_t cap = g_deferred_used;
    if (cap >= ((int64_t)1 << 31)) throw std::runtime_error("do_intersect_tile_generic: capacity beyond 2^31-1 intersections");
    int32_t* offs = DevicePool::global().acquire<int32_t>(PoolSlot::IsectOffsets, (size_t)n_tiles + 1);
    DeviceTensor3D<int32_t> offsets(offs, I, tile_h, tile_w);
    DeviceVector<int64_t> ids_a, ids_b; ids_a.resize(PoolSlot::IsectIdsA, cap); ids_b.resize(PoolSlot::IsectIdsB, cap);
    DeviceVector<int32_t> flat_a, flat_b; flat_a.resize(PoolSlot::IsectFlatA, cap); flat_b.resize(PoolSlot::IsectFlatB, cap);
    {
        StageTimer t(&g_times.k4);
        ssr_tile_write_capped_params p;
        std::memset(&p, 0, sizeof(p));
        p.n = total; p.num_images = (int32_t)I; p.rows_per_image = img_ids ? 0 : total / I; p.image_ids = img_ids;
        p.aabb = aabb.data_ptr(); p.sort_depth = depths.data_ptr(); p.xy = proj_xy.data_ptr(); p.conic = proj_conic.data_ptr();
        p.opac = proj_opac.data_ptr(); p.cum_tiles = cum.data_ptr(); p.width = image_width; p.height = image_height;
        p.isect_ids = ids_a.data_ptr(); p.flatten_ids = flat_a.data_ptr(); p.capacity = cap;
        if (g_visible_ids && I == 1) {
            p.visible_ids = g_visible_ids; p.n_visible = g_counters + 1;
        }
        p.tile_active = tile_active;
        ok(ssr_tile_write_capped(&p, nullptr), "do_intersect_tile_generic/write");
    }
    int selector = 0;
    {
        StageTimer t(&g_times.k5);
        const size_t sb = ssr_sort_tile_scratch_bytes(cap, n_tiles);
        void* scratch = DevicePool::global().acquire<uint8_t>(PoolSlot::IsectSortScratch, sb);
        ok(ssr_sort_tile_pairs_capped(ids_a.data_ptr(), ids_b.data_ptr(), flat_a.data_ptr(), flat_b.data_ptr(), cap, g_counters,
                                      n_tiles, offs, &selector, scratch, sb, nullptr), "do_intersect_tile_generic/tile_sort");
    }
    g_offsets_closed = offs;
    {
        StageTimer t(&g_times.k6);
        const size_t sb = ssr_tile_order_scratch_bytes(n_tiles);
        int32_t* order = DevicePool::global().acquire<int32_t>(PoolSlot::IsectTileOrder, (size_t)n_tiles + sb / sizeof(int32_t));
        ok(ssr_tile_order(offs, n_tiles, -1, order, order + n_tiles, sb, nullptr), "do_intersect_tile_generic/order");
        g_tile_order = order; g_tile_order_for = offs;
    }
    return std::make_tuple(selector ? ids_b : ids_a, selector ? flat_b : flat_a, offsets);
}
}  // namespace

std::tuple<DeviceVector<int64_t>, DeviceVector<int32_t>, DeviceTensor3D<int32_t>>
do_intersect_tile_generic(DeviceTensorFloatND aabb, DeviceTensorFloatND depths, DeviceTensorFloatND* proj_xy,
                          DeviceTensorFloatND* proj_conic, DeviceTensorFloatND* proj_opac, const uint32_t I,
                          TorchTensorView, const uint32_t image_width, const uint32_t image_height,
                          DeviceVector<int32_t>* image_ids, const int32_t* tile_active) {
    // Packed mode (image_ids given): `total` rows, one per visible (camera, splat) pair, and the
    // values written to flatten_ids are row numbers (src/kernels/tile/IntersectTile.cu:386-409). With
    // the single camera this backend runs, every image id is 0 and the array itself is not read.
    if (!proj_xy || !proj_conic || !proj_opac)
        throw std::runtime_error("do_intersect_tile_generic: AABB mode is not built in this backend (ellipse mode is)");
    if (I < 1) throw std::runtime_error("do_intersect_tile_generic: no image");
    g_tile_order = nullptr; g_tile_order_for = nullptr; g_offsets_closed = nullptr;
    g_block_masks = nullptr; g_block_masks_for = nullptr;   // new keys: the last forward's block masks are void
    if (g_counts_pending) {   // counts nobody asked for: settle them before the counters are reused
        try { ssr_ext::resolve_counts(); } catch (const std::runtime_error&) {}   // a short frame stays in short_frames() / last_error()
    }
    const int64_t total = depths.numel();
    const int32_t* img_ids = (image_ids && I > 1) ? image_ids->data_ptr() : nullptr;   // packed rows of several cameras
    if (!img_ids && total % I != 0) throw std::runtime_error("do_intersect_tile_generic: rows are not a multiple of the image count");
    const uint32_t tile_w = (image_width + 15) / 16, tile_h = (image_height + 15) / 16;
    const uint32_t n_tiles = tile_w * tile_h * I;

    DeviceVector<int64_t> tiles_per_splat; tiles_per_splat.resize(PoolSlot::IsectTilesPerSplat, total);
    // counts fused into the projection know nothing of a tile-skip map: count again when one is given
    if (!g_counts_fused || tile_active) {
        StageTimer t(&g_times.k2);
        if (I > 1)
            ok(ssr_tile_count_images(total, img_ids ? 0 : total / I, img_ids, (int32_t)I, aabb.data_ptr(), proj_xy->data_ptr(),
                                     proj_conic->data_ptr(), proj_opac->data_ptr(), image_width, image_height, tile_active,
                                     tiles_per_splat.data_ptr(), nullptr), "do_intersect_tile_generic/count");
        else
        ok(ssr_tile_count(total, aabb.data_ptr(), proj_xy->data_ptr(), proj_conic->data_ptr(), proj_opac->data_ptr(),
                          image_width, image_height, tile_active, tiles_per_splat.data_ptr(), nullptr), "do_intersect_tile_generic/count");
    } else {
        g_times.k2 = 0;
    }
    g_counts_fused = false;
    DeviceVector<int64_t> cum; cum.resize(PoolSlot::IsectCumTiles, total);
    int64_t n_isects = 0;
    {
        StageTimer t(&g_times.k3);
        const size_t sb = ssr_scan_scratch_bytes(total);
        void* scratch = DevicePool::global().acquire<uint8_t>(PoolSlot::IsectScanScratch, sb);
        if (!g_counters) g_counters = counters_pair(false);
        ok(ssr_inclusive_sum_i64(tiles_per_splat.data_ptr(), cum.data_ptr(), total, g_counters, scratch, sb, nullptr),
           "do_intersect_tile_generic/scan");
        if (total > 0 && g_opts.deferred_counts && g_opts.tile_sort && g_deferred_capacity > 0) {
            // the counts follow the scan to pinned memory; nobody waits here
            if (!g_counts_host) {
                g_counts_host = static_cast<int64_t*>(ssr_host_malloc_pinned(2 * sizeof(int64_t)));
                g_counts_event = ssr_event_create();
                if (!g_counts_host || !g_counts_event) throw_last("do_intersect_tile_generic/pinned counts");
            }
            ok(ssr_memcpy(g_counts_host, g_counters, 2 * sizeof(int64_t), 2 /* device to host */, nullptr, 1),
               "do_intersect_tile_generic/counts");
            ok(ssr_event_record(g_counts_event, nullptr), "do_intersect_tile_generic/counts");
            g_counts_pending = true;
            g_deferred_used = g_deferred_capacity;
        } else if (total > 0) {
            int64_t both[2] = {0, 0};
            ok(ssr_read_i64(g_counters, both, g_visible_ids ? 2 : 1, nullptr), "do_intersect_tile_generic/readback");
            n_isects = both[0];
            if (g_visible_ids) g_seen_visible = g_n_visible = both[1];
        }
    }
    if (g_counts_pending)
        return intersect_tile_deferred(aabb, depths, *proj_xy, *proj_conic, *proj_opac, I, image_width, image_height, img_ids,
                                       tile_active, cum, total);
    g_n_isects = n_isects;
    if (g_opts.deferred_counts) g_deferred_capacity = capacity_for(n_isects);
    DeviceTensor3D<int32_t> offsets; offsets.resize(PoolSlot::IsectOffsets, I, tile_h, tile_w);
    if (n_isects == 0) {
        offsets.zero();
        return std::make_tuple(DeviceVector<int64_t>{}, DeviceVector<int32_t>{}, offsets);
    }
    if (n_isects >= ((int64_t)1 << 31)) throw std::runtime_error("do_intersect_tile_generic: more than 2^31-1 intersections");
    DeviceVector<int64_t> ids_a, ids_b; ids_a.resize(PoolSlot::IsectIdsA, n_isects); ids_b.resize(PoolSlot::IsectIdsB, n_isects);
    DeviceVector<int32_t> flat_a, flat_b; flat_a.resize(PoolSlot::IsectFlatA, n_isects); flat_b.resize(PoolSlot::IsectFlatB, n_isects);
    {
        StageTimer t(&g_times.k4);
        if (I > 1)   // keys carry image * tiles + tile (IntersectTile.cu:215-262)
            ok(ssr_tile_write_images(total, img_ids ? 0 : total / I, img_ids, (int32_t)I, aabb.data_ptr(), depths.data_ptr(),
                                     proj_xy->data_ptr(), proj_conic->data_ptr(), proj_opac->data_ptr(), cum.data_ptr(),
                                     image_width, image_height, ids_a.data_ptr(), flat_a.data_ptr(), tile_active, nullptr),
               "do_intersect_tile_generic/write");
        else
        ok(ssr_tile_write(total, aabb.data_ptr(), depths.data_ptr(), proj_xy->data_ptr(), proj_conic->data_ptr(),
                          proj_opac->data_ptr(), cum.data_ptr(), image_width, image_height, ids_a.data_ptr(),
                          flat_a.data_ptr(), g_visible_ids, g_visible_ids ? g_n_visible : 0, tile_active, nullptr),
           "do_intersect_tile_generic/write");
    }
    int selector = 0;
    {
        StageTimer t(&g_times.k5);
        const size_t sb = g_opts.tile_sort ? ssr_sort_tile_scratch_bytes(n_isects, n_tiles) : ssr_sort_scratch_bytes(n_isects);
        void* scratch = DevicePool::global().acquire<uint8_t>(PoolSlot::IsectSortScratch, sb);
        if (g_opts.tile_sort)   // also writes the offsets
            ok(ssr_sort_tile_pairs(ids_a.data_ptr(), ids_b.data_ptr(), flat_a.data_ptr(), flat_b.data_ptr(), n_isects, n_tiles,
                                   offsets.data_ptr(), &selector, scratch, sb, nullptr), "do_intersect_tile_generic/tile_sort");
        else
            ok(ssr_sort_pairs_u64_i32(ids_a.data_ptr(), ids_b.data_ptr(), flat_a.data_ptr(), flat_b.data_ptr(), n_isects, 0,
                                      ssr_sort_end_bit(n_tiles), &selector, scratch, sb, nullptr), "do_intersect_tile_generic/sort");
    }
    DeviceVector<int64_t> ids_out = selector ? ids_b : ids_a;
    DeviceVector<int32_t> flat_out = selector ? flat_b : flat_a;
    if (!g_opts.tile_sort) {
        StageTimer t(&g_times.k6);
        ok(ssr_tile_offsets(n_isects, ids_out.data_ptr(), n_tiles, offsets.data_ptr(), nullptr), "do_intersect_tile_generic/offsets");
    }
    if (g_opts.tile_sort) {   // the native stage order also launches each XCD's longest tiles first
        StageTimer t(&g_times.k6);   // the offsets themselves came out of the sort
        // one slot: the order, then the scratch of the counting sort behind it
        const size_t sb = ssr_tile_order_scratch_bytes(n_tiles);
        int32_t* order = DevicePool::global().acquire<int32_t>(PoolSlot::IsectTileOrder, (size_t)n_tiles + sb / sizeof(int32_t));
        ok(ssr_tile_order(offsets.data_ptr(), n_tiles, n_isects, order, order + n_tiles, sb, nullptr), "do_intersect_tile_generic/order");
        g_tile_order = order; g_tile_order_for = offsets.data_ptr();
    }
    return std::make_tuple(ids_out, flat_out, offsets);
}

std::tuple<RenderOutput::TensorTuple, DeviceTensor3D<float>, DeviceTensor3D<int32_t>, RenderOutput::TensorTuple,
           DeviceTensor3D<float>>
rasterize_to_pixels_3dgs_fwd(int64_t num_splats, std::vector<DeviceTensorFloatND>, std::vector<DeviceTensorFloatND> splats_s,
                             DeviceVector<int32_t> gaussian_ids, const uint32_t image_width, const uint32_t image_height,
                             const DeviceTensor3D<int32_t> tile_offsets, const DeviceVector<int32_t> flatten_ids,
                             DistortionType dist_type, bool output_median) {
    // gaussian_ids (packed mode) maps a screen row to its world row; the 3dgs fragment is read from
    // the screen row alone (src/kernels/raster/RasterizationEval3DFwd_kernel.cuh:183-184), so it is
    // accepted and not read.
    if (gaussian_ids.data_ptr()) num_splats = gaussian_ids.size();
    if (dist_type == DistortionType::DN || dist_type == DistortionType::RGB_DN)
        throw std::runtime_error("rasterize_to_pixels_3dgs_fwd: normal distortion needs a normal channel, which the 3dgs pixel does not have");
    const int64_t I = tile_offsets.size<0>();
    if (I < 1) throw std::runtime_error("rasterize_to_pixels_3dgs_fwd: no image");
    RenderOutput::TensorTuple renders;
    std::get<0>(renders).resize(PoolSlot::RendersRgb, I, image_height, image_width);
    std::get<1>(renders).resize(PoolSlot::RendersDepth, I, image_height, image_width);
    DeviceTensor3D<float> Ts; Ts.resize(PoolSlot::RenderTs, I, image_height, image_width);
    DeviceTensor3D<int32_t> last; last.resize(PoolSlot::RenderLastIds, I, image_height, image_width);
    ssr_raster_fwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.num_splats = I > 1 && !splats_s.empty() ? splats_s[0].rows() : num_splats;   // [C,N] rows, or the packed rows of C cameras
    p.num_images = (int32_t)I;
    if (flatten_ids.size() > 0) p.screen = screen_of(splats_s);
    p.width = image_width; p.height = image_height;
    p.tile_offsets = tile_offsets.data_ptr(); p.flatten_ids = flatten_ids.data_ptr(); p.n_isects = flatten_ids.size();
    if (g_tile_order && g_tile_order_for == p.tile_offsets) p.tile_order = g_tile_order;
    p.tile_offsets_closed = (g_offsets_closed && g_offsets_closed == p.tile_offsets) ? 1 : 0;
    p.render_rgb = (float*)std::get<0>(renders).data_ptr(); p.render_depth = std::get<1>(renders).data_ptr();
    p.render_T = Ts.data_ptr(); p.last_ids = last.data_ptr();
    if (g_packed_rows && p.screen.xy == g_packed_for_xy) p.packed_rows = g_packed_rows;
    g_block_masks = nullptr; g_block_masks_for = nullptr;
    if (p.n_isects > 0) {   // the block masks of every staged entry, for the backward of these same keys
        uint16_t* bm = DevicePool::global().acquire<uint16_t>(PoolSlot::IsectBlockMasks, (size_t)p.n_isects);
        p.block_masks = bm;
        g_block_masks = bm; g_block_masks_for = p.flatten_ids;
    }
    // distortion channels present in dist_type only (RenderOutput::resizeDistortion, src/primitives/Primitive.cuh:88-101)
    RenderOutput::TensorTuple distortions;
    DeviceTensor3D<float> median;
    p.dist_type = (int32_t)dist_type;
    if (dist_type != DistortionType::None) {
        std::get<1>(distortions).resize(PoolSlot::RenderDistortionDepth, I, image_height, image_width);
        p.distortion_depth = std::get<1>(distortions).data_ptr();
        if (dist_type == DistortionType::RGB_D) {
            std::get<0>(distortions).resize(PoolSlot::RenderDistortionRgb, I, image_height, image_width);
            p.distortion_rgb = (float*)std::get<0>(distortions).data_ptr();
        }
    }
    if (output_median) {
        median.resize(PoolSlot::RenderMedian, I, image_height, image_width);
        p.render_median = median.data_ptr();
    }
    {
        StageTimer t(&g_times.k7);
        ok(ssr_raster_fwd(&p, nullptr), "rasterize_to_pixels_3dgs_fwd");
    }
    return std::make_tuple(renders, Ts, last, distortions, median);
}

std::tuple<std::vector<DeviceTensorFloatND>, std::vector<DeviceTensorFloatND>, DeviceVector<float>>
rasterize_to_pixels_3dgs_bwd(int64_t num_splats, std::vector<DeviceTensorFloatND> splats_w,
                             std::vector<DeviceTensorFloatND> splats_s, DeviceVector<int32_t> gaussian_ids,
                             const uint32_t image_width, const uint32_t image_height,
                             const DeviceTensor3D<int32_t> tile_offsets, const DeviceVector<int32_t> flatten_ids,
                             const DeviceTensor3D<float> render_Ts, const DeviceTensor3D<int32_t> last_ids,
                             RenderOutput::TensorTuple render_outputs_tuple,
                             std::optional<RenderOutput::TensorTuple> distortion_fwd_outputs, DistortionType dist_type, DeviceTensor3D<float> accum_weight_map, DensifyAccumMode accum_mode,
                             RenderOutput::TensorTuple v_render_outputs, const DeviceTensor3D<float> v_render_Ts,
                             const DeviceTensor3D<float> v_median,
                             std::optional<RenderOutput::TensorTuple> v_distortion_outputs,
                             std::optional<std::vector<DeviceTensorFloatND>> v_splats_w,
                             std::optional<std::vector<DeviceTensorFloatND>> v_splats_s) {
    const int64_t num_world = num_splats;   // rows of accum_weight (src/kernels/raster/RasterizationBwd.cu:82-84)
    if (gaussian_ids.data_ptr()) num_splats = gaussian_ids.size();   // packed: v_screen has one row per screen row
    if (dist_type == DistortionType::DN || dist_type == DistortionType::RGB_DN)
        throw std::runtime_error("rasterize_to_pixels_3dgs_bwd: normal distortion needs a normal channel, which the 3dgs pixel does not have");
    if (dist_type != DistortionType::None && (!distortion_fwd_outputs || !v_distortion_outputs))
        throw std::runtime_error("rasterize_to_pixels_3dgs_bwd: distortion needs the forward distortion image and its gradient");
    if (accum_weight_map.data_ptr() == nullptr) accum_mode = DensifyAccumMode::None;   // src/kernels/raster/RasterizationBwd.cu:234
    std::vector<DeviceTensorFloatND> vs;
    if (v_splats_s) {
        g_vrows = nullptr; g_vrows_for_xy = nullptr;
        vs = *v_splats_s;   // caller-provided accumulators are added into as they are
    } else {
        // the launcher owns and zero-fills v_screen (src/kernels/raster/RasterizationBwd.cu:143-146);
        // the five arrays sit back to back in one slot so that one fill clears them all
        const int64_t n = splats_s.empty() ? 0 : splats_s[0].rows();
        const int ch[5] = {2, 1, 3, 1, 3};
        float* base = DevicePool::global().acquire<float>(PoolSlot::RasterBwdVScreenXy, (size_t)(n * 10));
        g_vrows = nullptr; g_vrows_for_xy = nullptr;
        if (g_opts.packed_vscreen) {   // the rows take the gradients; the five arrays stay unfilled
            g_vrows = DevicePool::global().acquire<float>(PoolSlot::RasterBwdVRows, (size_t)(n * 12));
            g_vrows_for_xy = base;
            backend::memset_async(g_vrows, 0, (size_t)(n * 12) * sizeof(float));
        } else {
            backend::memset_async(base, 0, (size_t)(n * 10) * sizeof(float));
        }
        int64_t off = 0;
        for (int i = 0; i < 5; i++) {
            vs.emplace_back(base + off, std::vector<int64_t>{n, ch[i]});
            off += n * ch[i];
        }
    }
    ssr_raster_bwd_params p;
    std::memset(&p, 0, sizeof(p));
    const int64_t I = tile_offsets.size<0>();
    p.num_splats = I > 1 && !splats_s.empty() ? splats_s[0].rows() : num_splats;   // [C,N] rows
    p.num_images = (int32_t)I;
    p.screen = screen_of(splats_s);
    p.width = image_width; p.height = image_height;
    p.tile_offsets = tile_offsets.data_ptr(); p.flatten_ids = flatten_ids.data_ptr(); p.n_isects = flatten_ids.size();
    if (g_tile_order && g_tile_order_for == p.tile_offsets) p.tile_order = g_tile_order;
    p.tile_offsets_closed = (g_offsets_closed && g_offsets_closed == p.tile_offsets) ? 1 : 0;
    if (g_block_masks && g_block_masks_for == p.flatten_ids) p.block_masks = g_block_masks;
    {
        // The lane-per-fragment cut pays where a splat reaches several 4x4 blocks of a tile, which shows as tiles per
        // visible splat. Measured (K8, rows / lanes, ms): 3.9 tiles per splat 0.109 / 0.080 (100k splats, 800x800);
        // 3.7: 0.50 / 0.40 (1M, 1080p); 2.4: 0.592 / 0.558 (10M seen from inside, 4k); 1.9: 0.357 / 0.372 (3M, 1080p);
        // 1.8: 1.45 / 1.57 (6M, equirectangular 4096x2048). The counts are the last ones the host has seen (with deferred counts, the
        // iteration before's: a backward that needs no count of its own does not wait for this iteration's).
        const int64_t rows_seen = g_packed_mode ? p.num_splats : (g_n_visible >= 0 ? g_n_visible : g_seen_visible);
        const int64_t pairs_seen = g_n_isects > 0 ? g_n_isects : p.n_isects;
        p.schedule = (rows_seen > 0 && 5 * pairs_seen >= 11 * rows_seen) ? SSR_BWD_SCHEDULE_LANES : SSR_BWD_SCHEDULE_ROWS;
        if (g_opts.backward_schedule >= 0) p.schedule = g_opts.backward_schedule ? SSR_BWD_SCHEDULE_LANES : SSR_BWD_SCHEDULE_ROWS;
    }
    p.render_T = render_Ts.data_ptr(); p.last_ids = last_ids.data_ptr(); p.render_depth = std::get<1>(render_outputs_tuple).data_ptr();
    p.v_render_rgb = (const float*)std::get<0>(v_render_outputs).data_ptr();
    p.v_render_depth = std::get<1>(v_render_outputs).data_ptr();
    p.v_render_T = v_render_Ts.data_ptr();
    p.v_screen = screen_of(vs);
    if (g_packed_rows && p.screen.xy == g_packed_for_xy) p.packed_rows = g_packed_rows;
    if (g_vrows && p.v_screen.xy == g_vrows_for_xy) p.v_rows = g_vrows;
    p.dist_type = (int32_t)dist_type;
    if (dist_type != DistortionType::None) {
        p.distortion_depth = std::get<1>(*distortion_fwd_outputs).data_ptr();
        p.v_distortion_depth = std::get<1>(*v_distortion_outputs).data_ptr();
        if (dist_type == DistortionType::RGB_D) {
            p.render_rgb = (const float*)std::get<0>(render_outputs_tuple).data_ptr();
            p.distortion_rgb = (const float*)std::get<0>(*distortion_fwd_outputs).data_ptr();
            p.v_distortion_rgb = (const float*)std::get<0>(*v_distortion_outputs).data_ptr();
        }
    }
    p.v_render_median = v_median.data_ptr();
    DeviceVector<float> accum;
    p.accum_mode = (int32_t)accum_mode;
    if (accum_mode != DensifyAccumMode::None) {   // RasterizationBwd.cu:157-163
        accum.resize(PoolSlot::RasterBwdAccumWeight, num_world * (accum_mode == DensifyAccumMode::Avg ? 2 : 1));
        accum.zero();
        p.accum_weight_map = accum_weight_map.data_ptr();
        p.accum_weight = accum.data_ptr();
        p.num_world = num_world;
        p.gaussian_ids = gaussian_ids.data_ptr();
    }
    {
        StageTimer t(&g_times.k8);
        ok(ssr_raster_bwd(&p, nullptr), "rasterize_to_pixels_3dgs_bwd");
    }
    std::vector<DeviceTensorFloatND> vw = v_splats_w ? *v_splats_w : std::vector<DeviceTensorFloatND>{};
    (void)splats_w;
    return std::make_tuple(vw, vs, accum);
}

void projection_3dgs_backward(const int64_t num_splats, const int max_sh_degree,
                              const std::vector<DeviceTensorFloatND>& splats_world, TorchTensorView viewmats,
                              TorchTensorView intrins, const uint32_t image_width, const uint32_t image_height,
                              const std::string camera_model, const std::string distortion, const TorchTensorView dist_coeffs,
                              const DeviceVector<int32_t> camera_ids, const DeviceVector<int32_t> gaussian_ids,
                              const DeviceTensor2D<float4> aabb, const std::vector<DeviceTensorFloatND>& v_splats_screen,
                              const std::vector<DeviceTensorFloatND>& v_splats_world, DeviceTensor2D<float>* v_viewmats,
                              const std::optional<TorchTensorView> sh_value_packed,
                              const std::optional<TorchTensorView> sh_value_bounds, const uint32_t num_sh_buffer,
                              const int sh_value_bits, const int64_t sh_bounds_stride) {

    const bool is_packed = camera_ids.data_ptr() && gaussian_ids.data_ptr();   // src/kernels/projection/ProjectionBwd.cu:80
    g_bwd_list = nullptr; g_bwd_count = 0;
    if (num_splats == 0) return;   // ProjectionBwd.cu:86-87
    // a packed forward with no visible splat leaves ids and aabb null: nothing to do (ProjectionBwd.cu:89-97)
    if (!is_packed && !aabb.data_ptr()) return;
    ssr_projection_bwd_params p;
    std::memset(&p, 0, sizeof(p));
    p.num_splats = num_splats;
    ssr_ext::resolve_counts();   // the work list's length, when the forward left it on the device
    p.sh_degree = max_sh_degree;
    p.antialiased = g_antialiased ? 1 : 0;
    p.world = world_of(splats_world);
    p.sh = sh_of(sh_value_packed, sh_value_bounds, num_sh_buffer, sh_value_bits, sh_bounds_stride);
    const ssr_camera cameras = camera_of(camera_model, distortion, dist_coeffs, viewmats, intrins, image_width, image_height, true);
    const int64_t C = cameras.num_cameras;
    p.camera = camera_at(cameras, 0);
    p.aabb = (const float*)aabb.data_ptr();
    p.v_screen = screen_of(v_splats_screen);
    if (g_vrows && p.v_screen.xy == g_vrows_for_xy) p.v_rows = g_vrows;
    p.v_world = world_of(v_splats_world);
    p.accumulate = g_opts.overwrite_world_grads ? 0 : 1;
    if (v_viewmats) p.v_viewmat = v_viewmats->data_ptr();   // [C, 16]: accumulated into, as the reference does
    if (is_packed) {
        p.aabb = nullptr;
        p.packed_gaussian_ids = gaussian_ids.data_ptr(); p.num_packed = camera_ids.size();
        p.packed_ids_unique = 1;   // one camera per call: the packed projection lists a splat once
        if (g_world_rows && gaussian_ids.data_ptr() == g_world_rows_for_ids && (int64_t)camera_ids.size() == g_world_rows_count &&
            p.world.means == g_world_rows_for_means)
            { p.packed_world_rows = g_world_rows; p.packed_world_stride = g_world_rows_count; }
        g_bwd_list = gaussian_ids.data_ptr(); g_bwd_count = camera_ids.size();
    } else if (g_visible_ids && g_n_visible >= 0) {
        // the rows that end up non-zero are the listed ones either way
        g_bwd_list = g_visible_ids; g_bwd_count = g_n_visible;
        if (!ssr_ext::backward_overwrites_all_rows(num_splats)) { p.visible_ids = g_visible_ids; p.n_visible = g_n_visible; }
    }
    StageTimer t(&g_times.k9);
    if (is_packed && C > 1) {
        // Packed rows of several cameras are ordered by camera: one launch per camera over its run of rows, the first
        // in the mode the options ask for, the others adding (the reference's single launch adds atomically,
        // ProjectionBwd_kernel.cuh:107). The runs are those of the packed projection that produced the rows; rows
        // that did not come from it are split by reading camera_ids back.
        const int64_t total = camera_ids.size();
        std::vector<int64_t> counts = g_packed_counts;
        int64_t sum = 0;
        for (int64_t v : counts) sum += v;
        if ((int64_t)counts.size() != C || sum != total) {
            std::vector<int32_t> host_ids((size_t)total);
            backend::memcpy_sync(host_ids.data(), camera_ids.data_ptr(), (size_t)total * sizeof(int32_t), backend::MemcpyKind::DeviceToHost);
            counts.assign((size_t)C, 0);
            int32_t prev = 0;
            for (int32_t c : host_ids) {
                if (c < prev || c >= C) throw std::runtime_error("projection_3dgs_backward: packed rows must be ordered by camera id");
                counts[(size_t)c]++; prev = c;
            }
        }
        const ssr_projection_bwd_params all = p;
        int64_t row0 = 0;
        bool first_launch = true;
        for (int64_t c = 0; c < C; c++) {
            const int64_t rows = counts[(size_t)c];
            if (rows > 0) {
                p.camera = camera_at(cameras, (uint32_t)c);
                p.packed_gaussian_ids = all.packed_gaussian_ids + row0; p.num_packed = rows;
                p.v_screen = screen_rows_from(all.v_screen, row0);
                if (all.v_rows) p.v_rows = all.v_rows + 12 * row0;
                if (all.packed_world_rows) p.packed_world_rows = all.packed_world_rows + 4 * row0;
                if (all.v_viewmat) p.v_viewmat = all.v_viewmat + 16 * c;
                p.accumulate = first_launch ? all.accumulate : 1;
                ok(ssr_projection_bwd(&p, nullptr), "projection_3dgs_backward");
                first_launch = false;
            }
            row0 += rows;
        }
        return;
    }
    ok(ssr_projection_bwd(&p, nullptr), "projection_3dgs_backward");
    // further cameras: one launch each over row block c of the [C,N,...] gradients, added into the
    // world gradients the first launch wrote (the reference's single launch sums them with
    // atomicStore, src/kernels/projection/ProjectionBwd_kernel.cuh:107)
    const ssr_projection_bwd_params first = p;
    for (int64_t c = 1; c < C; c++) {
        p.camera = camera_at(cameras, (uint32_t)c);
        p.aabb = first.aabb + 4 * c * num_splats;
        p.v_screen = screen_rows_from(first.v_screen, c * num_splats);
        if (first.v_rows) p.v_rows = first.v_rows + 12 * c * num_splats;
        if (first.v_viewmat) p.v_viewmat = first.v_viewmat + 16 * c;
        p.accumulate = 1;
        ok(ssr_projection_bwd(&p, nullptr), "projection_3dgs_backward");
    }
}

void fused_projection_bwd_optimizer_3dgs(
    const int64_t num_splats, const int max_sh_degree, std::vector<DeviceTensorFloatND> splats_world,
    TorchTensorView viewmats, TorchTensorView intrins, const uint32_t image_width, const uint32_t image_height,
    const std::string camera_model, const std::string distortion, const TorchTensorView dist_coeffs,
    const DeviceVector<int32_t> camera_ids, const DeviceVector<int32_t> gaussian_ids, DeviceTensorFloatND aabb,
    const std::vector<DeviceTensorFloatND> v_splats_world, const std::vector<DeviceTensorFloatND> v_splats_screen,
    const std::vector<DeviceTensorFloatND> g1_splats_world, const std::vector<DeviceTensorFloatND> g2_splats_world,
    const std::optional<TorchTensorView> sh_packed, const std::optional<TorchTensorView> sh_quant_bounds,
    const std::optional<TorchTensorView> sh_value_packed, const std::optional<TorchTensorView> sh_value_bounds, NonShQuantState non_sh,
    DeviceVector<float> radii, DeviceVector<float> densify_score, const float lr_means, const float lr_quats,
    const float lr_scales, const float lr_opacs, const float lr_features_dc, const float lr_features_sh,
    const float max_gauss_ratio, const float scale_regularization_weight, const float mcmc_opacity_reg_weight,
    const float mcmc_scale_reg_weight, const float erank_reg_weight, const float erank_reg_weight_s3,
    const float quat_norm_reg_weight, const float sh_reg_weight, bool use_scale_agnostic_mean, bool color_trust_linear,
    float eps_tr, std::variant<int32_t, TorchTensorView> step, int quantization_level) {
    const char* w = "fused_projection_bwd_optimizer_3dgs: ";
    ssr_ext::resolve_counts();   // no parameter is stepped on gradients of an intersection that did not fit
    ssr_ext::forget_packed_world_rows();   // the parameters change here
    const bool is_packed = camera_ids.data_ptr() && gaussian_ids.data_ptr();   // src/kernels/optim/FusedProjectionBwdOptim.cu:160
    // quantization_level: 0 = fp32 SH and moments; 1 = 16-bit SH values, 8-bit moments
    // (src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:1104-1111; validation as FusedProjectionBwdOptim.cu:386-400)
    if (quantization_level != 0 && quantization_level != 1) throw std::runtime_error(std::string(w) + "quantization_level must be 0 or 1");
    const bool quant = quantization_level == 1;
    if (quant && !(sh_packed && sh_quant_bounds && sh_value_packed && sh_value_bounds))
        throw std::runtime_error(std::string(w) + "quantization level 1 needs the packed SH state, the packed SH values and both bounds");
    if (!quant && (sh_packed || sh_value_packed)) throw std::runtime_error(std::string(w) + "packed SH buffers given at quantization level 0");
    if (num_splats == 0) return;
    ssr_fpbo_params p;
    std::memset(&p, 0, sizeof(p));
    p.num_splats = num_splats;
    p.sh_degree = max_sh_degree;
    p.antialiased = g_antialiased ? 1 : 0;
    p.world = world_of(splats_world);
    if (quant) {
        p.sh_state_packed = (uint16_t*)std::get<0>(*sh_packed);
        p.sh_state_bounds = (float*)std::get<0>(*sh_quant_bounds);
        p.sh_value_packed = (uint16_t*)std::get<0>(*sh_value_packed);
        p.sh_value_bounds = (float*)std::get<0>(*sh_value_bounds);
        p.num_sh_buffer = (uint32_t)(splats_world[5].channels() / 3);   // the buffers' stride, not the active degree
        if (non_sh.enabled) {   // read only at a quantized level, as in the kernel (FusedProjectionBwdOptim_kernel.cuh:378)
            uint8_t* pk[5] = {non_sh.means_packed, non_sh.quats_packed, non_sh.scales_packed, non_sh.opacities_packed, non_sh.features_dc_packed};
            float* bd[5] = {non_sh.means_bounds, non_sh.quats_bounds, non_sh.scales_bounds, non_sh.opacities_bounds, non_sh.features_dc_bounds};
            for (int t = 0; t < 5; t++) {
                if (!pk[t] || !bd[t]) throw std::runtime_error(std::string(w) + "non_sh.enabled with a null buffer");
                p.non_sh_packed[t] = reinterpret_cast<uint32_t*>(pk[t]);
                p.non_sh_bounds[t] = bd[t];
            }
        }
    }
    const ssr_camera cameras = camera_of(camera_model, distortion, dist_coeffs, viewmats, intrins, image_width, image_height, true);
    const int64_t C = cameras.num_cameras;
    p.camera = camera_at(cameras, 0);
    p.aabb = aabb.data_ptr();
    p.v_screen = screen_of(v_splats_screen);
    if (g_vrows && p.v_screen.xy == g_vrows_for_xy) p.v_rows = g_vrows;
    if (!v_splats_world.empty()) p.v_world_in = world_of(v_splats_world);
    p.v_world_in.features_sh = nullptr;   // not read (FusedProjectionBwdOptim_kernel.cuh:250-255)
    // rows of camera 0 in the packed layout (all of them with one camera)
    int64_t rows0 = is_packed ? (int64_t)gaussian_ids.size() : 0;
    StageTimer t(&g_times.k9);
    if (C > 1) {
        // A camera batch: the reference walks every camera's row of a splat inside its kernel and steps once with
        // the sum (FusedProjectionBwdOptim.cu:160-212, FusedProjectionBwdOptim_kernel.cuh:262-330). Here the
        // projection backward of cameras 1..C-1 adds into a scratch copy of the incoming gradients, SH included,
        // and the fused kernel runs camera 0 on top of that sum.
        const int64_t N = num_splats, S = splats_world[5].channels();
        float* tmp = DevicePool::global().acquire<float>(PoolSlot::FusedMultiCamGrad, (size_t)(N * (14 + S)));
        ssr_world acc;
        acc.means = tmp; acc.quats = tmp + 3 * N; acc.log_scales = tmp + 7 * N; acc.opacity_logits = tmp + 10 * N;
        acc.features_dc = tmp + 11 * N; acc.features_sh = tmp + 14 * N; acc.sh_stride = (int32_t)S;
        backend::memset_async(tmp, 0, (size_t)(N * (14 + S)) * sizeof(float));
        const float* src[5] = {p.v_world_in.means, p.v_world_in.quats, p.v_world_in.log_scales, p.v_world_in.opacity_logits, p.v_world_in.features_dc};
        float* dst[5] = {acc.means, acc.quats, acc.log_scales, acc.opacity_logits, acc.features_dc};
        const int64_t width5[5] = {3, 4, 3, 1, 3};
        for (int i = 0; i < 5; i++)
            if (src[i]) backend::memcpy_async(dst[i], src[i], (size_t)(N * width5[i]) * sizeof(float), backend::MemcpyKind::DeviceToDevice);
        std::vector<int64_t> counts;
        if (is_packed) {
            counts = g_packed_counts;
            int64_t sum = 0;
            for (int64_t v : counts) sum += v;
            if ((int64_t)counts.size() != C || sum != (int64_t)camera_ids.size())
                throw std::runtime_error(std::string(w) + "the packed rows of a camera batch must come from the preceding projection_3dgs_packed_forward");
            rows0 = counts[0];
        }
        ssr_projection_bwd_params b;
        std::memset(&b, 0, sizeof(b));
        b.num_splats = N; b.sh_degree = max_sh_degree; b.antialiased = p.antialiased;
        b.world = p.world;
        if (quant) {   // the coefficients are the 16-bit value codes, one bound per 256 splats
            b.sh.codec = SSR_SH_REF_Q16; b.sh.packed = p.sh_value_packed; b.sh.bounds = p.sh_value_bounds;
            b.sh.num_sh_buffer = p.num_sh_buffer; b.sh.bounds_stride = (int64_t)256 * 3 * p.num_sh_buffer;
        }
        b.v_world = acc; b.accumulate = 1; b.packed_ids_unique = 1;
        int64_t row = rows0;
        for (int64_t c = 1; c < C; c++) {
            b.camera = camera_at(cameras, (uint32_t)c);
            if (is_packed) {
                const int64_t rows = counts[(size_t)c];
                b.packed_gaussian_ids = gaussian_ids.data_ptr() + row; b.num_packed = rows;
                b.v_screen = screen_rows_from(p.v_screen, row);
                b.v_rows = p.v_rows ? p.v_rows + 12 * row : nullptr;
                row += rows;
                if (rows == 0) continue;
            } else {
                b.aabb = p.aabb + 4 * c * N;
                b.v_screen = screen_rows_from(p.v_screen, c * N);
                b.v_rows = p.v_rows ? p.v_rows + 12 * c * N : nullptr;
            }
            ok(ssr_projection_bwd(&b, nullptr), "fused_projection_bwd_optimizer_3dgs/other cameras");
        }
        p.v_world_in = acc;
        p.v_world_in.features_sh = nullptr;
        p.v_sh_in = acc.features_sh; p.v_sh_in_stride = (int32_t)S;
    }
    if (!g1_splats_world.empty()) p.g1 = world_of(g1_splats_world);
    if (!g2_splats_world.empty()) p.g2 = world_of(g2_splats_world);
    p.densify_score = densify_score.data_ptr();
    p.lr_means = lr_means; p.lr_quats = lr_quats; p.lr_scales = lr_scales; p.lr_opacs = lr_opacs;
    p.lr_features_dc = lr_features_dc; p.lr_features_sh = lr_features_sh;
    p.max_gauss_ratio = max_gauss_ratio; p.scale_regularization_weight = scale_regularization_weight;
    p.mcmc_opacity_reg_weight = mcmc_opacity_reg_weight; p.mcmc_scale_reg_weight = mcmc_scale_reg_weight;
    p.quat_norm_reg_weight = quat_norm_reg_weight; p.sh_reg_weight = sh_reg_weight;
    p.erank_reg_weight = erank_reg_weight; p.erank_reg_weight_s3 = erank_reg_weight_s3;
    p.color_trust_linear = color_trust_linear ? 1 : 0; p.eps_tr = eps_tr;
    if (use_scale_agnostic_mean) {
        if (!radii.data_ptr()) throw std::runtime_error(std::string(w) + "the scale-agnostic mean step needs the forward's radii");
        p.scale_agnostic_radii = radii.data_ptr();
    }
    if (const int32_t* s = std::get_if<int32_t>(&step)) {
        p.step = *s;
    } else {
        p.steps = (const int32_t*)std::get<0>(std::get<TorchTensorView>(step));
    }
    if (is_packed) {   // aabb and v_splats_screen hold nnz compacted rows: find each splat's row (camera 0's rows)
        int32_t* row_of = DevicePool::global().acquire<int32_t>(PoolSlot::FusedProjBwdRowOf, (size_t)num_splats);
        ok(ssr_packed_row_map(gaussian_ids.data_ptr(), rows0, num_splats, row_of, nullptr),
           "fused_projection_bwd_optimizer_3dgs/row map");
        p.packed_row_of = row_of;
    }
    ok(ssr_fused_projection_bwd_optimizer(&p, nullptr), "fused_projection_bwd_optimizer_3dgs");
}
