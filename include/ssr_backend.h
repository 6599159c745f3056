/* ssr_backend.h -- C ABI of the MI355X (gfx950) Gaussian-splat rasterizer hot path.
 *
 * One shared library, libssr_hip.so, exports exactly the entry points below. They are what a
 * third backend of the reference (beside its CUDA and Vulkan ones) binds for this path: each
 * replaces one launch function or runtime call of the reference's backend seam
 * (src/backend/api/{Projection,TileIntersect,Rasterization}.h, src/backend/api/BackendRuntime.h,
 * src/backend/common/SortScan.h). The C++ adapter in spirula-studio_amd/host/ re-creates the
 * reference's own C++ signatures on top of these.
 *
 * Conventions
 *  - Every data pointer is a DEVICE pointer unless named host_*. Sizes are element counts unless
 *    named *_bytes. No entry point allocates device memory; scratch is passed in by the caller
 *    (sizes from the *_scratch_bytes functions). No entry point synchronises except
 *    ssr_read_i64, ssr_*_synchronize, ssr_memcpy (sync form) and ssr_event_elapsed_ms.
 *  - `stream` is a hipStream_t passed as void*; NULL is the default stream, which is what the
 *    reference launches on (src/core/Common.cuh:207).
 *  - Return value 0 = success. Non-zero = error; the message is kept per thread and returned (and
 *    cleared) by ssr_last_error(), like the reference's sticky backend::last_error()
 *    (src/backend/api/BackendRuntime.h:98). Nothing calls exit().
 *  - Supported variants: primitives "3dgs" and "mip" (the antialiased one: `antialiased` in the projection
 *    parameter blocks); camera PINHOLE with lens NONE / OPENCV / THIN_PRISM / RATIONAL, FISHEYE and EQUISOLID
 *    with NONE / OPENCV / THIN_PRISM, EQUIRECTANGULAR with NONE (the reference's own table,
 *    src/kernels/projection/CameraVariants.cuh:11-22; ssr_camera_variant_supported answers for a pair);
 *    SH degree 0..3 in fp32 or one of the quantised codecs; dist_type None / D / RGB_D, median depth,
 *    accumulation weights; the [C,N] layout and the packed (compacted, nnz rows) layout of the projection
 *    outputs; the projection backward alone or fused with the Adam step. One camera per projection launch:
 *    the host layer loops over a [C,4,4] set (packed rows ordered by camera, then splat), while tiling,
 *    sorting and compositing take the C images in one launch. Anything else is rejected with an error, as the
 *    reference rejects an uncompiled variant (src/kernels/projection/ProjectionFwd.cu:84-89).
 *  - Layouts are the reference's (src/primitives/PrimitiveBase3DGS.cuh:87-139,187-225).
 */
#ifndef SSR_BACKEND_H
#define SSR_BACKEND_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ssr_stream_t;
typedef void* ssr_event_t;

enum { SSR_CAM_PINHOLE = 0, SSR_CAM_FISHEYE = 1, SSR_CAM_EQUISOLID = 2, SSR_CAM_EQUIRECT = 3 };   /* CameraModelType, src/core/Common.cuh */
/* CameraDistortionType (src/core/CameraModel.h; coefficient order per tier:
 * src/shaders/projection_utils.slang:242-295). Pairs accepted: src/kernels/projection/CameraVariants.cuh:11-22. */
enum { SSR_LENS_NONE = 0, SSR_LENS_OPENCV = 1, SSR_LENS_THIN_PRISM = 2, SSR_LENS_RATIONAL = 3 };
enum { SSR_SH_F32 = 0, SSR_SH_REF_Q8 = 1, SSR_SH_REF_Q16 = 2, SSR_SH_I8_F16SCALE = 3 };
enum { SSR_DIST_NONE = 0, SSR_DIST_D = 1, SSR_DIST_RGB_D = 2 };   /* DistortionType, src/primitives/Primitive.cuh:24-32 */
enum { SSR_ACCUM_NONE = 0, SSR_ACCUM_MAX = 1, SSR_ACCUM_SUM = 2, SSR_ACCUM_AVG = 3 };   /* DensifyAccumMode, :37-42 */
enum { SSR_MEMCPY_H2D = 0, SSR_MEMCPY_D2H = 1, SSR_MEMCPY_D2D = 2, SSR_MEMCPY_H2H = 3,
       SSR_MEMCPY_AUTO = 4 };                             /* backend::MemcpyKind */

/* WorldBuffer = TensorArray<6> (src/primitives/PrimitiveBase3DGS.cuh:87-139). */
typedef struct {
    float* means;           /* [N,3] */
    float* quats;           /* [N,4] w,x,y,z */
    float* log_scales;      /* [N,3] */
    float* opacity_logits;  /* [N] */
    float* features_dc;     /* [N,3] */
    float* features_sh;     /* [N,sh_stride] coefficient-major, channel innermost */
    int32_t sh_stride;      /* floats per splat in features_sh (45 for SH3) */
} ssr_world;

/* ScreenBuffer = TensorArray<5> (src/primitives/PrimitiveBase3DGS.cuh:187-225). */
typedef struct {
    float* xy;      /* [N,2] */
    float* depth;   /* [N]   */
    float* conic;   /* [N,3] */
    float* opac;    /* [N]   */
    float* rgb;     /* [N,3] */
} ssr_screen;

/* Quantized SH source. REF_Q8/REF_Q16: the reference's codec, uint8/uint16 codes plus float2
 * (min,max) per `bounds_stride` cells, cell = gid*3*num_sh_buffer + 3*j + ch
 * (src/shaders/harmonics.slang:92-140; launcher args src/kernels/projection/ProjectionFwd.cuh:27-35;
 * bounds_stride 0 selects 256*3*num_sh_buffer as there). I8_F16SCALE: int8 codes [N,45] times one
 * fp16 scale per splat (the benchmark's storage format; no counterpart in the reference). */
typedef struct {
    int32_t codec;              /* SSR_SH_* ; SSR_SH_F32 reads ssr_world.features_sh */
    const void* packed;
    const float* bounds;        /* float2[n_bounds] */
    int64_t bounds_stride;
    uint32_t num_sh_buffer;
    const uint16_t* scale_f16;  /* [N] */
} ssr_sh_quant;

typedef struct {
    int32_t camera_model;   /* SSR_CAM_* */
    uint32_t num_cameras;   /* must be 1 */
    uint32_t width, height;
    const float* viewmats;  /* device [C,4,4] row-major world->camera */
    const float* intrins;   /* device [C,4] fx,fy,cx,cy */
    const float* dist_coeffs;   /* device [C,8] lens coefficients in the tier's order; unused (may be
                                 * NULL) with SSR_LENS_NONE */
    int32_t distortion;     /* SSR_LENS_* */
} ssr_camera;

/* ---- K1: projection_3dgs_forward (src/kernels/projection/ProjectionFwd.cuh:18-36,
 * kernel src/kernels/projection/ProjectionFwd_kernel.cuh:17-111). Writes aabb/sort_depth for every
 * splat, the screen row and atomic-max radii only for visible ones (radii_store: every row). If tiles_per_splat is
 * non-NULL the tile count of K2 is produced in the same pass. */
typedef struct {
    int64_t num_splats;
    int32_t sh_degree;
    ssr_world world;
    ssr_sh_quant sh;
    ssr_camera camera;
    float* aabb;            /* [C,N,4] */
    float* sort_depth;      /* [C,N] */
    float* radii;           /* [N], caller zero-fills (src/engine/EngineForward.cpp:66-69) unless radii_store */
    ssr_screen screen;
    int64_t* tiles_per_splat; /* optional [C*N] */
    /* Optional work list (no counterpart in the reference's non-packed path): the indices of the
     * splats whose screen row was written, in no particular order, appended at *visible_count
     * (which the caller zeroes). Later stages can then run over V entries instead of N. */
    int32_t* visible_ids;     /* optional [C*N] */
    int64_t* visible_count;   /* required when visible_ids is given */
    /* Optional second copy of the visible screen rows as one 48-byte record per splat,
     * (x, y, conic.x/2, conic.y | conic.z/2, opac, r, g | b, depth, sigma cut, footprint scale),
     * 16-byte aligned, [C*N,12]. The compositing kernels gather a splat from it with one or two
     * cache lines instead of five (same values, so same results). */
    float* packed_rows;
    /* The antialiased ("mip") variant of the primitive (src/shaders/primitive_3dgs.slang:528-543, the runtime
     * `antialiased` argument of the same projection function): screen-space blur 0.1 instead of 0.3 and the opacity
     * multiplied by sqrt(det cov2d / det (cov2d + blur)); everything after the projection is unchanged. */
    int32_t antialiased;
    /* Non-zero: radii[g] is stored -- the radius of a visible splat, 0 of a culled one -- instead of max-accumulated.
     * For a launch that is the only writer of `radii` (one camera) this gives what the zero-fill and the atomic max
     * give, and the caller needs no zero-fill. */
    int32_t radii_store;
    /* Optional: an int64 this launch sets to zero. A caller that alternates between two visible counters has the
     * one of its NEXT projection cleared here, in place of a fill launch of its own before every projection. */
    int64_t* clear_count;
} ssr_projection_fwd_params;
int ssr_projection_fwd(const ssr_projection_fwd_params* p, ssr_stream_t stream);

/* ---- K1, packed form: projection_3dgs_packed_forward (src/kernels/projection/ProjectionPackedFwd.cuh:18-37;
 * kernels src/kernels/projection/ProjectionPackedFwd_kernel.cuh:17-184; launcher
 * src/kernels/projection/ProjectionPackedFwd.cu:64-158). The outputs hold one row per VISIBLE
 * splat, in ascending splat order: camera_ids / gaussian_ids / aabb / sort_depth / screen, nnz rows.
 * The reference runs mask -> inclusive scan -> blocking readback of nnz -> a second full projection
 * that writes the compacted rows. Here the first call projects every splat once, compacts the
 * visible ones inside each workgroup's 1024-splat segment of `scratch`, and scans the workgroup counts into
 * *nnz; the second call evaluates SH colour for the nnz staged rows and places them. Between the
 * two the caller may read *nnz back (ssr_read_i64) to size its outputs, or skip the readback and
 * pass capacity num_splats as max_rows. Rows past *nnz are not written. radii is max-accumulated
 * by splat index, as in the non-packed form. */
typedef struct {
    int64_t num_splats;
    int32_t sh_degree;
    ssr_world world;
    ssr_sh_quant sh;
    ssr_camera camera;
    float* radii;               /* [N], caller zero-fills */
    void* scratch;              /* ssr_projection_packed_scratch_bytes(num_splats), 16-byte aligned */
    size_t scratch_bytes;
    int64_t* nnz;               /* device scalar: written by _mask, read by _emit */
    int64_t max_rows;           /* _emit: capacity of the arrays below, in rows (>= *nnz) */
    int32_t* camera_ids;        /* [nnz] every entry = camera_index */
    int32_t* gaussian_ids;      /* [nnz] ascending */
    float* aabb;                /* [nnz,4] */
    float* sort_depth;          /* [nnz] */
    ssr_screen screen;          /* [nnz] rows */
    int64_t* tiles_per_splat;   /* optional [nnz]: fused K2 */
    float* packed_rows;         /* optional [nnz,12]: 48-byte fragment rows, as in ssr_projection_fwd_params */
    /* The antialiased ("mip") variant of the primitive (src/shaders/primitive_3dgs.slang:528-543, the runtime
     * `antialiased` argument of the same projection function): screen-space blur 0.1 instead of 0.3 and the opacity
     * multiplied by sqrt(det cov2d / det (cov2d + blur)); everything after the projection is unchanged. */
    int32_t antialiased;
    /* Value written into camera_ids (0 for a single camera). A camera set is packed by one mask / emit pair per
     * camera, each emit writing its rows behind the previous camera's, so that the rows are ordered by
     * (camera, splat) as the reference's single scan over C * N leaves them (ProjectionPackedFwd.cu:64-158). */
    int32_t camera_index;
    /* Optional [4][world_rows_stride][4], 16-byte aligned: the parameters of each visible splat in the order of the
     * packed rows, as four planes of 16-byte entries, (mean.xyz, opacity logit), (quat wxyz), (log_scale.xyz, dc.r),
     * (dc.g, dc.b, 0, 0); entry i of every plane belongs to packed row i, world_rows_stride >= max_rows. Where a
     * view sees a small, scattered part of the splats, ssr_projection_bwd reads these planes, consecutive lanes
     * consecutive entries, instead of gathering 4- to 16-byte pieces of five arrays, one cache line each
     * (ssr_projection_bwd_params::packed_world_rows). The mask call stages them when stage_world_rows is non-zero (the row count, and with it
     * this array, is not known before); both calls then need stage_world_rows set and a scratch of
     * ssr_projection_packed_scratch_bytes_world_rows(num_splats) bytes. No counterpart in the reference. */
    float* world_rows;
    int64_t world_rows_stride;
    int32_t stage_world_rows;
} ssr_projection_packed_params;
size_t ssr_projection_packed_scratch_bytes(int64_t num_splats);
size_t ssr_projection_packed_scratch_bytes_world_rows(int64_t num_splats);   /* with world_rows: 48 bytes per splat more */
int ssr_projection_packed_mask(const ssr_projection_packed_params* p, ssr_stream_t stream);
int ssr_projection_packed_emit(const ssr_projection_packed_params* p, ssr_stream_t stream);

/* ---- K2..K6: do_intersect_tile_generic, ellipse mode (src/kernels/tile/IntersectTile.cuh:25-41,
 * src/kernels/tile/IntersectTile.cu:376-509) split at its data-dependent allocation. */
/* tile_active (optional, [tile_h,tile_w], 0 = skip): a tile the loss never reads is left out by
 * both passes, so that compositing sees an empty range for it (IntersectTile.cu:117-119,165-166). */
int ssr_tile_count(int64_t n, const float* aabb, const float* xy, const float* conic,
                   const float* opac, uint32_t width, uint32_t height, const int32_t* tile_active,
                   int64_t* tiles_per_splat, ssr_stream_t stream);
/* compute_tile_active (IntersectTile.cu:316-368): tile_active[t] = 1 when any pixel of tile t,
 * grown by one pixel, is unmasked; `mask` is [mask_height, mask_width] bytes (non-zero = keep),
 * sampled at the nearest source pixel (src/core/Interpolation.cuh:108-120). */
int ssr_compute_tile_active(const uint8_t* mask, int32_t mask_height, int32_t mask_width,
                            uint32_t width, uint32_t height, int32_t* tile_active,
                            ssr_stream_t stream);
/* inclusive_sum<int64> (src/backend/common/SortScan.h:58-72; IntersectTile.cu:425-428). */
size_t ssr_scan_scratch_bytes(int64_t n);
/* total_out (optional) also receives out[n-1], so that it can sit next to other counters and be
 * read back in one copy. */
int ssr_inclusive_sum_i64(const int64_t* in, int64_t* out, int64_t n, int64_t* total_out,
                          void* scratch, size_t scratch_bytes, ssr_stream_t stream);
/* The same scan for callers that cannot allocate device memory or pass a workspace (code under
 * graph capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the
 * reference. The block sums live in a 512 KiB array inside the library (one copy per GPU, held until
 * the process ends), so n is limited to 2^27 = 134 217 728 elements; a larger n is rejected with an
 * error. Same kernels and same results as ssr_inclusive_sum_i64. Calls on one GPU share that
 * array: calls that overlap in time on one GPU (different streams, different threads) race. */
int ssr_inclusive_sum_i64_static(const int64_t* in, int64_t* out, int64_t n, int64_t* total_out,
                                 ssr_stream_t stream);
/* The reference's blocking readback of n_isects (8 bytes, IntersectTile.cu:432-436); `count`
 * consecutive values are copied. */
int ssr_read_i64(const int64_t* device_values, int64_t* host_values, int count, ssr_stream_t stream);
/* visible_ids (optional, with n_visible entries): run over that work list instead of all n splats;
 * the keys written are the same. */
int ssr_tile_write(int64_t n, const float* aabb, const float* sort_depth, const float* xy,
                   const float* conic, const float* opac, const int64_t* cum_tiles,
                   uint32_t width, uint32_t height, int64_t* isect_ids, int32_t* flatten_ids,
                   const int32_t* visible_ids, int64_t n_visible, const int32_t* tile_active,
                   ssr_stream_t stream);
/* The count and the key write over the rows of several images at once. Row r belongs to image
 * image_ids[r] when image_ids is given (packed rows: the camera_ids of the packed projection), else to image
 * r / rows_per_image (the [C,N] layout; n must then be num_images * rows_per_image). Its keys carry tile ids
 * offset by image * tiles-per-image (the reference's (camera_id * n_tiles + tile) key, IntersectTile.cu:215-262),
 * and tile_active, when given, holds one [tile_h, tile_w] block per image (IntersectTile.cuh:18-22). No work
 * list here. */
int ssr_tile_count_images(int64_t n, int64_t rows_per_image, const int32_t* image_ids, int32_t num_images,
                          const float* aabb, const float* xy, const float* conic, const float* opac,
                          uint32_t width, uint32_t height, const int32_t* tile_active, int64_t* tiles_per_splat,
                          ssr_stream_t stream);
int ssr_tile_write_images(int64_t n, int64_t rows_per_image, const int32_t* image_ids, int32_t num_images,
                          const float* aabb, const float* sort_depth, const float* xy, const float* conic,
                          const float* opac, const int64_t* cum_tiles, uint32_t width, uint32_t height,
                          int64_t* isect_ids, int32_t* flatten_ids, const int32_t* tile_active,
                          ssr_stream_t stream);
/* The key write for a caller that does not read the counts back (the reference blocks on n_isects,
 * IntersectTile.cu:432-436; no counterpart there). isect_ids / flatten_ids hold `capacity` entries, sized from an
 * earlier iteration; the real number of keys stays on the device (the scan's total), and so does the work list's
 * length *n_visible when visible_ids is given. Keys are those of ssr_tile_write / ssr_tile_write_images; none is
 * written at or beyond `capacity`, so a count above the capacity loses keys but touches no memory outside the
 * arrays: the caller compares the count with its capacity once it has read it (asynchronously) and repeats the
 * iteration with larger arrays if it did not fit. Entries from the real count up to `capacity` are not written;
 * ssr_sort_tile_pairs_capped and the compositing launches (tile_offsets_closed) never read them. */
typedef struct {
    int64_t n;                      /* rows: splats, or num_images * rows_per_image, or packed rows */
    int64_t rows_per_image;         /* with num_images > 1 and no image_ids */
    const int32_t* image_ids;       /* optional, [n]: packed rows of several images */
    int32_t num_images;
    const float* aabb; const float* sort_depth; const float* xy; const float* conic; const float* opac;
    const int64_t* cum_tiles;       /* [n] inclusive scan of the counts */
    uint32_t width, height;
    int64_t* isect_ids;             /* [capacity] */
    int32_t* flatten_ids;           /* [capacity] */
    int64_t capacity;
    const int32_t* visible_ids;     /* optional work list (one image) ... */
    const int64_t* n_visible;       /* ... and its length, on the device (the launch covers n rows) */
    const int32_t* tile_active;
} ssr_tile_write_capped_params;
int ssr_tile_write_capped(const ssr_tile_write_capped_params* p, ssr_stream_t stream);
/* sort_pairs<int64,int32> with CUB DoubleBuffer semantics (src/backend/common/SortScan.h:42-56;
 * call site IntersectTile.cu:486-493): stable on bits [begin_bit,end_bit); *selector says which
 * of the (a,b) buffers holds the result. */
size_t ssr_sort_scratch_bytes(int64_t n);
int ssr_sort_pairs_u64_i32(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b,
                           int64_t n, int begin_bit, int end_bit, int* selector, void* scratch,
                           size_t scratch_bytes, ssr_stream_t stream);
/* intersect_offset_kernel (IntersectTile.cu:271-307); zero-fills when n_isects == 0 (:448-451). */
int ssr_tile_offsets(int64_t n_isects, const int64_t* sorted_ids, uint32_t n_tiles,
                     int32_t* offsets, ssr_stream_t stream);
/* Launch order for the compositing kernels (their optional tile_order field): order[n_tiles] receives all tile
 * ids by descending fragment count (in classes of 32 fragments; the order inside a class is arbitrary). Workgroup
 * w of a compositing launch takes order[w]: workgroups start in index order and are dealt round-robin to the XCDs,
 * so the longest tiles start first and every XCD gets the same mix. scratch: ssr_tile_order_scratch_bytes.
 * No counterpart in the reference (its grid is one block per tile in index order). */
size_t ssr_tile_order_scratch_bytes(uint32_t n_tiles);
/* n_isects < 0: tile_offsets holds n_tiles + 1 entries, the last one ending the last tile
 * (ssr_sort_tile_pairs_capped). */
int ssr_tile_order(const int32_t* tile_offsets, uint32_t n_tiles, int64_t n_isects, int32_t* order, void* scratch,
                   size_t scratch_bytes, ssr_stream_t stream);
/* Number of key bits the sort must cover: 32 + tile_n_bits (IntersectTile.cu:489-490). */
int ssr_sort_end_bit(uint32_t n_tiles);
/* The sort of IntersectTile.cu:486-493 and the offsets of :271-307 in one call, for keys of the
 * form (tile << 32) | depth_bits with tile < n_tiles: partitions by tile (stable, tile bits only),
 * writes tile_offsets, then sorts every tile's range on the depth bits with one workgroup per
 * tile. Result (in the buffer pair *selector names) and tile_offsets are bit-identical to
 * ssr_sort_pairs_u64_i32 on bits [0, ssr_sort_end_bit(n_tiles)) followed by ssr_tile_offsets.
 * The other buffer pair is used as working space. */
size_t ssr_sort_tile_scratch_bytes(int64_t n, uint32_t n_tiles);
int ssr_sort_tile_pairs(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b,
                        int64_t n, uint32_t n_tiles, int32_t* tile_offsets, int* selector,
                        void* scratch, size_t scratch_bytes, ssr_stream_t stream);
/* The same over arrays of `capacity` entries of which the first *n_isects (device; clamped to capacity) are
 * keys, as ssr_tile_write_capped leaves them. tile_offsets holds n_tiles + 1 entries; tile_offsets[n_tiles]
 * receives that number, the end of the last tile. The first tile_offsets[n_tiles] entries of the result and
 * tile_offsets[0..n_tiles) are those of ssr_sort_tile_pairs on the keys; the entries behind them are unspecified.
 * Launches are sized for `capacity`; workgroups behind the count leave at once.
 * Scratch: ssr_sort_tile_scratch_bytes(capacity, n_tiles). No counterpart in the reference. */
int ssr_sort_tile_pairs_capped(int64_t* keys_a, int64_t* keys_b, int32_t* vals_a, int32_t* vals_b,
                               int64_t capacity, const int64_t* n_isects, uint32_t n_tiles, int32_t* tile_offsets,
                               int* selector, void* scratch, size_t scratch_bytes, ssr_stream_t stream);
/* ssr_tile_offsets over the first *n_isects (device) of `capacity` sorted keys, with the one entry more:
 * offsets[n_tiles] = min(*n_isects, capacity). */
int ssr_tile_offsets_capped(int64_t capacity, const int64_t* n_isects, const int64_t* sorted_ids, uint32_t n_tiles,
                            int32_t* offsets, ssr_stream_t stream);

/* ---- K7: rasterize_to_pixels_3dgs_fwd (src/kernels/raster/RasterizationFwd.cuh:18-38, kernel
 * src/kernels/raster/RasterizationEval3DFwd_kernel.cuh:48-313, IS_EVAL3D=0). */
typedef struct {
    int64_t num_splats;
    ssr_screen screen;          /* read */
    uint32_t width, height;
    const int32_t* tile_offsets;  /* [tile_h,tile_w] */
    const int32_t* flatten_ids;   /* [n_isects] */
    int64_t n_isects;
    float* render_rgb;      /* [H,W,3] */
    float* render_depth;    /* [H,W] */
    float* render_T;        /* [H,W] */
    int32_t* last_ids;      /* [H,W] */
    const float* packed_rows; /* optional: rows written by ssr_projection_fwd for this screen;
                                 when given, `screen` is not read */
    /* Variants (RasterizationEval3DFwd_kernel.cuh:143-148,245-307). dist_type SSR_DIST_D / _RGB_D:
     * the depth channel is composited as ln(max(z, 1e-6)) and rendered as exp(mean), and the
     * distortion image D = W S - C^2 (W = 1 - T, C / S first / second moments of the weights) is
     * written for depth (and rgb). render_median non-NULL: depth where the post-splat
     * transmittance crosses 1/2, interpolated in ln T; 0 where it never does. */
    int32_t dist_type;          /* SSR_DIST_* */
    float* distortion_rgb;      /* [H,W,3], RGB_D */
    float* distortion_depth;    /* [H,W], D and RGB_D */
    float* render_median;       /* optional [H,W] */
    /* Images rendered by one launch (0 counts as 1). Image c owns tiles [c T, (c+1) T) of
     * tile_offsets (T = tiles of one image) and pixels [c H W, (c+1) H W) of every per-pixel
     * buffer; the splat rows stay global, as the reference's [C,N,...] layout has them
     * (RasterizationFwd.cu grid = {C, tile_h, tile_w}). */
    int32_t num_images;
    const int32_t* tile_order;  /* optional: ssr_tile_order's output for these tile_offsets; NULL = tiles in index order, one contiguous band per XCD */
    int32_t tile_offsets_closed; /* nonzero: tile_offsets holds one more entry, the end of the last tile (ssr_sort_tile_pairs_capped); n_isects is then only the capacity of flatten_ids */
    /* Optional [n_isects]: receives, for every sorted entry the forward stages, the 4x4-pixel blocks of its tile that the
     * fragment can reach (bit 4 * sub_tile + quadrant; the reference's sub-tile test of RasterizationEval3DFwd_kernel.cuh:
     * 203-209 and the block tests under it). The backward takes them from here (its block_masks field) instead of
     * repeating the tests. Entries of batches the forward never reached (every pixel of the tile finished before them)
     * are not written; the backward never reads them, since they lie behind every last_id. No counterpart in the
     * reference. */
    uint16_t* block_masks;
} ssr_raster_fwd_params;
int ssr_raster_fwd(const ssr_raster_fwd_params* p, ssr_stream_t stream);

/* ---- K8: rasterize_to_pixels_3dgs_bwd (src/kernels/raster/RasterizationBwd.cuh:18-48, kernel
 * src/kernels/raster/RasterizationEval3DBwd_kernel.cuh:48-636, IS_EVAL3D=0). Gradients are ADDED
 * into v_screen with float atomics; the caller zero-fills it first, as the reference's launcher
 * does (src/kernels/raster/RasterizationBwd.cu:143-146). */
typedef struct {
    int64_t num_splats;
    ssr_screen screen;
    uint32_t width, height;
    const int32_t* tile_offsets;
    const int32_t* flatten_ids;
    int64_t n_isects;
    const float* render_T;
    const int32_t* last_ids;
    const float* render_depth;
    const float* v_render_rgb;    /* [H,W,3] */
    const float* v_render_depth;  /* [H,W] */
    const float* v_render_T;      /* [H,W] */
    ssr_screen v_screen;          /* accumulated into */
    const float* packed_rows;     /* optional, as in ssr_raster_fwd_params */
    /* Optional [num_splats,12] (16-byte aligned, caller zero-fills): the ten gradient channels of a
     * splat as ONE row (x, y, depth, conic[3], opac, rgb[3], 2 pad) instead of five arrays, so that
     * its atomics land in one or two cache lines instead of five. When given, v_screen is not
     * written; ssr_projection_bwd / ssr_fused_projection_bwd_optimizer read the rows through their
     * own v_rows field. With accum_mode sum or avg the two spare
     * floats of a row carry that row's weight sums on their way to accum_weight; the readers ignore
     * them. No counterpart in the reference. */
    float* v_rows;
    /* Variants (RasterizationEval3DBwd_kernel.cuh:150-172,207-279,433-585). With dist_type set:
     * render_rgb and distortion_* are the forward's outputs, v_distortion_* the cotangents of the
     * distortion image. v_render_median non-NULL: cotangent of the median depth. accum_mode
     * SSR_ACCUM_*: accum_weight[w] receives max / sum over pixels of accum_weight_map[pixel] *
     * alpha * T for world row w = gaussian_ids ? gaussian_ids[row] : row; AVG adds the sum of
     * alpha * T at accum_weight[num_world + w]. The caller zero-fills accum_weight. */
    int32_t dist_type;
    const float* render_rgb;          /* [H,W,3], RGB_D */
    const float* distortion_rgb;      /* [H,W,3], RGB_D */
    const float* distortion_depth;    /* [H,W] */
    const float* v_distortion_rgb;    /* [H,W,3], RGB_D */
    const float* v_distortion_depth;  /* [H,W] */
    const float* v_render_median;     /* optional [H,W] */
    int32_t accum_mode;
    const float* accum_weight_map;    /* [H,W] */
    const int32_t* gaussian_ids;      /* optional [num_splats] (packed projection) */
    int64_t num_world;                /* rows per lane of accum_weight */
    float* accum_weight;              /* [num_world] or [2 num_world] (AVG) */
    int32_t num_images;               /* as in ssr_raster_fwd_params; with accum_mode, screen row r
                                       * adds into world row r % num_world */
    const int32_t* tile_order;        /* optional, as in ssr_raster_fwd_params */
    int32_t tile_offsets_closed;      /* as in ssr_raster_fwd_params */
    /* How the plain variant (no distortion, median or accumulation) cuts its work; the results agree to summation
     * order. ROWS: a 16-lane row takes one fragment against the sixteen pixels of a 4x4 block per step. LANES: a row
     * takes sixteen consecutive fragments of the block's list, one a lane, against four pixels each, the recursions
     * along the list as scans over the lanes. LANES is the faster cut where a splat reaches several blocks of a tile
     * (n_isects of three times the visible splats and more: 0.50 -> 0.44 ms on the 1M-splat 1080p scene) and the slower
     * one for small footprints, whose block lists are too short to fill sixteen lanes. The variants always run ROWS.
     * No counterpart in the reference. */
    int32_t schedule;                 /* SSR_BWD_SCHEDULE_* */
    /* Optional [n_isects]: the block masks ssr_raster_fwd left for these same tile_offsets / flatten_ids (its
     * block_masks field). When given the sub-tile and block tests are not repeated; the results are the same. */
    const uint16_t* block_masks;
} ssr_raster_bwd_params;
enum { SSR_BWD_SCHEDULE_ROWS = 0, SSR_BWD_SCHEDULE_LANES = 1 };
int ssr_raster_bwd(const ssr_raster_bwd_params* p, ssr_stream_t stream);

/* ---- K9: projection_3dgs_backward (src/kernels/projection/ProjectionBwd.cuh:18-46, kernel
 * src/kernels/projection/ProjectionBwd_kernel.cuh:16-130). accumulate != 0:
 * gradients are added into v_world (the reference's behaviour; caller zero-fills,
 * src/engine/EngineLoss.cpp:120-127). Over [N] rows or a visible list the add is a plain
 * read-add-write: a launch holds one camera, so one thread owns a row. Launches that share v_world
 * must be ordered on one stream (two launches on different streams race). accumulate == 0: every row of v_world is overwritten
 * (zeros for culled splats), which gives the same values with C = 1 and needs no zero-fill. */
typedef struct {
    int64_t num_splats;
    int32_t sh_degree;
    ssr_world world;
    ssr_sh_quant sh;
    ssr_camera camera;
    const float* aabb;
    ssr_screen v_screen;    /* read */
    ssr_world v_world;      /* written / accumulated */
    int32_t accumulate;
    /* Optional work list from ssr_projection_fwd: only these splats are processed. With
     * accumulate == 0 their rows are overwritten and rows of other splats are NOT touched (the
     * caller zero-fills v_world once, as the reference does). */
    const int32_t* visible_ids;
    int64_t n_visible;
    /* Packed mode (src/kernels/projection/ProjectionBwd_kernel.cuh:51-56, launcher
     * src/kernels/projection/ProjectionBwd.cu:80-84): v_screen holds num_packed rows, row i belongs
     * to splat packed_gaussian_ids[i]; aabb is not consulted and visible_ids must be NULL.
     * num_packed == 0 with the pointer set is a no-op (ProjectionBwd.cu:89-97). */
    const int32_t* packed_gaussian_ids;
    int64_t num_packed;
    const float* v_rows;    /* optional: ssr_raster_bwd's row output; when given, v_screen is not read */
    /* Optional gradient of the camera pose (the reference's v_viewmats, ProjectionBwd_kernel.cuh:89-127): 16
     * floats laid out like the row-major [R|t] view matrix; the sums over all processed splats of dL/dR (rows
     * 0..2, columns 0..2) and dL/dt (column 3) are ADDED to it (caller zero-fills), the last row is not touched.
     * Both the projection and the SH view direction contribute. Computed by a second pass over the splats. */
    float* v_viewmat;
    /* The antialiased ("mip") variant of the primitive (src/shaders/primitive_3dgs.slang:528-543, the runtime
     * `antialiased` argument of the same projection function): screen-space blur 0.1 instead of 0.3 and the opacity
     * multiplied by sqrt(det cov2d / det (cov2d + blur)); everything after the projection is unchanged. */
    int32_t antialiased;
    /* Packed mode with accumulate != 0: non-zero declares that packed_gaussian_ids names no splat twice
     * (the rows of ONE camera), which lets the launch add with a plain read-add-write. Zero (the
     * default) adds atomically, as the reference does, so that lists holding several cameras' rows
     * stay correct. Store mode (accumulate == 0) always needs unique ids. */
    int32_t packed_ids_unique;
    /* Packed mode, optional [4][packed_world_stride][4]: the planes ssr_projection_packed_emit wrote into world_rows
     * for these same packed rows (entry i of each plane = packed row i; packed_world_stride = its
     * world_rows_stride). The parameters of row i are then read from here, not from `world` at
     * packed_gaussian_ids[i] (the SH coefficients still are): the caller vouches that `world` has not changed
     * since that projection. 16-byte aligned. */
    const float* packed_world_rows;
    int64_t packed_world_stride;
} ssr_projection_bwd_params;
int ssr_projection_bwd(const ssr_projection_bwd_params* p, ssr_stream_t stream);

/* ---- K9 fused with the optimizer step: fused_projection_bwd_optimizer_3dgs
 * (src/kernels/optim/FusedProjectionBwdOptim.cuh:18-62; kernel
 * src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:146-1030, the fp32-state branch). One pass
 * over ALL num_splats splats: the projection VJP of the visible ones (aabb test as in K9) is kept in
 * registers, the per-splat regularizer gradients are added, and Adam (beta1 0.9, beta2 0.999,
 * eps 1e-15, bias-corrected) updates the six parameter arrays and both moment sets in place --
 * the 236 B/splat gradient round trip through HBM disappears. Quaternions take the Riemannian
 * step (gradient projected on the tangent of the unit sphere, result re-normalised). Splats that
 * are not visible still decay their moments, as in the reference.
 * Built: fp32 parameters and moments, one camera, non-packed and packed (aabb and v_screen holding
 * the nnz compacted rows of the packed projection; the reference sorts the rows by splat and walks a
 * per-splat range, FusedProjectionBwdOptim.cu:160-212 -- with one camera a splat has at most one
 * row, found through packed_row_of), regularizers mcmc_opacity, mcmc_scale, scale ratio, effective
 * rank, quaternion norm and SH/DC magnitude; the scale-agnostic step of the means; the quantized SH
 * state, the quantized moments of the non-SH tensors and the colour trust region (below). */
typedef struct {
    int64_t num_splats;
    int32_t sh_degree;
    ssr_world world;            /* parameters, updated in place; features_sh fp32 */
    ssr_camera camera;
    const float* aabb;          /* [N,4] of the forward */
    ssr_screen v_screen;        /* read: output of ssr_raster_bwd */
    const float* v_rows;        /* optional: ssr_raster_bwd's row output; when given, v_screen is not read */
    ssr_world v_world_in;       /* optional gradient contributions already accumulated (any member may
                                   be NULL = zero; features_sh is not read, as in the reference) */
    ssr_world g1, g2;           /* Adam first / second moments, same shapes as world, updated in place */
    float* densify_score;       /* optional [N]: exp(max log-scale) * |dL/dmean| */
    float lr_means, lr_quats, lr_scales, lr_opacs, lr_features_dc, lr_features_sh;
    float max_gauss_ratio, scale_regularization_weight;
    float mcmc_opacity_reg_weight, mcmc_scale_reg_weight, quat_norm_reg_weight, sh_reg_weight;
    int32_t step;               /* Adam step (>= 1) when `steps` is NULL */
    const int32_t* steps;       /* optional per-splat step [N] */
    float erank_reg_weight, erank_reg_weight_s3;   /* effective-rank regularizer of the scales */
    const float* scale_agnostic_radii;   /* optional [N] apparent radii of the forward (its `radii` output): when
                                            given, the means take the scale-agnostic step
                                            (use_scale_agnostic_mean, FusedProjectionBwdOptim_kernel.cuh:519-534) */
    const int32_t* packed_row_of;   /* packed mode: [N], row of aabb / v_screen / v_rows that belongs to
                                       splat g, or -1 (ssr_packed_row_map); NULL = row g */
    /* Quantized SH state, the reference's quantization level 1 (QUANT_BITS 8, VALUE_BITS 16;
     * FusedProjectionBwdOptim_kernel.cuh:709-1030, codecs src/core/Tensor.h:936-1133,1300-1405): when
     * sh_state_packed is given, the SH coefficients live in sh_value_packed (16-bit codes, one (min,max)
     * per block of 256 splats) and their Adam moments in sh_state_packed (u, log_s bytes, one float4 of
     * bounds per block), num_sh_buffer coefficients per splat in both; world / g1 / g2 .features_sh are
     * then not used. All four arrays are updated in place; all-zero state arrays are the zero moments. */
    uint16_t* sh_state_packed;      /* [N * 3 * num_sh_buffer] */
    float* sh_state_bounds;         /* float4[ceil(N / 256)] */
    uint16_t* sh_value_packed;      /* [N * 3 * num_sh_buffer] */
    float* sh_value_bounds;         /* float2[ceil(N / 256)] */
    uint32_t num_sh_buffer;
    /* Quantized Adam state of the five non-SH tensors (NonShQuantState, 16-bit codec;
     * FusedProjectionBwdOptim_kernel.cuh:97-143,373-638), which the reference turns on together with the
     * quantized SH state: per parameter one 32-bit cell (u code | log_s code << 16), per tensor one float4
     * of bounds per block of 256 splats, in the order means, quats, log_scales, opacity_logits, features_dc.
     * All ten given (then the matching members of g1 / g2 are not used) or all NULL; all-zero arrays are
     * the zero moments. The parameters themselves stay fp32. */
    uint32_t* non_sh_packed[5];     /* [N * 3], [N * 4], [N * 3], [N], [N * 3] */
    float* non_sh_bounds[5];        /* float4[ceil(N / 256)] each */
    /* Colour trust region of the linear-colour preset (color_trust_linear, eps_tr;
     * FusedProjectionBwdOptim_kernel.cuh:551-596,651-705,774-794): the DC colour steps in the space of
     * splat_dc_encode with its gradient divided by the slope of the sRGB curve at the DC colour and the step
     * clipped to kSh0 sqrt(2 eps_tr / opacity); the SH gradients are divided by the same slopes and their steps
     * clipped to kSh0 sqrt(4 eps_tr colour / opacity) per channel. */
    int32_t color_trust_linear;
    float eps_tr;
    /* The antialiased ("mip") variant of the primitive (src/shaders/primitive_3dgs.slang:528-543, the runtime
     * `antialiased` argument of the same projection function): screen-space blur 0.1 instead of 0.3 and the opacity
     * multiplied by sqrt(det cov2d / det (cov2d + blur)); everything after the projection is unchanged. */
    int32_t antialiased;
    /* Optional [N, v_sh_in_stride] fp32: gradient contributions to the higher-order SH coefficients that are already
     * there, added to this camera's before the step (coefficient k of splat g at g * v_sh_in_stride + k). This is how
     * a camera batch is summed: the other cameras' projection backward adds into v_world_in and v_sh_in first
     * (the reference sums the cameras inside its kernel, FusedProjectionBwdOptim_kernel.cuh:262-330). */
    const float* v_sh_in;
    int32_t v_sh_in_stride;
} ssr_fpbo_params;
int ssr_fused_projection_bwd_optimizer(const ssr_fpbo_params* p, ssr_stream_t stream);
/* row_of[g] = i where gaussian_ids[i] == g, -1 for splats without a packed row (one camera, so ids
 * are unique); the per-splat lookup the packed mode above needs (FusedProjectionBwdOptim.cu:160-212
 * builds the multi-camera form of it with a sort). */
int ssr_packed_row_map(const int32_t* gaussian_ids, int64_t nnz, int64_t num_splats, int32_t* row_of,
                       ssr_stream_t stream);

/* Zeroes the gradient rows of the listed splats only (the rows a previous ssr_projection_bwd run
 * over that list wrote), instead of refilling all N rows. No counterpart in the reference, which
 * always refills (src/engine/EngineLoss.cpp:120-127).
 * Rows that an ssr_projection_bwd in store mode is about to overwrite can be left alone, named either way:
 * skip_visible_aabb (optional, [N,4]): splats whose aabb is non-empty;
 * skip_sorted_ids (optional, n_skip ascending splat ids, e.g. one camera's packed gaussian_ids): splats in
 * that list, found by bisection. */
int ssr_zero_world_rows(const ssr_world* v_world, const int32_t* ids, int64_t n,
                        const float* skip_visible_aabb, const int32_t* skip_sorted_ids, int64_t n_skip,
                        ssr_stream_t stream);

/* ---- K10 and runtime (src/backend/api/BackendRuntime.h:29-168). */
int ssr_fill_u32(void* dst, uint32_t value, int64_t count, ssr_stream_t stream);
int ssr_init(int device);                       /* select the device, warm the context */
int ssr_device_count(void);
const char* ssr_device_name(void);
void* ssr_device_malloc(size_t bytes);          /* 0 bytes -> NULL; failure -> NULL */
int ssr_device_free(void* ptr);                 /* drains in-flight work first */
void* ssr_host_malloc_pinned(size_t bytes);
int ssr_host_free_pinned(void* ptr);
int ssr_memcpy(void* dst, const void* src, size_t bytes, int kind, ssr_stream_t stream, int async);
int ssr_memset(void* dst, int byte_value, size_t bytes, ssr_stream_t stream, int async);
int ssr_is_device_pointer(const void* ptr);     /* pinned host memory is NOT a device pointer */
int ssr_device_synchronize(void);
int ssr_stream_synchronize(ssr_stream_t stream);
ssr_stream_t ssr_stream_create(void);
int ssr_stream_destroy(ssr_stream_t stream);
ssr_event_t ssr_event_create(void);
int ssr_event_record(ssr_event_t ev, ssr_stream_t stream);
int ssr_event_synchronize(ssr_event_t ev);
int ssr_event_elapsed_ms(ssr_event_t start, ssr_event_t stop, float* ms);
int ssr_event_destroy(ssr_event_t ev);
const char* ssr_last_error(void);               /* returns and clears; "" when none */

/* Diagnostics: include/ssr_math.h evaluated on the device (op: 0 exp, 1 log, 2 atan2(a,b),
 * 3 sigmoid, 4 / 5 Adam's inverse bias correction for beta1 / beta2 at step a), to check that host
 * and device produce identical bits. */
int ssr_debug_math(int op, int64_t n, const float* a, const float* b, float* out,
                   ssr_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* SSR_BACKEND_H */
