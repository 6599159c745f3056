// projection.hip -- K1 (projection + SH colour, optional fused tile count) and K9 (their VJP).
//
// K1 follows projection_fused_fwd_kernel (src/kernels/projection/ProjectionFwd_kernel.cuh:17-111)
// with World::project (src/primitives/Primitive3DGS.cuh:56-110). K9 follows
// projection_fused_bwd_kernel (src/kernels/projection/ProjectionBwd_kernel.cuh:16-130) with
// World::project_vjp (src/primitives/Primitive3DGS.cuh:119-201); the projection VJP is written out
// by hand with the conventions of the reference's generated derivative
// (src/generated/primitive_3dgs.cuh:12782-13230): a clamped Jacobian entry sends its gradient to
// the violated bound, v_conic enters as [[vx, vy],[0, vz]], normalize(quat) and length() are
// differentiated, extents / sorting depth / radius carry no gradient.
//
// One thread per Gaussian, 256 threads (4 wavefronts) per workgroup. Both kernels are bound by
// HBM traffic (236 B in, 60 B out per visible splat forward; 472 B in/out backward).
#include <math.h>
#include <type_traits>
#include <string.h>

#include "projection_device.h"
#include "../../include/ssr_quant.h"
#include "../../include/ssr_colour.h"
#include "raster_device.h"

namespace ssr {

constexpr int kProjBlock = 256;

__device__ __forceinline__ void load_splat(const ssr_world& w, int64_t g, float mean[3], float quat[4],
                                           float ls[3], float& logit) {
    const float* m = w.means + 3 * g;
    mean[0] = m[0]; mean[1] = m[1]; mean[2] = m[2];
    const float4 q = *reinterpret_cast<const float4*>(w.quats + 4 * g);
    quat[0] = q.x; quat[1] = q.y; quat[2] = q.z; quat[3] = q.w;
    const float* s = w.log_scales + 3 * g;
    ls[0] = s[0]; ls[1] = s[1]; ls[2] = s[2];
    logit = w.opacity_logits[g];
}

// atomicMax for non-negative floats through the integer ordering (src/core/Common.cuh:785-789)
__device__ __forceinline__ void atomic_max_nonneg(float* p, float v) {
    atomicMax(reinterpret_cast<int*>(p), __float_as_int(v));
}

template <int kDegree>
__device__ __forceinline__ void sh_colour(const ssr_world& W, const ssr_sh_quant& Q, const CamD& cam, int64_t g,
                                          float* rgb_row, float* packed_row, const float* mean_in = nullptr,
                                          float* dc_out = nullptr);

// Two phases per workgroup of 256 splats. Phase 1: every thread projects its splat (44 B in) and
// writes aabb / sorting depth / geometry row / tile count; splats that stay visible are appended
// to a list in LDS. Phase 2: the first n_visible threads evaluate SH colour (192 B in) for the
// listed splats, so the expensive part runs on dense wavefronts however sparse visibility is.
// (Running phase 2 as a kernel of its own over the global list was measured and is slower in every
// configuration, sparse or dense.)
template <int kDegree, bool kLens>
__global__ __launch_bounds__(kProjBlock) void projection_fwd_kernel(ssr_projection_fwd_params P) {
    __shared__ int s_list[kProjBlock];
    __shared__ int s_count;
    __shared__ long long s_base;
    if (threadIdx.x == 0) s_count = 0;
    if (P.clear_count && blockIdx.x == 0 && threadIdx.x == 0) *P.clear_count = 0;
    __syncthreads();
    const int64_t block0 = (int64_t)blockIdx.x * kProjBlock;
    const int64_t g = block0 + threadIdx.x;
    CamD cam = load_camera(P.camera);
    cam.aa = P.antialiased != 0;
    if (g < P.num_splats) {
        float mean[3], quat[4], ls[3], logit;
        load_splat(P.world, g, mean, quat, ls, logit);
        ProjD p;
        project<false, kLens>(cam, mean, quat, ls, logit, p);
        float bb[4] = {p.aabb[0], p.aabb[1], p.aabb[2], p.aabb[3]};
        bb[0] = ssr_min(ssr_max(bb[0], 0.0f), cam.Wf - 1.0f);
        bb[1] = ssr_min(ssr_max(bb[1], 0.0f), cam.Hf - 1.0f);
        bb[2] = ssr_min(ssr_max(bb[2], 0.0f), cam.Wf - 1.0f);
        bb[3] = ssr_min(ssr_max(bb[3], 0.0f), cam.Hf - 1.0f);
        float4* aabb_out = reinterpret_cast<float4*>(P.aabb);
        // a clamped extent > 1e-3 implies the unclamped aabb is non-empty, which is the reference's
        // condition for evaluating the colour (src/primitives/Primitive3DGS.cuh:74)
        if (bb[2] - bb[0] > 1e-3f && bb[3] - bb[1] > 1e-3f) {
            *reinterpret_cast<float2*>(P.screen.xy + 2 * g) = make_float2(p.xy[0], p.xy[1]);
            P.screen.depth[g] = p.depth;
            float* cn = P.screen.conic + 3 * g;
            cn[0] = p.conic[0]; cn[1] = p.conic[1]; cn[2] = p.conic[2];
            P.screen.opac[g] = p.opac;
            aabb_out[g] = make_float4(bb[0], bb[1], bb[2], bb[3]);
            P.sort_depth[g] = p.sort_depth;
            // stored: what the integer-ordered maximum with a zero leaves (a negative bit pattern loses to the zero)
            if (P.radii_store) P.radii[g] = __float_as_int(p.radius) > 0 ? p.radius : 0.0f;
            else atomic_max_nonneg(P.radii + g, p.radius);
            if (P.tiles_per_splat) {
                const int tw = (int)((P.camera.width + kTile - 1) / kTile), th = (int)((P.camera.height + kTile - 1) / kTile);
                TileGeomD tg;
                tile_geom(bb, p.xy, p.conic, p.opac, tw, th, tg);
                P.tiles_per_splat[g] = count_tiles(tg);
            }
            if (P.packed_rows) {   // geometry part of the row; phase 2 adds the colour
                float cut, kk;
                fragment_constants(p.opac, cut, kk);
                float4* row = reinterpret_cast<float4*>(P.packed_rows) + 3 * g;
                row[0] = make_float4(p.xy[0], p.xy[1], 0.5f * p.conic[0], p.conic[1]);
                *reinterpret_cast<float2*>(&row[1]) = make_float2(0.5f * p.conic[2], p.opac);
                float* r2 = reinterpret_cast<float*>(&row[2]);
                r2[1] = p.depth; r2[2] = cut; r2[3] = kk;
            }
            s_list[atomicAdd(&s_count, 1)] = threadIdx.x;
        } else {
            aabb_out[g] = make_float4(0.f, 0.f, 0.f, 0.f);
            P.sort_depth[g] = 0.0f;
            if (P.tiles_per_splat) P.tiles_per_splat[g] = 0;
            if (P.radii_store) P.radii[g] = 0.0f;
        }
    }
    __syncthreads();
    const int n_vis = s_count;
    if (P.visible_ids) {
        if (threadIdx.x == 0 && n_vis > 0)
            s_base = (long long)atomicAdd(reinterpret_cast<unsigned long long*>(P.visible_count), (unsigned long long)n_vis);
        __syncthreads();
        if ((int)threadIdx.x < n_vis) P.visible_ids[s_base + threadIdx.x] = (int32_t)(block0 + s_list[threadIdx.x]);
    }
    if ((int)threadIdx.x >= n_vis) return;
    const int64_t v = block0 + s_list[threadIdx.x];
    sh_colour<kDegree>(P.world, P.sh, cam, v, P.screen.rgb + 3 * v,
                       P.packed_rows ? P.packed_rows + kPackedRowFloats * v : nullptr);
}

// SH colour of one visible splat g: max(0.5 + sum_j Y_j c_j, 0) (src/shaders/harmonics.slang:1055-1066),
// written to rgb_row[0..2] and, when given, to the colour slots of its 48-byte fragment row.
template <int kDegree>
// mean_in: the splat's mean where the caller holds it already; dc_out: receives the DC colour coefficients
__device__ __forceinline__ void sh_colour(const ssr_world& W, const ssr_sh_quant& Q, const CamD& cam, int64_t g,
                                          float* rgb_row, float* packed_row, const float* mean_in, float* dc_out) {
    const float* mp = mean_in ? mean_in : W.means + 3 * g;
    const float mean[3] = {mp[0], mp[1], mp[2]};
    constexpr int kCoef = kDegree * (kDegree + 2);
    float coef[kCoef > 0 ? 3 * kCoef : 1];
    if (kCoef > 0) decode_sh<kCoef>(W, Q, g, coef);
    float dir[3];
    view_dir(cam, mean, dir);
    ShBasisD b;
    sh_basis<kDegree>(dir, b);
    const float* dcp = W.features_dc + 3 * g;
    const float dc[3] = {dcp[0], dcp[1], dcp[2]};
    if (dc_out) { dc_out[0] = dc[0]; dc_out[1] = dc[1]; dc_out[2] = dc[2]; }
    float raw[3];
    sh_color_raw<kDegree>(b, dc, coef, raw);
    float col[3];
#pragma unroll
    for (int c = 0; c < 3; c++) { col[c] = ssr_max(raw[c] + 0.5f, 0.0f); rgb_row[c] = col[c]; }
    if (packed_row) {
        *reinterpret_cast<float2*>(packed_row + 6) = make_float2(col[0], col[1]);
        packed_row[8] = col[2];
    }
}

// ---- packed form -------------------------------------------------------------------------------
// Staging area of the packed projection inside the caller's scratch buffer: per-workgroup visible
// counts, their exclusive scan, and the geometry of the visible splats compacted within each
// workgroup's own segment of kPackSeg rows (structure of arrays, so both passes access it coalesced).
constexpr int kPackPer = 4;                       // splats per thread of the mask kernel
constexpr int kPackSeg = kProjBlock * kPackPer;   // splats per workgroup of the mask kernel = rows of its segment
struct PackedStage {
    int32_t* block_counts;    // [nb]
    int64_t* block_offsets;   // [nb + 1], block_offsets[nb] = nnz
    float4* aabb;             // [N]
    float2* xy;               // [N]
    float* conic;             // [3][N], component-major
    float* sort_depth;        // [N]
    float* depth;             // [N]
    float* opac;              // [N]
    int32_t* gid;             // [N]
    float4* world;            // optional [3][N]: (mean, logit), quat, (log_scale, 0) of the staged rows
};

__host__ __device__ inline size_t align16(size_t b) { return (b + 15) & ~(size_t)15; }

inline size_t packed_stage_layout(int64_t n, void* base, PackedStage* st, bool with_world = false) {
    const size_t nb = (size_t)ceil_div(n, kPackSeg), N = (size_t)n;
    char* p = static_cast<char*>(base);
    size_t off = 0;
    auto take = [&](size_t bytes) { char* r = p ? p + off : nullptr; off += align16(bytes); return r; };
    char* a0 = take(N * 16); char* a1 = take(N * 8); char* a2 = take(N * 12); char* a3 = take(N * 4);
    char* a4 = take(N * 4); char* a5 = take(N * 4); char* a6 = take(N * 4);
    char* a7 = take((nb + 1) * 8); char* a8 = take(nb * 4);
    char* a9 = with_world ? take(N * 48) : nullptr;   // last, so that the layout without it is a prefix
    if (st) {
        st->world = reinterpret_cast<float4*>(a9);
        st->aabb = reinterpret_cast<float4*>(a0); st->xy = reinterpret_cast<float2*>(a1);
        st->conic = reinterpret_cast<float*>(a2); st->sort_depth = reinterpret_cast<float*>(a3);
        st->depth = reinterpret_cast<float*>(a4); st->opac = reinterpret_cast<float*>(a5);
        st->gid = reinterpret_cast<int32_t*>(a6); st->block_offsets = reinterpret_cast<int64_t*>(a7);
        st->block_counts = reinterpret_cast<int32_t*>(a8);
    }
    return off;
}

// Pass 1 of the packed projection (projection_packed_mask_kernel,
// src/kernels/projection/ProjectionPackedFwd_kernel.cuh:17-94): the visibility rule is the clamped
// aabb extent test. Unlike the reference, which keeps only the mask and projects again later, the
// projected geometry of the visible splats is kept: compacted in splat order within the
// workgroup's segment of the staging area (ballot ranks inside a wavefront, wavefront totals through
// LDS), so that the second pass never touches a culled splat.
// A pinhole view is sparse when the camera stands inside the scene, and this kernel is bound by the projection's
// arithmetic, not by memory: so a first pass over the workgroup's 1024 splats, four per thread, reads only the
// mean and the scales and rejects what is certainly behind the camera or off the image; the rest are listed in
// splat order and projected 256 at a time, on dense wavefronts. The test is one-sided: z <= 0 is the
// projection's own rule on the identically computed z; the screen radius is bounded by
// 3.33 sqrt(s_max^2 |J row|^2 + blur) with |J row|^2 <= (f^2 + L^2) / z^2, L the clamp of J[.][2]
// (clamp_pinhole_jacobian), enlarged by 1 % and a pixel, so whatever is rejected here the projection's
// off-image test rejects as well; anything unordered (NaN) is kept.
__device__ __forceinline__ bool pinhole_may_be_visible(const CamD& cam, const ssr_world& W, int64_t g) {
    const float* m = W.means + 3 * g;
    const float mean[3] = {m[0], m[1], m[2]};
    float mc[3];
#pragma unroll
    for (int i = 0; i < 3; i++)
        mc[i] = ((cam.R[i][0] * mean[0] + cam.R[i][1] * mean[1]) + cam.R[i][2] * mean[2]) + cam.t[i];
    const float z = mc[2];
    if (z <= 0.0f) return false;
    const float* sc = W.log_scales + 3 * g;
    const float smax = __builtin_amdgcn_exp2f(ssr_max(sc[0], ssr_max(sc[1], sc[2])) * 1.44269504f) * 1.001f;   // hardware exp2, an ulp off at most
    const float lim_pos = cam.Wf + 0.3f * (0.5f * cam.Wf), lim_neg = 0.3f * (0.5f * cam.Wf);
    const float Lx = ssr_max(lim_pos - cam.cx, lim_neg + cam.cx), Ly = ssr_max(lim_pos - cam.cy, lim_neg + cam.cy);
    // hardware reciprocal and square root (an ulp off): the 1 % and the pixel cover them
    const float rz = __builtin_amdgcn_rcpf(z), sz = smax * rz;
    const float Rx = 3.33f * 1.01f * __builtin_amdgcn_sqrtf((sz * sz) * (cam.fx * cam.fx + Lx * Lx) + 0.3f) + 1.0f;
    const float Ry = 3.33f * 1.01f * __builtin_amdgcn_sqrtf((sz * sz) * (cam.fy * cam.fy + Ly * Ly) + 0.3f) + 1.0f;
    const float u = cam.fx * (mc[0] * rz) + cam.cx, v = cam.fy * (mc[1] * rz) + cam.cy;
    return !(u + Rx < 0.0f || u - Rx > cam.Wf || v + Ry < 0.0f || v - Ry > cam.Hf);
}

template <bool kLens>
__global__ __launch_bounds__(kProjBlock) void projection_packed_mask_kernel(ssr_projection_packed_params P, PackedStage S) {
    __shared__ int s_pre[kPackPer * (kProjBlock / 64)];   // candidates per (slice, wavefront)
    __shared__ uint16_t s_cand[kPackSeg];                 // the candidates' offsets in the segment, in splat order
    __shared__ int s_wave[2][kProjBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t block0 = (int64_t)blockIdx.x * kPackSeg;
    const int n_here = (int)min((int64_t)kPackSeg, P.num_splats - block0);
    CamD cam = load_camera(P.camera);
    cam.aa = P.antialiased != 0;
    const bool pretest = !kLens && cam.model == SSR_CAM_PINHOLE;
    // 1. candidates: slice k of the segment is splats k * 256 .. k * 256 + 255, one per thread
    unsigned long long km[kPackPer];
#pragma unroll
    for (int k = 0; k < kPackPer; k++) {
        const int off = k * kProjBlock + (int)threadIdx.x;
        const bool keep = off < n_here && (!pretest || pinhole_may_be_visible(cam, P.world, block0 + off));
        km[k] = __ballot(keep);
        if (lane == 0) s_pre[k * (kProjBlock / 64) + wave] = __popcll(km[k]);
    }
    __syncthreads();
    int n_cand = 0;
#pragma unroll
    for (int k = 0; k < kPackPer; k++) {
        int before = n_cand;   // the slices before this one
#pragma unroll
        for (int w = 0; w < kProjBlock / 64; w++) {
            const int c = s_pre[k * (kProjBlock / 64) + w];
            if (w < wave) before += c;
            n_cand += c;
        }
        if ((km[k] >> lane) & 1ull)
            s_cand[before + __popcll(km[k] & ((1ull << lane) - 1ull))] = (uint16_t)(k * kProjBlock + (int)threadIdx.x);
    }
    __syncthreads();
    // 2. the projection, 256 candidates a round; rounds and ranks keep the splat order
    const int64_t N = P.num_splats;
    int n_out = 0;
    for (int c0 = 0; c0 < n_cand; c0 += kProjBlock) {
        const int c = c0 + (int)threadIdx.x;
        bool vis = false;
        ProjD p;
        float bb[4] = {0.f, 0.f, 0.f, 0.f};
        int64_t g = 0;
        float mean[3], quat[4], ls[3], logit;
        if (c < n_cand) {
            g = block0 + s_cand[c];
            load_splat(P.world, g, mean, quat, ls, logit);
            project<false, kLens>(cam, mean, quat, ls, logit, p);
            bb[0] = ssr_min(ssr_max(p.aabb[0], 0.0f), cam.Wf - 1.0f);
            bb[1] = ssr_min(ssr_max(p.aabb[1], 0.0f), cam.Hf - 1.0f);
            bb[2] = ssr_min(ssr_max(p.aabb[2], 0.0f), cam.Wf - 1.0f);
            bb[3] = ssr_min(ssr_max(p.aabb[3], 0.0f), cam.Hf - 1.0f);
            vis = bb[2] - bb[0] > 1e-3f && bb[3] - bb[1] > 1e-3f;   // ProjectionPackedFwd_kernel.cuh:93
        }
        const unsigned long long m = __ballot(vis);
        const int rank = __popcll(m & ((1ull << lane) - 1ull));
        int* totals = s_wave[(c0 / kProjBlock) & 1];   // two sets in turn: one barrier a round is enough
        if (lane == 0) totals[wave] = __popcll(m);
        __syncthreads();
        int base = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kProjBlock / 64; w++) { if (w < wave) base += totals[w]; total += totals[w]; }
        if (vis) {
            const int64_t d = block0 + n_out + base + rank;
            S.aabb[d] = make_float4(bb[0], bb[1], bb[2], bb[3]);
            S.xy[d] = make_float2(p.xy[0], p.xy[1]);
            S.conic[d] = p.conic[0]; S.conic[N + d] = p.conic[1]; S.conic[2 * N + d] = p.conic[2];
            S.sort_depth[d] = p.sort_depth;
            S.depth[d] = p.depth;
            S.opac[d] = p.opac;
            S.gid[d] = (int32_t)g;
            if (S.world) {
                S.world[d] = make_float4(mean[0], mean[1], mean[2], logit);
                S.world[N + d] = make_float4(quat[0], quat[1], quat[2], quat[3]);
                S.world[2 * N + d] = make_float4(ls[0], ls[1], ls[2], 0.0f);
            }
            atomic_max_nonneg(P.radii + g, p.radius);   // ProjectionPackedFwd_kernel.cuh:183
        }
        n_out += total;
    }
    if (threadIdx.x == 0) S.block_counts[blockIdx.x] = n_out;
}

// Exclusive scan of the workgroup counts by ONE workgroup (the counts are N/256 values, 39k for ten million
// splats; one workgroup saves two launches). It walks the counts in tiles of 4096: every thread holds four
// consecutive values, a wavefront scans its 256 with shuffles, the sixteen wavefront totals are scanned by
// each thread from LDS, and a running total carries from tile to tile. The next tile's loads are issued
// before the current tile is scanned.
constexpr int kScanOneBlock = 1024;
__global__ __launch_bounds__(kScanOneBlock) void packed_block_scan_kernel(const int32_t* __restrict__ counts, int64_t nb,
                                                                          int64_t* __restrict__ offsets, int64_t* __restrict__ nnz) {
    __shared__ int s_wave[2][kScanOneBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int kPer = 4;
    auto load_run = [&](int64_t base, int v[kPer]) {
#pragma unroll
        for (int k = 0; k < kPer; k++) v[k] = base + k < nb ? counts[base + k] : 0;
    };
    long long carry = 0;
    int cur[kPer], nxt[kPer];
    load_run((int64_t)threadIdx.x * kPer, cur);
    int parity = 0;
    for (int64_t tile0 = 0; tile0 < nb; tile0 += kPer * kScanOneBlock, parity ^= 1) {
        const int64_t base = tile0 + (int64_t)threadIdx.x * kPer;
        load_run(base + kPer * kScanOneBlock, nxt);
        int mine = 0;
#pragma unroll
        for (int k = 0; k < kPer; k++) mine += cur[k];
        int incl = mine;   // inclusive scan over the wavefront
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d, 64);
            if (lane >= d) incl += up;
        }
        if (lane == 63) s_wave[parity][wave] = incl;
        __syncthreads();
        int before = 0, total = 0;
#pragma unroll
        for (int w = 0; w < kScanOneBlock / 64; w++) {
            const int t = s_wave[parity][w];
            if (w < wave) before += t;
            total += t;
        }
        long long acc = carry + before + (incl - mine);
#pragma unroll
        for (int k = 0; k < kPer; k++) {
            if (base + k < nb) offsets[base + k] = acc;
            acc += cur[k];
        }
        carry += total;
#pragma unroll
        for (int k = 0; k < kPer; k++) cur[k] = nxt[k];
    }
    if (threadIdx.x == 0) { offsets[nb] = carry; *nnz = carry; }
}

// Pass 2 (projection_packed_fwd_kernel, ProjectionPackedFwd_kernel.cuh:97-184): one thread per
// OUTPUT row j < nnz. The source workgroup of row j is found by bisection over the scanned
// offsets: two searches with uniform arguments bracket the workgroups this 256-row span touches, a
// short per-thread search finishes inside the bracket.
__device__ __forceinline__ int64_t last_block_at_or_before(const int64_t* __restrict__ off, int64_t nb, int64_t j) {
    int64_t lo = 0, hi = nb;   // invariant: off[lo] <= j < off[hi]
    while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (off[mid] <= j) lo = mid; else hi = mid;
    }
    return lo;
}

template <int kDegree>
__global__ __launch_bounds__(kProjBlock) void projection_packed_emit_kernel(ssr_projection_packed_params P, PackedStage S) {
    const int64_t nnz = *P.nnz < P.max_rows ? *P.nnz : P.max_rows;
    const int64_t j0 = (int64_t)blockIdx.x * kProjBlock;
    if (j0 >= nnz) return;
    const int64_t nb = (P.num_splats + kPackSeg - 1) / kPackSeg;
    const int64_t j1 = j0 + kProjBlock - 1 < nnz - 1 ? j0 + kProjBlock - 1 : nnz - 1;
    int64_t lo = last_block_at_or_before(S.block_offsets, nb, j0);
    int64_t hi = last_block_at_or_before(S.block_offsets, nb, j1) + 1;
    const int64_t j = j0 + threadIdx.x;
    if (j >= nnz) return;
    while (hi - lo > 1) {
        const int64_t mid = (lo + hi) >> 1;
        if (S.block_offsets[mid] <= j) lo = mid; else hi = mid;
    }
    const int64_t src = lo * kPackSeg + (j - S.block_offsets[lo]);
    const int64_t N = P.num_splats;
    CamD cam = load_camera(P.camera);
    cam.aa = P.antialiased != 0;
    const float4 bb4 = S.aabb[src];
    const float2 xy = S.xy[src];
    const float conic[3] = {S.conic[src], S.conic[N + src], S.conic[2 * N + src]};
    const float opac = S.opac[src], depth = S.depth[src];
    const int32_t g = S.gid[src];
    P.camera_ids[j] = P.camera_index;
    P.gaussian_ids[j] = g;
    reinterpret_cast<float4*>(P.aabb)[j] = bb4;
    P.sort_depth[j] = S.sort_depth[src];
    *reinterpret_cast<float2*>(P.screen.xy + 2 * j) = xy;
    P.screen.depth[j] = depth;
    float* cn = P.screen.conic + 3 * j;
    cn[0] = conic[0]; cn[1] = conic[1]; cn[2] = conic[2];
    P.screen.opac[j] = opac;
    if (P.tiles_per_splat) {
        const int tw = (int)((P.camera.width + kTile - 1) / kTile), th = (int)((P.camera.height + kTile - 1) / kTile);
        const float bb[4] = {bb4.x, bb4.y, bb4.z, bb4.w};
        const float c2[2] = {xy.x, xy.y};
        TileGeomD tg;
        tile_geom(bb, c2, conic, opac, tw, th, tg);
        P.tiles_per_splat[j] = count_tiles(tg);
    }
    float* prow = nullptr;
    if (P.packed_rows) {
        float cut, kk;
        fragment_constants(opac, cut, kk);
        prow = P.packed_rows + kPackedRowFloats * j;
        float4* row = reinterpret_cast<float4*>(prow);
        row[0] = make_float4(xy.x, xy.y, 0.5f * conic[0], conic[1]);
        *reinterpret_cast<float2*>(&row[1]) = make_float2(0.5f * conic[2], opac);
        prow[9] = depth; prow[10] = cut; prow[11] = kk;
    }
    if (P.world_rows) {   // the splat's parameters, plane by plane, for the projection backward
        const float4 w0 = S.world[src], w2 = S.world[2 * N + src];
        const float mean[3] = {w0.x, w0.y, w0.z};
        float dc[3];
        sh_colour<kDegree>(P.world, P.sh, cam, g, P.screen.rgb + 3 * j, prow, mean, dc);
        float4* wr = reinterpret_cast<float4*>(P.world_rows) + j;
        const int64_t plane = P.world_rows_stride;
        wr[0] = w0;
        wr[plane] = S.world[N + src];
        wr[2 * plane] = make_float4(w2.x, w2.y, w2.z, dc[0]);
        wr[3 * plane] = make_float4(dc[1], dc[2], 0.0f, 0.0f);
        return;
    }
    sh_colour<kDegree>(P.world, P.sh, cam, g, P.screen.rgb + 3 * j, prow);
}

__device__ __forceinline__ float fin(float v) { return ssr_isfinite(v) ? v : 0.0f; }

// How K9 leaves a value in the world gradients. kPutStore overwrites; kPutAdd is a plain
// read-add-write, valid when exactly one thread of the launch owns the row (one camera and, in packed
// mode, no splat id listed twice) -- the sum is the same float an atomic would give; kPutAtomic is the
// reference's atomic add (its launch covers C cameras at once), used when rows may repeat.
enum { kPutStore = 0, kPutAdd = 1, kPutAtomic = 2 };
template <int kMode>
__device__ __forceinline__ void put(float* p, float v) {
    if (kMode == kPutStore) *p = v;
    else if (v != 0.0f) { if (kMode == kPutAtomic) atomicAdd(p, v); else *p += v; }
}

// Gradient of one splat's screen row with respect to its world row (everything K9 computes before
// it stores): g is the splat's row in `W`, r its row in `VS`. sh_sink(j, Yj, vc) receives the two
// factors of the gradient of SH coefficient j (j < kDegree (kDegree + 2)), which is Yj * vc[0..2].
struct WorldGradD { float mean[3], quat[4], scale[3], logit, dc[3]; };

// Where the screen-space gradient of row r lives: five arrays (the reference's layout) or one
// 12-float row per splat (x, y, depth, conic[3], opac, rgb[3], pad[2]) written by the compositing backward.
struct VScreenD {
    const float *xy, *depth, *conic, *opac, *rgb;
    int s_xy, s_depth, s_conic, s_opac, s_rgb;   // floats between consecutive rows
};
__device__ __forceinline__ VScreenD vscreen_of(const ssr_screen& s, const float* rows) {
    if (rows) return VScreenD{rows, rows + 2, rows + 3, rows + 6, rows + 7, 12, 12, 12, 12, 12};
    return VScreenD{s.xy, s.depth, s.conic, s.opac, s.rgb, 2, 1, 3, 1, 3};
}

// dL/dR and dL/dt of the world-to-camera transform, one splat's share
struct PoseGradD { float R[3][3], t[3]; };

template <int kDegree, bool kLens, bool kPose = false, bool kShFirst = false, class ShSink>
__device__ __forceinline__ void projection_vjp(const CamD& cam, const ssr_world& W, const ssr_sh_quant& Q, int64_t g,
                                               const VScreenD& VS, int64_t r, WorldGradD& out, ShSink&& sh_sink,
                                               PoseGradD* pose = nullptr, const float* world_row = nullptr,
                                               int64_t world_plane = 0) {
    constexpr int kCoef = kDegree * (kDegree + 2);
    float mean[3], quat[4], ls[3], logit;
    float dc[3];
    if (world_row) {   // what ssr_projection_packed_emit left: the same values, four coalesced reads
        const float4* wr = reinterpret_cast<const float4*>(world_row);
        const float4 a = wr[0], b = wr[world_plane], c = wr[2 * world_plane], d = wr[3 * world_plane];
        mean[0] = a.x; mean[1] = a.y; mean[2] = a.z; logit = a.w;
        quat[0] = b.x; quat[1] = b.y; quat[2] = b.z; quat[3] = b.w;
        ls[0] = c.x; ls[1] = c.y; ls[2] = c.z;
        dc[0] = c.w; dc[1] = d.x; dc[2] = d.y;
    } else {
        load_splat(W, g, mean, quat, ls, logit);
    }
    float vc[3] = {0.f, 0.f, 0.f};
    float vdir[3] = {0.f, 0.f, 0.f};
    // (kShFirst: ahead of the geometry, whose live values then do not overlap the 45 coefficients)
    auto sh_part = [&]() {
        // SH colour VJP (src/shaders/harmonics.slang:373-649,1087-1126)
        float coef[kCoef > 0 ? 3 * kCoef : 1];
        if (kCoef > 0) decode_sh<kCoef>(W, Q, g, coef);
        float dir[3];
        view_dir(cam, mean, dir);
        ShBasisD b;
        sh_basis<kDegree>(dir, b);
        if (!world_row) {
            const float* dcp = W.features_dc + 3 * g;
            dc[0] = dcp[0]; dc[1] = dcp[1]; dc[2] = dcp[2];
        }
        float raw[3];
        sh_color_raw<kDegree>(b, dc, coef, raw);
        const float* vrg = VS.rgb + VS.s_rgb * r;
    #pragma unroll
        for (int c = 0; c < 3; c++) vc[c] = vrg[c] * (raw[c] >= -0.5f ? 1.0f : 0.0f);
        if (kDegree >= 1) {
    #pragma unroll
            for (int j = 0; j < kCoef; j++) {
                sh_sink(j, b.Y[j], vc);
            }
            // gY(j) = dL/dY_j. With Y(l, +-m) = A(z) {Re, Im} w^m, w = x + i y, and d w^m = m w^(m-1) dw:
            //   dL/dx += m A (g_c Re w^(m-1) + g_s Im w^(m-1)),  dL/dy += m A (g_s Re w^(m-1) - g_c Im w^(m-1)),
            //   dL/dz += A'(z) (g_c Re w^m + g_s Im w^m);        zonal terms B(z) add B'(z) g to dL/dz only.
            auto gY = [&](int j) { return (coef[3 * j] * vc[0] + coef[3 * j + 1] * vc[1]) + coef[3 * j + 2] * vc[2]; };
            const float X = b.x, Y = b.y, Z = b.z;
            float vx = 0.0f, vy = 0.0f, vz = 0.0f;
            auto order = [&](int m, float A, float dA, float gc, float gs) {
                const float mA = (float)m * A;
                vx += mA * (gc * b.re[m - 1] + gs * b.im[m - 1]);
                vy += mA * (gs * b.re[m - 1] - gc * b.im[m - 1]);
                vz += dA * (gc * b.re[m] + gs * b.im[m]);
            };
            order(1, -shk::k1, 0.0f, gY(2), gY(0));
            vz += shk::k1 * gY(1);
            if (kDegree >= 2) {
                order(2, shk::k22, 0.0f, gY(7), gY(3));
                order(1, -shk::k21 * Z, -shk::k21, gY(6), gY(4));
                vz += (2.0f * shk::k20a * Z) * gY(5);
                if (kDegree >= 3) {
                    const float zz = Z * Z;
                    order(3, -shk::k33, 0.0f, gY(14), gY(8));
                    order(2, shk::k32 * Z, shk::k32, gY(13), gY(9));
                    order(1, shk::k31b - shk::k31a * zz, -2.0f * shk::k31a * Z, gY(12), gY(10));
                    vz += (3.0f * shk::k30a * zz - shk::k30b) * gY(11);
                }
            }
            const float dn = (vx * X + vy * Y) + vz * Z;
            vdir[0] = (vx - dn * X) * b.inorm;
            vdir[1] = (vy - dn * Y) * b.inorm;
            vdir[2] = (vz - dn * Z) * b.inorm;
        }
    };
    if constexpr (kShFirst) sh_part();
    ProjD p;
    project<true, kLens>(cam, mean, quat, ls, logit, p);
    const float x = p.mc[0], y = p.mc[1], z = p.mc[2];
    float vmc[3] = {0.f, 0.f, 0.f};
    // conic = inverse(cov2d)
    const float c00 = p.c2[0][0], c01 = p.c2[0][1], c10 = p.c2[1][0], c11 = p.c2[1][1];
    const float det = c00 * c11 - c01 * c10, inv = 1.0f / det;
    const float* vcn = VS.conic + VS.s_conic * r;
    const float g00 = vcn[0], g01 = vcn[1], g11 = vcn[2];
    const float v_inv = (c11 * g00 - c01 * g01) + c00 * g11;
    const float v_det = -(v_inv / (det * det));
    float vC[2][2];
    vC[0][0] = inv * g11 + c11 * v_det;
    vC[1][1] = inv * g00 + c00 * v_det;
    vC[0][1] = -(inv * g01) - c10 * v_det;
    vC[1][0] = -(c01 * v_det);
    if (cam.aa) {
        // opacity = sigmoid(logit) * sqrt(max(0, det_orig / det_blur)): the gradient of the opacity reaches the 2D
        // covariance through both determinants (sqrt derivative guarded at 1e-7, max(0, .) passes where positive)
        const float ratio = p.det_orig / p.det_blur;
        const float v_comp = VS.opac[VS.s_opac * r] * p.sig;
        const float v_ratio = ratio > 0.0f ? v_comp * (0.5f / ssr_sqrt(ssr_max(1e-7f, ratio))) : 0.0f;
        const float v_do = v_ratio / p.det_blur;
        const float v_db = -((v_ratio * p.det_orig) / (p.det_blur * p.det_blur));
        vC[0][0] += v_do * p.c2o[1] + v_db * c11;
        vC[1][1] += v_do * p.c2o[0] + v_db * c00;
        vC[0][1] += (v_do + v_db) * (-c10);
        vC[1][0] += (v_do + v_db) * (-c01);
    }
    // cov2d = J covc J^T
    float vJ[2][3], vS[3][3];
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int k = 0; k < 3; k++) {
            float s = 0.0f;
#pragma unroll
            for (int j = 0; j < 2; j++)
#pragma unroll
                for (int l = 0; l < 3; l++)
                    s += vC[i][j] * p.J[j][l] * p.covc[k][l] + vC[j][i] * p.J[j][l] * p.covc[l][k];
            vJ[i][k] = s;
        }
#pragma unroll
    for (int k = 0; k < 3; k++)
#pragma unroll
        for (int l = 0; l < 3; l++) {
            float s = 0.0f;
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) s += p.J[i][k] * vC[i][j] * p.J[j][l];
            vS[k][l] = s;
        }
    const float vm0 = VS.xy[VS.s_xy * r], vm1 = VS.xy[VS.s_xy * r + 1];
    if (kLens) {
        // uv, J and dJ/dp of the model from one second-order evaluation: v_p = J^T v_uv + sum_ij v_J[i][j] dJ[i][j]/dp.
        // A clamped J[i][2] of the perspective camera is a function of z alone (its bound).
        typedef SsrJet<3, 2> Jet;
        Jet px, py;
        ssr_model_pixel<Jet>(cam.model, cam.tier, cam.dc, cam.fx, cam.fy, cam.cx, cam.cy, ssr_jet_seed<3, 2>(x, 0),
                             ssr_jet_seed<3, 2>(y, 1), ssr_jet_seed<3, 2>(z, 2), px, py);
        const float iz2 = 1.0f / (z * z);
        const float lim_pos = cam.Wf + 0.3f * (0.5f * cam.Wf), lim_neg = 0.3f * (0.5f * cam.Wf);
        const float bound_lo[2] = {-(lim_pos - cam.cx), -(lim_pos - cam.cy)}, bound_hi[2] = {lim_neg + cam.cx, lim_neg + cam.cy};
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const Jet& f = i == 0 ? px : py;
            const float vm = i == 0 ? vm0 : vm1;
#pragma unroll
            for (int k = 0; k < 3; k++) vmc[k] += vm * f.d[k];
#pragma unroll
            for (int j = 0; j < 3; j++) {
                if (j == 2 && p.clamp_lo[i]) { vmc[2] += vJ[i][2] * bound_lo[i] * (-iz2); continue; }
                if (j == 2 && p.clamp_hi[i]) { vmc[2] += vJ[i][2] * bound_hi[i] * (-iz2); continue; }
#pragma unroll
                for (int k = 0; k < 3; k++) vmc[k] += vJ[i][j] * f.h[j <= k ? ssr_jet_idx<3>(j, k) : ssr_jet_idx<3>(k, j)];
            }
        }
    } else if (cam.model == SSR_CAM_PINHOLE) {
        const float z2 = z * z, iz = 1.0f / z, iz2 = 1.0f / z2;
        vmc[2] += vJ[0][0] * (-cam.fx * iz2) + vJ[1][1] * (-cam.fy * iz2);
        const float lim_pos = cam.Wf + 0.3f * (0.5f * cam.Wf), lim_neg = 0.3f * (0.5f * cam.Wf);
        const float cmaxx = lim_neg + cam.cx, cminx = -(lim_pos - cam.cx);
        const float cmaxy = lim_neg + cam.cy, cminy = -(lim_pos - cam.cy);
        if (p.clamp_lo[0]) vmc[2] += vJ[0][2] * cminx * (-iz2);
        else if (p.clamp_hi[0]) vmc[2] += vJ[0][2] * cmaxx * (-iz2);
        else { vmc[0] += vJ[0][2] * (-cam.fx * iz2); vmc[2] += vJ[0][2] * (2.0f * cam.fx * x * iz2 * iz); }
        if (p.clamp_lo[1]) vmc[2] += vJ[1][2] * cminy * (-iz2);
        else if (p.clamp_hi[1]) vmc[2] += vJ[1][2] * cmaxy * (-iz2);
        else { vmc[1] += vJ[1][2] * (-cam.fy * iz2); vmc[2] += vJ[1][2] * (2.0f * cam.fy * y * iz2 * iz); }
        vmc[0] += vm0 * cam.fx * iz;
        vmc[1] += vm1 * cam.fy * iz;
        vmc[2] += -(vm0 * cam.fx * x + vm1 * cam.fy * y) * iz2;
    } else {
        const float h2 = x * x + z * z, h = ssr_sqrt(h2), r2 = h2 + y * y;
        const float A = 1.0f / h2, B = 1.0f / (h * r2);
        const float dAx = -2.0f * x * A * A, dAz = -2.0f * z * A * A;
        const float dBx = -B * B * (x * r2 / h + 2.0f * x * h);
        const float dBy = -B * B * (2.0f * y * h);
        const float dBz = -B * B * (z * r2 / h + 2.0f * z * h);
        const float fx = cam.fx, fy = cam.fy;
        const float ir2 = 1.0f / r2, ir4 = ir2 * ir2;
        vmc[0] += vJ[0][0] * fx * z * dAx + vJ[0][2] * (-fx) * (A + x * dAx);
        vmc[2] += vJ[0][0] * fx * (A + z * dAz) + vJ[0][2] * (-fx) * x * dAz;
        vmc[0] += vJ[1][0] * (-fy) * (y * B + x * y * dBx) + vJ[1][2] * (-fy) * (z * y * dBx) +
                  vJ[1][1] * fy * ((x / h) * ir2 - h * 2.0f * x * ir4);
        vmc[1] += vJ[1][0] * (-fy) * (x * B + x * y * dBy) + vJ[1][2] * (-fy) * (z * B + z * y * dBy) +
                  vJ[1][1] * fy * (-h * 2.0f * y * ir4);
        vmc[2] += vJ[1][0] * (-fy) * (x * y * dBz) + vJ[1][2] * (-fy) * (y * B + z * y * dBz) +
                  vJ[1][1] * fy * ((z / h) * ir2 - h * 2.0f * z * ir4);
        vmc[0] += vm0 * fx * z * A + vm1 * fy * (-(x * y) * B);
        vmc[1] += vm1 * fy * h * ir2;
        vmc[2] += vm0 * fx * (-x * A) + vm1 * fy * (-(z * y) * B);
    }
    {   // depth = length(mean_c); the sqrt derivative is guarded at 1e-7
        const float s2 = dot3(p.mc, p.mc);
        const float vs = VS.depth[VS.s_depth * r] * (0.5f / ssr_sqrt(ssr_max(1e-7f, s2)));
#pragma unroll
        for (int i = 0; i < 3; i++) vmc[i] += 2.0f * p.mc[i] * vs;
    }
    float vmean[3];
#pragma unroll
    for (int i = 0; i < 3; i++) vmean[i] = (cam.R[0][i] * vmc[0] + cam.R[1][i] * vmc[1]) + cam.R[2][i] * vmc[2];
    float t1[3][3], vcov[3][3], vM[3][3];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            t1[i][j] = (cam.R[0][i] * vS[0][j] + cam.R[1][i] * vS[1][j]) + cam.R[2][i] * vS[2][j];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++)
            vcov[i][j] = (t1[i][0] * cam.R[0][j] + t1[i][1] * cam.R[1][j]) + t1[i][2] * cam.R[2][j];
#pragma unroll
    for (int i = 0; i < 3; i++)
#pragma unroll
        for (int j = 0; j < 3; j++) {
            float s = 0.0f;
#pragma unroll
            for (int k = 0; k < 3; k++) s += (vcov[i][k] + vcov[k][i]) * p.M[k][j];
            vM[i][j] = s;
        }
    float vRq[3][3], vscale[3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
        float s = 0.0f;
#pragma unroll
        for (int i = 0; i < 3; i++) { vRq[i][j] = vM[i][j] * p.s[j]; s += vM[i][j] * p.Rq[i][j]; }
        vscale[j] = s * p.s[j];
    }
    const float qw = p.qn[0], qx = p.qn[1], qy = p.qn[2], qz = p.qn[3];
    float vqn[4];
    vqn[0] = 2.0f * (qx * (vRq[2][1] - vRq[1][2]) + qy * (vRq[0][2] - vRq[2][0]) + qz * (vRq[1][0] - vRq[0][1]));
    vqn[1] = 2.0f * (-2.0f * qx * (vRq[1][1] + vRq[2][2]) + qy * (vRq[0][1] + vRq[1][0]) +
                     qz * (vRq[0][2] + vRq[2][0]) + qw * (vRq[2][1] - vRq[1][2]));
    vqn[2] = 2.0f * (-2.0f * qy * (vRq[0][0] + vRq[2][2]) + qx * (vRq[0][1] + vRq[1][0]) +
                     qz * (vRq[1][2] + vRq[2][1]) + qw * (vRq[0][2] - vRq[2][0]));
    vqn[3] = 2.0f * (-2.0f * qz * (vRq[0][0] + vRq[1][1]) + qx * (vRq[0][2] + vRq[2][0]) +
                     qy * (vRq[1][2] + vRq[2][1]) + qw * (vRq[1][0] - vRq[0][1]));
    const float qd = ((p.qn[0] * vqn[0] + p.qn[1] * vqn[1]) + p.qn[2] * vqn[2]) + p.qn[3] * vqn[3];
    float vquat[4];
#pragma unroll
    for (int i = 0; i < 4; i++) vquat[i] = (vqn[i] - p.qn[i] * qd) * p.qinv;
    const float vlogit = (VS.opac[VS.s_opac * r] * p.comp) * (p.sig * (1.0f - p.sig));

    if constexpr (!kShFirst) sh_part();
#pragma unroll
    for (int i = 0; i < 3; i++) { out.mean[i] = vmean[i] + vdir[i]; out.scale[i] = vscale[i]; out.dc[i] = 0.2820947917738781f * vc[i]; }
#pragma unroll
    for (int i = 0; i < 4; i++) out.quat[i] = vquat[i];
    out.logit = vlogit;
    if (kPose) {
        // mean_c = R mean + t, cov_c = R cov R^T (cov = M M^T), view direction = mean + R^T t
        // (src/shaders/primitive_3dgs.slang:434-436, src/shaders/harmonics.slang:145-149):
        //   dL/dt = v_mean_c + R v_dir,   dL/dR = v_mean_c mean^T + (v_cov_c + v_cov_c^T) R cov + t v_dir^T
        float cov[3][3], RS[3][3];
#pragma unroll
        for (int a = 0; a < 3; a++)
#pragma unroll
            for (int j = 0; j < 3; j++) cov[a][j] = (p.M[a][0] * p.M[j][0] + p.M[a][1] * p.M[j][1]) + p.M[a][2] * p.M[j][2];
#pragma unroll
        for (int k = 0; k < 3; k++)
#pragma unroll
            for (int j = 0; j < 3; j++) RS[k][j] = (cam.R[k][0] * cov[0][j] + cam.R[k][1] * cov[1][j]) + cam.R[k][2] * cov[2][j];
#pragma unroll
        for (int i = 0; i < 3; i++) {
            pose->t[i] = vmc[i] + ((cam.R[i][0] * vdir[0] + cam.R[i][1] * vdir[1]) + cam.R[i][2] * vdir[2]);
#pragma unroll
            for (int j = 0; j < 3; j++) {
                float s = vmc[i] * mean[j] + cam.t[i] * vdir[j];
#pragma unroll
                for (int k = 0; k < 3; k++) s += (vS[i][k] + vS[k][i]) * RS[k][j];
                pose->R[i][j] = s;
            }
        }
    }
}

template <int kDegree, int kPut, bool kLens>
__global__ __launch_bounds__(kProjBlock) void projection_bwd_kernel(ssr_projection_bwd_params P) {
    constexpr bool kAccumulate = kPut != kPutStore;
    const int64_t i = (int64_t)blockIdx.x * kProjBlock + threadIdx.x;
    if (i >= (P.packed_gaussian_ids ? P.num_packed : (P.visible_ids ? P.n_visible : P.num_splats))) return;
    // g: row of the splat in world / v_world; r: its row in v_screen (ProjectionBwd_kernel.cuh:51-63)
    const int64_t g = P.packed_gaussian_ids ? (int64_t)P.packed_gaussian_ids[i] : (P.visible_ids ? (int64_t)P.visible_ids[i] : i);
    const int64_t r = P.packed_gaussian_ids ? i : g;
    constexpr int kCoef = kDegree * (kDegree + 2);
    float4 bb = make_float4(0.f, 0.f, 1.f, 1.f);
    if (!P.packed_gaussian_ids) bb = reinterpret_cast<const float4*>(P.aabb)[g];
    ssr_world& V = P.v_world;
    if (bb.z <= bb.x || bb.w <= bb.y) {   // ProjectionBwd_kernel.cuh:58
        if (!kAccumulate && !P.visible_ids) {
#pragma unroll
            for (int i = 0; i < 3; i++) { V.means[3 * g + i] = 0.f; V.log_scales[3 * g + i] = 0.f; V.features_dc[3 * g + i] = 0.f; }
            *reinterpret_cast<float4*>(V.quats + 4 * g) = make_float4(0.f, 0.f, 0.f, 0.f);
            V.opacity_logits[g] = 0.f;
            float* vs = V.features_sh + g * (int64_t)V.sh_stride;
            for (int i = 0; i < V.sh_stride; i++) vs[i] = 0.f;
        }
        return;
    }
    CamD cam = load_camera(P.camera);
    cam.aa = P.antialiased != 0;
    WorldGradD wg;
    float* vsh = V.features_sh + g * (int64_t)V.sh_stride;
    projection_vjp<kDegree, kLens>(cam, P.world, P.sh, g, vscreen_of(P.v_screen, P.v_rows), r, wg, [&](int j, float Yj, const float vc[3]) {
        const float tv[3] = {Yj * vc[0], Yj * vc[1], Yj * vc[2]};
        const float d2 = dot3(tv, tv);
        const bool ok = ssr_isfinite(d2) && d2 != 0.0f;   // harmonics.slang:397-403
#pragma unroll
        for (int c = 0; c < 3; c++) {
            put<kPut>(vsh + 3 * j + c, ok ? tv[c] : 0.0f);
        }
    }, nullptr, P.packed_world_rows ? P.packed_world_rows + 4 * r : nullptr, P.packed_world_stride);
    if (!kAccumulate) {   // coefficients above the active degree receive nothing
        for (int i = 3 * kCoef; i < V.sh_stride; i++) vsh[i] = 0.0f;
    }
    // World::atomicStore (src/primitives/PrimitiveBase3DGS.cuh:75-83): per-component finite filter
#pragma unroll
    for (int i = 0; i < 3; i++) put<kPut>(V.means + 3 * g + i, fin(wg.mean[i]));
#pragma unroll
    for (int i = 0; i < 4; i++) put<kPut>(V.quats + 4 * g + i, fin(wg.quat[i]));
#pragma unroll
    for (int i = 0; i < 3; i++) put<kPut>(V.log_scales + 3 * g + i, fin(wg.scale[i]));
    put<kPut>(V.opacity_logits + g, fin(wg.logit));
#pragma unroll
    for (int i = 0; i < 3; i++) put<kPut>(V.features_dc + 3 * g + i, fin(wg.dc[i]));
}

// The degree-3 kernel with the SH gradient rows staged through LDS. A thread writing its own 180-byte row in
// fifteen 12-byte pieces makes every store instruction of a wavefront touch 64 rows (90 cache lines for 768
// bytes), and those partial-line writes, not the reads and not HBM, are what the kernel above waits for (the
// texture-address unit 70 % busy, counted; staging the coefficient reads the same way made things slower).
// Here every lane leaves its row in the wavefront's own 11.25 KB of LDS and the wavefront moves its 64 rows as one
// run: sixteen-byte pieces in address order when the rows are consecutive (no work list), else 12-byte pieces
// row after row through the lanes' row numbers. LDS operations of one wavefront execute in order, so no barrier
// is involved. kPut: store or plain add (the atomic mode keeps the kernel above).
constexpr int kShRow = 45;
// piece e of a wavefront's 64 * 15 twelve-byte pieces lies in row e / 15 (the multiply-shift is exact below 960)
__device__ __forceinline__ int sh_piece_row(int e) { return (int)(((uint32_t)e * 34953u) >> 19); }

template <int kPut, bool kLens>
__global__ __launch_bounds__(kProjBlock) void projection_bwd_staged_kernel(ssr_projection_bwd_params P) {
    static_assert(kPut == kPutStore || kPut == kPutAdd, "atomic adds go element by element");
    __shared__ __attribute__((aligned(16))) float s_sh[kProjBlock / 64][64 * kShRow];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float* my = s_sh[wave];
    const int64_t n_rows = P.packed_gaussian_ids ? P.num_packed : (P.visible_ids ? P.n_visible : P.num_splats);
    const int64_t i0 = (int64_t)blockIdx.x * kProjBlock + wave * 64;   // the wavefront's first work item
    if (i0 >= n_rows) return;
    const int64_t i = i0 + lane;
    const bool in_range = i < n_rows;
    const bool listed = P.packed_gaussian_ids || P.visible_ids;
    const int64_t g = !in_range ? 0 : (P.packed_gaussian_ids ? (int64_t)P.packed_gaussian_ids[i] : (P.visible_ids ? (int64_t)P.visible_ids[i] : i));
    const int64_t r = P.packed_gaussian_ids ? i : g;
    float4 bb = make_float4(0.f, 0.f, 1.f, 1.f);
    if (in_range && !P.packed_gaussian_ids) bb = reinterpret_cast<const float4*>(P.aabb)[g];
    const bool valid = in_range && !(bb.z <= bb.x || bb.w <= bb.y);
    ssr_world& V = P.v_world;
    float* __restrict__ dst = V.features_sh;

    // one splat per lane; its SH gradient row goes to LDS
    float* mine = my + lane * kShRow;
    WorldGradD wg;
    if (valid) {
        CamD cam = load_camera(P.camera);
        cam.aa = P.antialiased != 0;
        projection_vjp<3, kLens, false, true>(cam, P.world, P.sh, g, vscreen_of(P.v_screen, P.v_rows), r, wg, [&](int j, float Yj, const float vc[3]) {
            const float tv[3] = {Yj * vc[0], Yj * vc[1], Yj * vc[2]};
            const float d2 = dot3(tv, tv);
            const bool ok = ssr_isfinite(d2) && d2 != 0.0f;   // harmonics.slang:397-403
#pragma unroll
            for (int c = 0; c < 3; c++) mine[3 * j + c] = ok ? tv[c] : 0.0f;
        }, nullptr, P.packed_world_rows ? P.packed_world_rows + 4 * r : nullptr, P.packed_world_stride);
    } else if (!listed) {
        for (int k = 0; k < kShRow; k++) mine[k] = 0.0f;   // a culled row of a run that is written whole
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();

    // LDS -> the wavefront's gradient rows
    if (!listed) {
        const int count = (int)min((int64_t)64, n_rows - i0);   // rows of this wavefront
        float4* __restrict__ d4 = reinterpret_cast<float4*>(dst + i0 * kShRow);
        const int n4 = (count * kShRow) >> 2;   // whole pieces; at most three floats remain (a last, short wavefront)
#pragma unroll
        for (int t = 0; t < (64 * kShRow / 4 + 63) / 64; t++) {
            const int e = t * 64 + lane;
            if (e < n4) {
                float4 v = reinterpret_cast<const float4*>(my)[e];
                if (kPut == kPutAdd) { const float4 o = d4[e]; v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w; }
                d4[e] = v;
            }
        }
        if (lane < count * kShRow - 4 * n4) {
            float* q = dst + i0 * kShRow + 4 * n4 + lane;
            const float v = my[4 * n4 + lane];
            *q = kPut == kPutAdd ? *q + v : v;
        }
    } else {
        const int gl = valid ? (int)g : -1;
#pragma unroll
        for (int t = 0; t < kShRow / 3; t++) {
            const int e = t * 64 + lane;
            const int row = sh_piece_row(e), c3 = e - row * 15;
            const int gr = __shfl(gl, row, 64);
            if (gr >= 0) {
                float* q = dst + (int64_t)gr * kShRow + 3 * c3;
                const float* d = my + row * kShRow + 3 * c3;
                if (kPut == kPutAdd) { q[0] += d[0]; q[1] += d[1]; q[2] += d[2]; }
                else { q[0] = d[0]; q[1] = d[1]; q[2] = d[2]; }
            }
        }
    }
    // the other fourteen gradients, as in the kernel above
    if (!valid) {
        if (kPut == kPutStore && !listed && in_range) {
#pragma unroll
            for (int k = 0; k < 3; k++) { V.means[3 * g + k] = 0.f; V.log_scales[3 * g + k] = 0.f; V.features_dc[3 * g + k] = 0.f; }
            *reinterpret_cast<float4*>(V.quats + 4 * g) = make_float4(0.f, 0.f, 0.f, 0.f);
            V.opacity_logits[g] = 0.f;
        }
        return;
    }
#pragma unroll
    for (int k = 0; k < 3; k++) put<kPut>(V.means + 3 * g + k, fin(wg.mean[k]));
#pragma unroll
    for (int k = 0; k < 4; k++) put<kPut>(V.quats + 4 * g + k, fin(wg.quat[k]));
#pragma unroll
    for (int k = 0; k < 3; k++) put<kPut>(V.log_scales + 3 * g + k, fin(wg.scale[k]));
    put<kPut>(V.opacity_logits + g, fin(wg.logit));
#pragma unroll
    for (int k = 0; k < 3; k++) put<kPut>(V.features_dc + 3 * g + k, fin(wg.dc[k]));
}

// Camera-pose gradient: the same VJP once more, keeping only dL/dR and dL/dt, summed over the workgroup and added
// to the 16-float view-matrix gradient with one atomic per entry and workgroup (the reference sums per warp,
// ProjectionBwd_kernel.cuh:108-127).
template <int kDegree, bool kLens>
__global__ __launch_bounds__(kProjBlock) void projection_pose_bwd_kernel(ssr_projection_bwd_params P) {
    __shared__ float s_part[kProjBlock / 64][12];
    const int64_t i = (int64_t)blockIdx.x * kProjBlock + threadIdx.x;
    const int64_t n_rows = P.packed_gaussian_ids ? P.num_packed : (P.visible_ids ? P.n_visible : P.num_splats);
    float v[12];
#pragma unroll
    for (int k = 0; k < 12; k++) v[k] = 0.f;
    if (i < n_rows) {
        const int64_t g = P.packed_gaussian_ids ? (int64_t)P.packed_gaussian_ids[i] : (P.visible_ids ? (int64_t)P.visible_ids[i] : i);
        const int64_t r = P.packed_gaussian_ids ? i : g;
        float4 bb = make_float4(0.f, 0.f, 1.f, 1.f);
        if (!P.packed_gaussian_ids) bb = reinterpret_cast<const float4*>(P.aabb)[g];
        if (!(bb.z <= bb.x || bb.w <= bb.y)) {
            CamD cam = load_camera(P.camera);
    cam.aa = P.antialiased != 0;
            WorldGradD wg;
            PoseGradD pg;
            projection_vjp<kDegree, kLens, true>(cam, P.world, P.sh, g, vscreen_of(P.v_screen, P.v_rows), r, wg,
                                                 [](int, float, const float*) {}, &pg);
#pragma unroll
            for (int a = 0; a < 3; a++) {
#pragma unroll
                for (int b = 0; b < 3; b++) v[4 * a + b] = pg.R[a][b];
                v[4 * a + 3] = pg.t[a];
            }
        }
    }
#pragma unroll
    for (int k = 0; k < 12; k++) {
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) v[k] += __shfl_xor(v[k], d, 64);
        if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6][k] = v[k];
    }
    __syncthreads();
    if (threadIdx.x < 12) {
        float s = s_part[0][threadIdx.x];
#pragma unroll
        for (int w = 1; w < kProjBlock / 64; w++) s += s_part[w][threadIdx.x];
        atomicAdd(P.v_viewmat + threadIdx.x, s);
    }
}

// ---- projection backward fused with Adam ---------------------------------------------------------
struct AdamD { float b1c, b2c; };   // 1/(1-beta1^t), 1/(1-beta2^t)

// one Adam step on values: the moments are updated in place, the stepped parameter is returned
__device__ __forceinline__ float adam_core(float x, float v, float lr, const AdamD& a, float& g1, float& g2) {
    constexpr float kBeta1 = 0.9f, kBeta2 = 0.999f, kEps = 1e-15f;
    g1 = kBeta1 * g1 + (1.f - kBeta1) * v;
    g2 = kBeta2 * g2 + (1.f - kBeta2) * (v * v);
    return x - ((lr * a.b1c) * g1) / (ssr_sqrt(g2 * a.b2c) + kEps);
}
__device__ __forceinline__ float adam_step(float x, float v, float lr, const AdamD& a, float* g1p, float* g2p) {
    float g1 = *g1p, g2 = *g2p;
    const float r = adam_core(x, v, lr, a, g1, g2);
    *g1p = g1; *g2p = g2;
    return r;
}

// The five non-SH tensors in the order of the quantized non-SH state: means, quats, log_scales, opacity_logits,
// features_dc; kNsOff = first of a tensor's parameters among a splat's 14, kNsPrims = how many it has.
__device__ __forceinline__ float* non_sh_tensor(const ssr_world& w, int t) {
    return t == 0 ? w.means : t == 1 ? w.quats : t == 2 ? w.log_scales : t == 3 ? w.opacity_logits : w.features_dc;
}
__device__ __forceinline__ constexpr int ns_off(int t) { return t == 0 ? 0 : t == 1 ? 3 : t == 2 ? 7 : t == 3 ? 10 : 11; }
__device__ __forceinline__ constexpr int ns_prims(int t) { return t == 1 ? 4 : t == 3 ? 1 : 3; }

// Two phases per workgroup of 256 splats. Phase 1, one thread per splat: projection VJP in
// registers, regularizers, Adam on the 14 non-SH parameters; the SH gradient is rank one
// (Y_j * v_colour), so only its factors (15 + 3 floats) go to LDS. Phase 2, the workgroup streams
// over its 256 x 3 kCoef SH coefficients in memory order: parameter and both moments are read and
// written fully coalesced, the gradient is rebuilt from the factors in LDS.
template <int kDegree, bool kLens, bool kQuant, bool kNsq>
__global__ __launch_bounds__(kProjBlock) void fused_projection_bwd_optimizer_kernel(ssr_fpbo_params P, AdamD scalar_adam) {
    constexpr int kCoef = kDegree * (kDegree + 2);
    constexpr int kY = kCoef > 0 ? kCoef : 1;
    __shared__ float s_Y[kProjBlock][kY + 1];   // +1: odd row pitch, conflict-free column reads
    __shared__ float s_vc[kProjBlock][3];
    __shared__ float s_b1c[kProjBlock], s_b2c[kProjBlock];
    __shared__ float s_red[kProjBlock / 64][6];   // quantized state: per-wave min / max of the new bounds
    __shared__ float s_sqrt_g2[kQuant ? 256 : 1];  // quantized state: sqrt(g2) of each 8-bit log_s code under the old bounds
    __shared__ float s_ns[kNsq ? kProjBlock / 64 : 1][20];   // quantized non-SH state: per-wave (min, max) x (u, log_s) x 5 tensors
    __shared__ float s_ctl[kProjBlock][6];         // colour trust region: per splat the sRGB slope (3) and the SH step clip (3)
    const bool ctl = P.color_trust_linear != 0;
    const int64_t block0 = (int64_t)blockIdx.x * kProjBlock;
    const int64_t g = block0 + threadIdx.x;
    const ssr_world& W = P.world;
    AdamD ad = scalar_adam;
#pragma unroll
    for (int j = 0; j < kY; j++) s_Y[threadIdx.x][j] = 0.f;
    s_vc[threadIdx.x][0] = s_vc[threadIdx.x][1] = s_vc[threadIdx.x][2] = 0.f;
    // Moments of the 14 non-SH parameters: fp32 arrays, or (NonShQuantState, FusedProjectionBwdOptim_kernel.cuh:97-143,
    // 373-638) 16-bit (u, log_s) cells decoded against the block's old bounds, kept in registers after the step
    // and encoded once the block's new bounds are known.
    float ns_g1[kNsq ? 14 : 1], ns_g2[kNsq ? 14 : 1];
    float ns_mm[kNsq ? 5 : 1][4];
    if (kNsq) {
#pragma unroll
        for (int t = 0; t < 5; t++) { ns_mm[t][0] = 1e30f; ns_mm[t][1] = -1e30f; ns_mm[t][2] = 1e30f; ns_mm[t][3] = -1e30f; }
#pragma unroll
        for (int i = 0; i < 14; i++) { ns_g1[i] = 0.f; ns_g2[i] = 0.f; }
    }
    float ns_old[kNsq ? 5 : 1][4];
    if (kNsq) {
#pragma unroll
        for (int t = 0; t < 5; t++)
#pragma unroll
            for (int k = 0; k < 4; k++) ns_old[t][k] = P.non_sh_bounds[t][4 * blockIdx.x + k];
    }
    auto fetch_moments = [&](int t, int i, float& m1, float& m2) {
        if (kNsq) {
            ssr_adamq16_decode(P.non_sh_packed[t][(int64_t)ns_prims(t) * g + i], ns_old[t], &m1, &m2);
        } else {
            m1 = non_sh_tensor(P.g1, t)[(int64_t)ns_prims(t) * g + i];
            m2 = non_sh_tensor(P.g2, t)[(int64_t)ns_prims(t) * g + i];
        }
    };
    auto keep_moments = [&](int t, int i, float m1, float m2) {
        if (kNsq) {
            ns_g1[ns_off(t) + i] = m1; ns_g2[ns_off(t) + i] = m2;
            float u, ls;
            ssr_adamq_to_us(m1, m2, &u, &ls);
            ns_mm[t][0] = ssr_min(ns_mm[t][0], u); ns_mm[t][1] = ssr_max(ns_mm[t][1], u);
            ns_mm[t][2] = ssr_min(ns_mm[t][2], ls); ns_mm[t][3] = ssr_max(ns_mm[t][3], ls);
        } else {
            non_sh_tensor(P.g1, t)[(int64_t)ns_prims(t) * g + i] = m1;
            non_sh_tensor(P.g2, t)[(int64_t)ns_prims(t) * g + i] = m2;
        }
    };
    // Adam on parameter i of tensor t: returns the stepped value
    auto step_param = [&](int t, int i, float x, float v, float lr) {
        float m1, m2;
        fetch_moments(t, i, m1, m2);
        const float r = adam_core(x, v, lr, ad, m1, m2);
        keep_moments(t, i, m1, m2);
        return r;
    };
    if (g < P.num_splats) {
        if (P.steps) {   // per-splat step: beta^t = exp(t ln beta)
            const float t = (float)P.steps[g];
            ad.b1c = ssr_adam_inv_bias1(t);
            ad.b2c = ssr_adam_inv_bias2(t);
        }
        // gradient contributions that are already there (World::atomicLoad, FusedProjectionBwdOptim_kernel.cuh:250-251)
        WorldGradD wg;
        const ssr_world& VI = P.v_world_in;
#pragma unroll
        for (int i = 0; i < 3; i++) {
            wg.mean[i] = VI.means ? VI.means[3 * g + i] : 0.f;
            wg.scale[i] = VI.log_scales ? VI.log_scales[3 * g + i] : 0.f;
            wg.dc[i] = VI.features_dc ? VI.features_dc[3 * g + i] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) wg.quat[i] = VI.quats ? VI.quats[4 * g + i] : 0.f;
        wg.logit = VI.opacity_logits ? VI.opacity_logits[g] : 0.f;

        // the row that holds this splat's aabb and screen gradients: g, or its packed row (none: skipped)
        const int64_t row = P.packed_row_of ? (int64_t)P.packed_row_of[g] : g;
        float4 bb = make_float4(0.f, 0.f, 0.f, 0.f);
        if (row >= 0) bb = reinterpret_cast<const float4*>(P.aabb)[row];
        if (!(bb.z <= bb.x || bb.w <= bb.y)) {   // FusedProjectionBwdOptim_kernel.cuh:271-272
            CamD cam = load_camera(P.camera);
    cam.aa = P.antialiased != 0;
            WorldGradD pg;
            ssr_sh_quant none;
            none.codec = SSR_SH_F32; none.packed = nullptr; none.bounds = nullptr; none.bounds_stride = 0;
            none.num_sh_buffer = 0; none.scale_f16 = nullptr;
            if (kQuant) {   // the view-direction gradient is taken against the decoded 16-bit coefficients
                none.codec = SSR_SH_REF_Q16; none.packed = P.sh_value_packed; none.bounds = P.sh_value_bounds;
                none.num_sh_buffer = P.num_sh_buffer; none.bounds_stride = (int64_t)kProjBlock * 3 * P.num_sh_buffer;
            }
            projection_vjp<kDegree, kLens>(cam, W, none, g, vscreen_of(P.v_screen, P.v_rows), row, pg, [&](int j, float Yj, const float vc[3]) {
                s_Y[threadIdx.x][j] = Yj;
                if (j == 0) { s_vc[threadIdx.x][0] = vc[0]; s_vc[threadIdx.x][1] = vc[1]; s_vc[threadIdx.x][2] = vc[2]; }
            });
#pragma unroll
            for (int i = 0; i < 3; i++) { wg.mean[i] += pg.mean[i]; wg.scale[i] += pg.scale[i]; wg.dc[i] += pg.dc[i]; }
#pragma unroll
            for (int i = 0; i < 4; i++) wg.quat[i] += pg.quat[i];
            wg.logit += pg.logit;
        }
        // parameters as they were before this step
        float mean[3], quat[4], ls[3], logit;
        load_splat(W, g, mean, quat, ls, logit);
        const float* dcp = W.features_dc + 3 * g;
        const float dc[3] = {dcp[0], dcp[1], dcp[2]};

        // per-splat regularizers (src/shaders/per_splat_losses.slang:30-81, v_loss = 1)
        {
            const float sg = ssr_sigmoid(logit);
            wg.logit += P.mcmc_opacity_reg_weight * (sg * (1.0f - sg));
            const float ms = (P.mcmc_scale_reg_weight * 1e-2f) / 3.0f;
            const float e[3] = {ssr_exp(ls[0]), ssr_exp(ls[1]), ssr_exp(ls[2])};
            int imax = 0, imin = 0;
            for (int i = 1; i < 3; i++) { if (e[i] > e[imax]) imax = i; if (e[i] < e[imin]) imin = i; }
            const float ratio = e[imax] / e[imin];
            const float rg = ratio > P.max_gauss_ratio ? P.scale_regularization_weight * ratio : 0.0f;
#pragma unroll
            for (int i = 0; i < 3; i++) wg.scale[i] += ms + (i == imax ? rg : 0.f) - (i == imin ? rg : 0.f);
            if (P.erank_reg_weight != 0.0f || P.erank_reg_weight_s3 != 0.0f) {   // per_splat_losses.slang:3-15,101
                float ge[3];
                ssr_erank_reg_grad(ls, P.erank_reg_weight, P.erank_reg_weight_s3, ge);
#pragma unroll
                for (int i = 0; i < 3; i++) wg.scale[i] += ge[i];
            }
            const float qn = ssr_sqrt((quat[0] * quat[0] + quat[1] * quat[1]) + (quat[2] * quat[2] + quat[3] * quat[3]));
            const float qg = P.quat_norm_reg_weight * ((1.0f - 1.0f / qn) / qn);
#pragma unroll
            for (int i = 0; i < 4; i++) wg.quat[i] += qg * quat[i];
            const float lim = 0.5f / 0.28209479177387814f;   // FusedProjectionBwdOptim_kernel.cuh:354-357
#pragma unroll
            for (int i = 0; i < 3; i++) wg.dc[i] += P.sh_reg_weight * (ssr_max(dc[i] - lim, 0.0f) + ssr_min(dc[i] + lim, 0.0f));
        }

        // scales, quats (Riemannian), opacity, means, dc -- FusedProjectionBwdOptim_kernel.cuh:390-612
#pragma unroll
        for (int i = 0; i < 3; i++) W.log_scales[3 * g + i] = step_param(2, i, ls[i], wg.scale[i], P.lr_scales);
        {
            const float n2 = (quat[0] * quat[0] + quat[1] * quat[1]) + (quat[2] * quat[2] + quat[3] * quat[3]);
            const float inv = 1.0f / ssr_sqrt(n2);
            float q[4], v[4];
#pragma unroll
            for (int i = 0; i < 4; i++) q[i] = quat[i] * inv;
            const float d = (q[0] * wg.quat[0] + q[1] * wg.quat[1]) + (q[2] * wg.quat[2] + q[3] * wg.quat[3]);
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] = wg.quat[i] - d * q[i];
#pragma unroll
            for (int i = 0; i < 4; i++) q[i] = step_param(1, i, q[i], v[i], P.lr_quats);
            const float m2 = (q[0] * q[0] + q[1] * q[1]) + (q[2] * q[2] + q[3] * q[3]);
            const float minv = 1.0f / ssr_sqrt(m2);
            *reinterpret_cast<float4*>(W.quats + 4 * g) = make_float4(q[0] * minv, q[1] * minv, q[2] * minv, q[3] * minv);
        }
        W.opacity_logits[g] = step_param(3, 0, logit, wg.logit, P.lr_opacs);
        if (P.densify_score) {
            const float smax = ssr_max(ssr_max(ls[0], ls[1]), ls[2]);
            P.densify_score[g] = ssr_exp(smax) * ssr_sqrt(dot3(wg.mean, wg.mean));
        }
        if (P.scale_agnostic_radii) {
            // use_scale_agnostic_mean (FusedProjectionBwdOptim_kernel.cuh:519-534): the first moment takes the
            // gradient pushed through the splat's own covariance R diag(exp(log_scale)) R^T (R from the stored,
            // un-normalised quaternion, as apply_covar_to_vec does) times its opacity-aware extent, the second
            // moment the gradient scaled by 0.6 x the splat's apparent radius
            const float w = quat[0], qx = quat[1], qy = quat[2], qz = quat[3];
            const float x2 = qx * qx, y2 = qy * qy, z2 = qz * qz, xy = qx * qy, xz = qx * qz, yz = qy * qz;
            const float wx = w * qx, wy = w * qy, wz = w * qz;
            const float R[3][3] = {{1.f - 2.f * (y2 + z2), 2.f * (xy - wz), 2.f * (xz + wy)},
                                   {2.f * (xy + wz), 1.f - 2.f * (x2 + z2), 2.f * (yz - wx)},
                                   {2.f * (xz - wy), 2.f * (yz + wx), 1.f - 2.f * (x2 + y2)}};
            const float hs[3] = {ssr_exp(0.5f * ls[0]), ssr_exp(0.5f * ls[1]), ssr_exp(0.5f * ls[2])};
            float M[3][3], cov[3][3];
#pragma unroll
            for (int i = 0; i < 3; i++)
#pragma unroll
                for (int j = 0; j < 3; j++) M[i][j] = R[i][j] * hs[j];
#pragma unroll
            for (int i = 0; i < 3; i++)
#pragma unroll
                for (int j = 0; j < 3; j++) cov[i][j] = (M[i][0] * M[j][0] + M[i][1] * M[j][1]) + M[i][2] * M[j][2];
            const float extent = ssr_sqrt(2.0f * ssr_log(ssr_max(255.0f * ssr_sigmoid(logit), 1.00001f)));
            const float den = P.scale_agnostic_radii[g] * 0.6f;
            constexpr float kBeta1 = 0.9f, kBeta2 = 0.999f, kEps = 1e-15f;
#pragma unroll
            for (int i = 0; i < 3; i++) {
                const float num = ((cov[i][0] * wg.mean[0] + cov[i][1] * wg.mean[1]) + cov[i][2] * wg.mean[2]) * extent;
                float m1, m2;
                fetch_moments(0, i, m1, m2);
                m1 = kBeta1 * m1 + (1.f - kBeta1) * num;
                m2 = kBeta2 * m2 + (1.f - kBeta2) * (((wg.mean[i] * wg.mean[i]) * den) * den);
                keep_moments(0, i, m1, m2);
                W.means[3 * g + i] = mean[i] - ((P.lr_means * ad.b1c) * m1) / (ssr_sqrt(m2 * ad.b2c) + kEps);
            }
        } else {
#pragma unroll
            for (int i = 0; i < 3; i++) W.means[3 * g + i] = step_param(0, i, mean[i], wg.mean[i], P.lr_means);
        }
        // features_dc: the plain step, or (colour trust region, FusedProjectionBwdOptim_kernel.cuh:551-596) the step in the
        // space of splat_dc_encode, gradient divided by the slope of the sRGB curve at the DC colour, clipped
        constexpr float kSh0 = 0.28209479177387814f;
        float slope[3] = {1.f, 1.f, 1.f};
        if (ctl) {
            const float opac = ssr_sigmoid(logit);
            const float inv_opac = 1.0f / ssr_max(opac, 1e-12f);
#pragma unroll
            for (int c = 0; c < 3; c++) {
                const float c_dc = kSh0 * dc[c] + 0.5f;
                slope[c] = ssr_srgb_slope(c_dc);
                s_ctl[threadIdx.x][c] = slope[c];
                const float cc = ssr_max(c_dc, (1.0f / 255.0f) * (1.0f / 255.0f));
                s_ctl[threadIdx.x][3 + c] = kSh0 * ssr_sqrt(((4.0f * P.eps_tr) * cc) * inv_opac);   // :656-666
            }
        }
#pragma unroll
        for (int i = 0; i < 3; i++) {
            const float v = ctl ? wg.dc[i] / slope[i] : wg.dc[i];
            float delta = step_param(4, i, 0.0f, v, P.lr_features_dc);   // 0 - step: the step itself, exactly
            if (ctl) {
                const float clip = kSh0 * ssr_sqrt((2.0f * P.eps_tr) / ssr_max(ssr_sigmoid(logit), 1e-12f));
                delta = ssr_min(ssr_max(delta, -clip), clip);
                delta = ssr_isfinite(delta) ? delta : 0.0f;
                W.features_dc[3 * g + i] = ssr_splat_dc_decode(ssr_splat_dc_encode(dc[i]) + delta);
            } else {
                W.features_dc[3 * g + i] = dc[i] + delta;
            }
        }
    } else if (ctl) {
#pragma unroll
        for (int c = 0; c < 6; c++) s_ctl[threadIdx.x][c] = 1.0f;
    }
    if (kNsq) {
        // new bounds of the block: every thread takes part (those past the last splat hold the neutral element),
        // then each splat's 14 cells are encoded against them
#pragma unroll
        for (int t = 0; t < 5; t++) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                float v = ns_mm[t][k];
#pragma unroll
                for (int d = 32; d >= 1; d >>= 1) v = (k & 1) ? ssr_max(v, __shfl_xor(v, d, 64)) : ssr_min(v, __shfl_xor(v, d, 64));
                if ((threadIdx.x & 63) == 0) s_ns[threadIdx.x >> 6][4 * t + k] = v;
            }
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < 5; t++) {
            float mm[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                mm[k] = s_ns[0][4 * t + k];
#pragma unroll
                for (int w = 1; w < kProjBlock / 64; w++) mm[k] = (k & 1) ? ssr_max(mm[k], s_ns[w][4 * t + k]) : ssr_min(mm[k], s_ns[w][4 * t + k]);
            }
            if (threadIdx.x == 0) {
#pragma unroll
                for (int k = 0; k < 4; k++) P.non_sh_bounds[t][4 * blockIdx.x + k] = mm[k];
            }
            if (g < P.num_splats) {
#pragma unroll
                for (int i = 0; i < ns_prims(t); i++)
                    P.non_sh_packed[t][(int64_t)ns_prims(t) * g + i] = ssr_adamq16_encode(ns_g1[ns_off(t) + i], ns_g2[ns_off(t) + i], mm);
            }
        }
    }
    s_b1c[threadIdx.x] = ad.b1c; s_b2c[threadIdx.x] = ad.b2c;
    if (kCoef == 0) return;
    float old_mm[4] = {0.f, 0.f, 0.f, 0.f};
    if (kQuant) {
        static_assert(!kQuant || kProjBlock == 256, "one table entry per thread");
#pragma unroll
        for (int k = 0; k < 4; k++) old_mm[k] = P.sh_state_bounds[4 * blockIdx.x + k];
        s_sqrt_g2[threadIdx.x] = ssr_adamq_decode_sqrt_g2(threadIdx.x, old_mm);
    }
    __syncthreads();
    // phase 2: SH coefficients of the workgroup's splats in memory order (FusedProjectionBwdOptim_kernel.cuh:667-710)
    const int64_t rest = P.num_splats - block0;
    const int n_here = rest < kProjBlock ? (int)rest : kProjBlock;
    const float sh_reg = P.sh_reg_weight * (1.0f / (float)kY);
    constexpr int kPer = 3 * kCoef;
    // the colour trust region is a uniform choice: two copies of the loops, so that the plain one stays free of the branch
    auto phase2 = [&](auto ctl_tag) {
    constexpr bool kCtl = decltype(ctl_tag)::value;
    if (kQuant) {
        // Quantized state (FusedProjectionBwdOptim_kernel.cuh:709-1030 at QUANT_BITS 8, VALUE_BITS 16): moments and
        // values of this block's cells are decoded against the block's old bounds, stepped in fp32, and encoded
        // against the min / max of the results. The workgroup walks the cells in memory order twice -- once for
        // the new bounds, once (recomputing the same step from the same old codes) to encode -- rather than
        // holding 3 x 45 results per thread.
        const int R = 3 * (int)P.num_sh_buffer;                    // cells per splat
        const int64_t cell0 = block0 * R;
        const int n_cells = n_here * R;
        const float old_lo = P.sh_value_bounds[2 * blockIdx.x], old_hi = P.sh_value_bounds[2 * blockIdx.x + 1];
        // the block's cells through 32-bit offsets from its first cell: cell (sp, k) is at sp * R + k
        uint16_t* const state_cells = P.sh_state_packed + cell0;
        uint16_t* const value_cells = P.sh_value_packed + cell0;
        auto step_cell = [&](int sp, int k, float& m1, float& m2, float& xn) {
            const int cell = sp * R + k;
            const uint32_t code = state_cells[cell];
            ssr_adamq_decode_with(code, old_mm, s_sqrt_g2[code >> 8], &m1, &m2);
            const float x = ssr_q16_decode(value_cells[cell], old_lo, old_hi);
            const int j = k / 3, c = k - 3 * j;
            float v = s_Y[sp][j] * s_vc[sp][c];
            if (P.v_sh_in) v = v + P.v_sh_in[(block0 + sp) * (int64_t)P.v_sh_in_stride + k];
            v = v + sh_reg * x;
            if (kCtl) v = v / s_ctl[sp][c];
            constexpr float kBeta1 = 0.9f, kBeta2 = 0.999f, kEps = 1e-15f;
            m1 = kBeta1 * m1 + (1.f - kBeta1) * v;
            m2 = kBeta2 * m2 + (1.f - kBeta2) * (v * v);
            float delta = 0.0f - ((P.lr_features_sh * s_b1c[sp]) * m1) / (ssr_sqrt(m2 * s_b2c[sp]) + kEps);
            if (kCtl) {   // FusedProjectionBwdOptim_kernel.cuh:787-794
                const float clip = s_ctl[sp][3 + c];
                delta = ssr_min(ssr_max(delta, -clip), clip);
                delta = ssr_isfinite(delta) ? delta : 0.0f;
            }
            xn = x + delta;
        };
        float mn[3] = {1e30f, 1e30f, 1e30f}, mx[3] = {-1e30f, -1e30f, -1e30f};   // u, log_s, value
        {
            int sp = (int)threadIdx.x / R, k = (int)threadIdx.x - sp * R;
            const int dsp = kProjBlock / R, dk = kProjBlock - dsp * R;
            for (int e = threadIdx.x; e < n_cells; e += kProjBlock) {
                if (k < kPer) {
                    float m1, m2, xn, u, ls;
                    step_cell(sp, k, m1, m2, xn);
                    ssr_adamq_to_us(m1, m2, &u, &ls);
                    // the running bounds are never NaN (a NaN candidate loses every comparison), so the plain
                    // comparisons give what ssr_min / ssr_max give
                    mn[0] = (u < mn[0]) ? u : mn[0]; mx[0] = (u > mx[0]) ? u : mx[0];
                    mn[1] = (ls < mn[1]) ? ls : mn[1]; mx[1] = (ls > mx[1]) ? ls : mx[1];
                    mn[2] = (xn < mn[2]) ? xn : mn[2]; mx[2] = (xn > mx[2]) ? xn : mx[2];
                }
                sp += dsp; k += dk;
                if (k >= R) { k -= R; sp++; }
            }
        }
        if (R > kPer && n_here > 0) {   // coefficients above the active degree are re-encoded as zeros: cover zero
            mn[0] = ssr_min(mn[0], 0.0f); mx[0] = ssr_max(mx[0], 0.0f);
            mn[1] = ssr_min(mn[1], 0.0f);
            mn[2] = ssr_min(mn[2], 0.0f); mx[2] = ssr_max(mx[2], 0.0f);
        }
#pragma unroll
        for (int k = 0; k < 3; k++) {
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) {
                mn[k] = ssr_min(mn[k], __shfl_xor(mn[k], d, 64));
                mx[k] = ssr_max(mx[k], __shfl_xor(mx[k], d, 64));
            }
        }
        __syncthreads();   // s_red is free (first use), and every wavefront has finished reading the old codes
        if ((threadIdx.x & 63) == 0) {
#pragma unroll
            for (int k = 0; k < 3; k++) { s_red[threadIdx.x >> 6][2 * k] = mn[k]; s_red[threadIdx.x >> 6][2 * k + 1] = mx[k]; }
        }
        __syncthreads();
        float new_mm[4], new_lo, new_hi;
        {
            float a[6];
#pragma unroll
            for (int k = 0; k < 6; k++) {
                a[k] = s_red[0][k];
#pragma unroll
                for (int w = 1; w < kProjBlock / 64; w++) a[k] = (k & 1) ? ssr_max(a[k], s_red[w][k]) : ssr_min(a[k], s_red[w][k]);
            }
            new_mm[0] = a[0]; new_mm[1] = a[1]; new_mm[2] = a[2]; new_mm[3] = a[3]; new_lo = a[4]; new_hi = a[5];
        }
        // second walk: the same step from the same old codes, encoded against the new bounds. A cell is read and
        // written by the same thread, and the bounds are written only after every thread has them in registers.
        {
            int sp = (int)threadIdx.x / R, k = (int)threadIdx.x - sp * R;
            const int dsp = kProjBlock / R, dk = kProjBlock - dsp * R;
            for (int e = threadIdx.x; e < n_cells; e += kProjBlock) {
                float m1 = 0.0f, m2 = 0.0f, xn = 0.0f;
                if (k < kPer) step_cell(sp, k, m1, m2, xn);
                state_cells[e] = (uint16_t)ssr_adamq_encode(m1, m2, new_mm);     // e == sp * R + k
                value_cells[e] = (uint16_t)ssr_q16_encode(xn, new_lo, new_hi);
                sp += dsp; k += dk;
                if (k >= R) { k -= R; sp++; }
            }
        }
        if (threadIdx.x == 0) {
#pragma unroll
            for (int k = 0; k < 4; k++) P.sh_state_bounds[4 * blockIdx.x + k] = new_mm[k];
            P.sh_value_bounds[2 * blockIdx.x] = new_lo; P.sh_value_bounds[2 * blockIdx.x + 1] = new_hi;
        }
        return;
    }
    for (int e = threadIdx.x; e < n_here * kPer; e += kProjBlock) {
        const int sp = e / (kPer > 0 ? kPer : 1), i = e - sp * kPer;   // degree 0: no trip
        const int j = i / 3, c = i - 3 * j;
        const int64_t row = block0 + sp;
        float* xp = W.features_sh + row * W.sh_stride + i;
        const float x = *xp;
        float v = s_Y[sp][j] * s_vc[sp][c];
        if (P.v_sh_in) v = v + P.v_sh_in[row * (int64_t)P.v_sh_in_stride + i];
        v = v + sh_reg * x;
        if (kCtl) v = v / s_ctl[sp][c];     // FusedProjectionBwdOptim_kernel.cuh:694-705
        AdamD a;
        a.b1c = s_b1c[sp]; a.b2c = s_b2c[sp];
        float* g1p = P.g1.features_sh + row * P.g1.sh_stride + i;
        float* g2p = P.g2.features_sh + row * P.g2.sh_stride + i;
        float m1 = *g1p, m2 = *g2p;
        float delta = adam_core(0.0f, v, P.lr_features_sh, a, m1, m2);   // 0 - step: the step itself, exactly
        if (kCtl) {
            const float clip = s_ctl[sp][3 + c];
            delta = ssr_min(ssr_max(delta, -clip), clip);
            delta = ssr_isfinite(delta) ? delta : 0.0f;
        }
        *xp = x + delta;
        *g1p = m1; *g2p = m2;
    }
    };
    if (ctl) phase2(std::true_type{}); else phase2(std::false_type{});
}

__global__ __launch_bounds__(kProjBlock) void packed_row_map_kernel(const int32_t* __restrict__ gaussian_ids, int64_t nnz,
                                                                    int64_t num_splats, int32_t* __restrict__ row_of) {
    const int64_t i = (int64_t)blockIdx.x * kProjBlock + threadIdx.x;
    if (i >= nnz) return;
    const int32_t g = gaussian_ids[i];
    if (g >= 0 && g < num_splats) row_of[g] = (int32_t)i;
}

// One wavefront per listed splat: lane l zeroes float l of its 59-float gradient row
// (3 mean, 4 quat, 3 scale, 1 opacity, 3 dc, sh_stride SH).
// The first index i in [0, n] with a[i] >= x in the ascending array a, searched outwards from `start` in doubling
// steps and then by bisection: a few probes when the answer is near the guess, the usual logarithm otherwise.
__device__ __forceinline__ int64_t first_at_or_above(const int32_t* __restrict__ a, int64_t n, int64_t start, int x) {
    if (n <= 0) return 0;
    start = start < 0 ? 0 : (start >= n ? n - 1 : start);
    int64_t lo, hi, step = 1;
    if (a[start] < x) {          // the answer lies to the right of start
        lo = start + 1;
        int64_t i = start + step;
        while (i < n && a[i] < x) { lo = i + 1; step <<= 1; i = start + step; }
        hi = i < n ? i : n;
    } else {                     // at start or to its left
        hi = start;
        int64_t i = start - step;
        while (i >= 0 && a[i] >= x) { hi = i; step <<= 1; i = start - step; }
        lo = i >= 0 ? i + 1 : 0;
    }
    while (lo < hi) {
        const int64_t mid = (lo + hi) >> 1;
        if (a[mid] < x) lo = mid + 1; else hi = mid;
    }
    return lo;
}

// Rows of splats that are visible now (non-empty aabb when `aabb` is given, member of the ascending list
// `keep` when that is given) are skipped: the projection backward that follows overwrites them.
// A workgroup takes 256 listed rows. First every thread decides about one row: the `keep` list is bracketed
// once per workgroup by the smallest and largest id of its rows (two searches with uniform arguments; lists
// that ascend together, as two packed projections' do, leave a bracket of a few hundred entries), and each
// thread bisects inside the bracket. Then the rows that remain are zeroed, one wavefront per row.
__global__ __launch_bounds__(kProjBlock) void zero_world_rows_kernel(ssr_world V, const int32_t* __restrict__ ids, int64_t n,
                                                                     const float4* __restrict__ aabb,
                                                                     const int32_t* __restrict__ keep, int64_t n_keep) {
    __shared__ int s_rows[kProjBlock];
    __shared__ int s_count;
    __shared__ int s_lo[kProjBlock / 64], s_hi[kProjBlock / 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (threadIdx.x == 0) s_count = 0;
    const int64_t row = (int64_t)blockIdx.x * kProjBlock + threadIdx.x;
    const bool valid = row < n;
    const int g = valid ? ids[row] : 0;
    bool alive = valid;
    if (aabb && alive) {
        const float4 bb = aabb[g];
        alive = bb.z <= bb.x || bb.w <= bb.y;
    }
    if (keep && n_keep > 0) {
        int gmin = valid ? g : 0x7fffffff, gmax = valid ? g : -1;
#pragma unroll
        for (int d = 32; d >= 1; d >>= 1) {
            gmin = min(gmin, __shfl_xor(gmin, d, 64));
            gmax = max(gmax, __shfl_xor(gmax, d, 64));
        }
        if (lane == 0) { s_lo[wave] = gmin; s_hi[wave] = gmax; }
        __syncthreads();
#pragma unroll
        for (int w = 0; w < kProjBlock / 64; w++) { gmin = min(gmin, s_lo[w]); gmax = max(gmax, s_hi[w]); }
        // lists of two views of one scene name much the same splats at much the same places: guess, then gallop
        const int64_t row0 = (int64_t)blockIdx.x * kProjBlock;
        const int64_t first = first_at_or_above(keep, n_keep, row0 * n_keep / n, gmin);
        const int64_t rows_here = n - row0 < kProjBlock ? n - row0 : kProjBlock;
        const int64_t lo = first_at_or_above(keep, n_keep, first + rows_here, gmax + 1);   // ids stay below 2^31 - 1
        if (alive) {
            int64_t a = first, b = lo;     // first entry >= g inside the bracket
            while (a < b) {
                const int64_t mid = (a + b) >> 1;
                if (keep[mid] < g) a = mid + 1; else b = mid;
            }
            if (a < lo && keep[a] == g) alive = false;
        }
    } else {
        __syncthreads();
    }
    if (alive) s_rows[atomicAdd(&s_count, 1)] = g;
    __syncthreads();
    const int count = s_count;
    for (int k = wave; k < count; k += kProjBlock / 64) {
        const int64_t z = s_rows[k];
        if (lane < 3) V.means[3 * z + lane] = 0.f;
        else if (lane < 7) V.quats[4 * z + lane - 3] = 0.f;
        else if (lane < 10) V.log_scales[3 * z + lane - 7] = 0.f;
        else if (lane < 11) V.opacity_logits[z] = 0.f;
        else if (lane < 14) V.features_dc[3 * z + lane - 11] = 0.f;
        for (int c = lane; c < V.sh_stride; c += 64) V.features_sh[z * (int64_t)V.sh_stride + c] = 0.f;
    }
}

static int check_common(const char* where, int64_t n, int sh_degree, const ssr_world& w, const ssr_sh_quant& sh,
                        const ssr_camera& cam) {
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, where, "num_splats must be in [0, 2^31)");
    SSR_REQUIRE(sh_degree >= 0 && sh_degree <= 3, where, "SH degree must be 0..3");
    SSR_REQUIRE(ssr_camera_variant_supported(cam.camera_model, cam.distortion), where,
                "unsupported camera model / lens distortion pair (PINHOLE: none, opencv, thin prism, rational; FISHEYE and "
                "EQUISOLID: none, opencv, thin prism; EQUIRECTANGULAR: none)");
    SSR_REQUIRE(cam.distortion == SSR_LENS_NONE || cam.dist_coeffs, where, "null lens coefficients");
    SSR_REQUIRE(cam.num_cameras == 1, where, "exactly one camera per call is supported");
    SSR_REQUIRE(cam.width > 0 && cam.height > 0, where, "empty image");
    SSR_REQUIRE(cam.viewmats && cam.intrins, where, "null camera pointer");
    if (n == 0) return 0;
    SSR_REQUIRE(w.means && w.quats && w.log_scales && w.opacity_logits && w.features_dc, where, "null world buffer");
    if (sh_degree > 0) {
        switch (sh.codec) {
            case SSR_SH_F32:
                SSR_REQUIRE(w.features_sh, where, "null features_sh");
                SSR_REQUIRE(w.sh_stride >= 3 * sh_degree * (sh_degree + 2), where, "sh_stride too small for the SH degree");
                break;
            case SSR_SH_REF_Q8: case SSR_SH_REF_Q16:
                SSR_REQUIRE(sh.packed && sh.bounds, where, "null quantized SH buffer");
                SSR_REQUIRE(sh.num_sh_buffer >= (uint32_t)(sh_degree * (sh_degree + 2)), where, "num_sh_buffer too small");
                SSR_REQUIRE(sh.bounds_stride >= 0, where, "negative bounds stride");
                break;
            case SSR_SH_I8_F16SCALE:
                SSR_REQUIRE(sh.packed && sh.scale_f16, where, "null quantized SH buffer");
                break;
            default: return fail(where, "unknown SH codec");
        }
    }
    return 0;
}

}  // namespace ssr

using namespace ssr;

extern "C" int ssr_projection_fwd(const ssr_projection_fwd_params* p, ssr_stream_t stream) {
    SSR_REQUIRE(p, "ssr_projection_fwd", "null params");
    int e = check_common("ssr_projection_fwd", p->num_splats, p->sh_degree, p->world, p->sh, p->camera);
    if (e) return e;
    if (p->num_splats == 0) return 0;
    SSR_REQUIRE(p->aabb && p->sort_depth && p->radii, "ssr_projection_fwd", "null output");
    SSR_REQUIRE(p->screen.xy && p->screen.depth && p->screen.conic && p->screen.opac && p->screen.rgb,
                "ssr_projection_fwd", "null screen buffer");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->aabb) & 15) == 0 && (reinterpret_cast<uintptr_t>(p->world.quats) & 15) == 0,
                "ssr_projection_fwd", "aabb and quats must be 16-byte aligned");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->screen.xy) & 7) == 0, "ssr_projection_fwd", "screen.xy must be 8-byte aligned");
    SSR_REQUIRE(!p->visible_ids || p->visible_count, "ssr_projection_fwd", "visible_ids needs visible_count");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->packed_rows) & 15) == 0, "ssr_projection_fwd", "packed_rows must be 16-byte aligned");
    const dim3 grid((unsigned)ceil_div(p->num_splats, kProjBlock)), block(kProjBlock);
    hipStream_t s = as_stream(stream);
    const bool lens = camera_needs_lens_path(p->camera.camera_model, p->camera.distortion);
#define SSR_LAUNCH_FWD(D)                                                                          \
    if (lens) hipLaunchKernelGGL((projection_fwd_kernel<D, true>), grid, block, 0, s, *p);         \
    else hipLaunchKernelGGL((projection_fwd_kernel<D, false>), grid, block, 0, s, *p)
    switch (p->sh_degree) {
        case 0: SSR_LAUNCH_FWD(0); break;
        case 1: SSR_LAUNCH_FWD(1); break;
        case 2: SSR_LAUNCH_FWD(2); break;
        default: SSR_LAUNCH_FWD(3); break;
    }
#undef SSR_LAUNCH_FWD
    SSR_CHECK_LAUNCH("ssr_projection_fwd");
    return 0;
}

extern "C" size_t ssr_projection_packed_scratch_bytes(int64_t num_splats) {
    if (num_splats <= 0) return 16;
    return packed_stage_layout(num_splats, nullptr, nullptr);
}

extern "C" size_t ssr_projection_packed_scratch_bytes_world_rows(int64_t num_splats) {
    if (num_splats <= 0) return 16;
    return packed_stage_layout(num_splats, nullptr, nullptr, true);
}

static int check_packed(const char* where, const ssr_projection_packed_params* p) {
    SSR_REQUIRE(p, where, "null params");
    int e = check_common(where, p->num_splats, p->sh_degree, p->world, p->sh, p->camera);
    if (e) return e;
    SSR_REQUIRE(p->nnz, where, "null nnz");
    if (p->num_splats == 0) return 0;
    SSR_REQUIRE(p->scratch && (reinterpret_cast<uintptr_t>(p->scratch) & 15) == 0, where, "scratch must be non-null and 16-byte aligned");
    if (p->stage_world_rows)
        SSR_REQUIRE(p->scratch_bytes >= ssr_projection_packed_scratch_bytes_world_rows(p->num_splats), where,
                    "scratch too small (with stage_world_rows it holds ssr_projection_packed_scratch_bytes_world_rows bytes)");
    SSR_REQUIRE(!p->world_rows || p->stage_world_rows, where, "world_rows needs stage_world_rows set, in the mask call as well");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->world_rows) & 15) == 0, where, "world_rows must be 16-byte aligned");
    SSR_REQUIRE(!p->world_rows || p->world_rows_stride >= p->max_rows, where, "world_rows_stride must be at least max_rows");
    SSR_REQUIRE(p->scratch_bytes >= ssr_projection_packed_scratch_bytes(p->num_splats), where, "scratch too small");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->world.quats) & 15) == 0, where, "quats must be 16-byte aligned");
    return 0;
}

extern "C" int ssr_projection_packed_mask(const ssr_projection_packed_params* p, ssr_stream_t stream) {
    const char* where = "ssr_projection_packed_mask";
    int e = check_packed(where, p);
    if (e) return e;
    hipStream_t s = as_stream(stream);
    if (p->num_splats == 0) {   // nnz = 0 without touching the scratch
        hipLaunchKernelGGL(packed_block_scan_kernel, dim3(1), dim3(kScanOneBlock), 0, s, (const int32_t*)nullptr, (int64_t)0,
                           p->nnz, p->nnz);
        SSR_CHECK_LAUNCH(where);
        return 0;
    }
    SSR_REQUIRE(p->radii, where, "null radii");
    PackedStage st;
    packed_stage_layout(p->num_splats, p->scratch, &st, p->stage_world_rows != 0);
    const int64_t nb = ceil_div(p->num_splats, kPackSeg);
    if (camera_needs_lens_path(p->camera.camera_model, p->camera.distortion))
        hipLaunchKernelGGL(projection_packed_mask_kernel<true>, dim3((unsigned)nb), dim3(kProjBlock), 0, s, *p, st);
    else
        hipLaunchKernelGGL(projection_packed_mask_kernel<false>, dim3((unsigned)nb), dim3(kProjBlock), 0, s, *p, st);
    SSR_CHECK_LAUNCH(where);
    hipLaunchKernelGGL(packed_block_scan_kernel, dim3(1), dim3(kScanOneBlock), 0, s, (const int32_t*)st.block_counts, nb,
                       st.block_offsets, p->nnz);
    SSR_CHECK_LAUNCH(where);
    return 0;
}

extern "C" int ssr_projection_packed_emit(const ssr_projection_packed_params* p, ssr_stream_t stream) {
    const char* where = "ssr_projection_packed_emit";
    int e = check_packed(where, p);
    if (e) return e;
    SSR_REQUIRE(p->max_rows >= 0 && p->max_rows <= p->num_splats, where, "max_rows must be in [0, num_splats]");
    if (p->num_splats == 0 || p->max_rows == 0) return 0;
    SSR_REQUIRE(p->camera_ids && p->gaussian_ids && p->aabb && p->sort_depth, where, "null output");
    SSR_REQUIRE(p->screen.xy && p->screen.depth && p->screen.conic && p->screen.opac && p->screen.rgb, where, "null screen buffer");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->aabb) & 15) == 0, where, "aabb must be 16-byte aligned");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->screen.xy) & 7) == 0, where, "screen.xy must be 8-byte aligned");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->packed_rows) & 15) == 0, where, "packed_rows must be 16-byte aligned");
    PackedStage st;
    packed_stage_layout(p->num_splats, p->scratch, &st, p->stage_world_rows != 0);
    const dim3 grid((unsigned)ceil_div(p->max_rows, kProjBlock)), block(kProjBlock);
    hipStream_t s = as_stream(stream);
    switch (p->sh_degree) {
        case 0: hipLaunchKernelGGL(projection_packed_emit_kernel<0>, grid, block, 0, s, *p, st); break;
        case 1: hipLaunchKernelGGL(projection_packed_emit_kernel<1>, grid, block, 0, s, *p, st); break;
        case 2: hipLaunchKernelGGL(projection_packed_emit_kernel<2>, grid, block, 0, s, *p, st); break;
        default: hipLaunchKernelGGL(projection_packed_emit_kernel<3>, grid, block, 0, s, *p, st); break;
    }
    SSR_CHECK_LAUNCH(where);
    return 0;
}

extern "C" int ssr_projection_bwd(const ssr_projection_bwd_params* p, ssr_stream_t stream) {
    SSR_REQUIRE(p, "ssr_projection_bwd", "null params");
    int e = check_common("ssr_projection_bwd", p->num_splats, p->sh_degree, p->world, p->sh, p->camera);
    if (e) return e;
    if (p->num_splats == 0) return 0;   // src/kernels/projection/ProjectionBwd.cu:86-87
    const bool packed = p->packed_gaussian_ids != nullptr;
    if (packed) {
        SSR_REQUIRE(!p->visible_ids, "ssr_projection_bwd", "packed mode takes no visible list");
        SSR_REQUIRE(p->num_packed >= 0 && p->num_packed <= p->num_splats, "ssr_projection_bwd", "num_packed out of range");
        if (p->num_packed == 0) return 0;
        SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->packed_world_rows) & 15) == 0, "ssr_projection_bwd", "packed_world_rows must be 16-byte aligned");
        SSR_REQUIRE(!p->packed_world_rows || p->packed_world_stride >= p->num_packed, "ssr_projection_bwd", "packed_world_stride must be at least num_packed");
    } else {
        SSR_REQUIRE(p->aabb, "ssr_projection_bwd", "null aabb");   // ProjectionBwd.cu:89-97
        SSR_REQUIRE(!p->packed_world_rows, "ssr_projection_bwd", "packed_world_rows belongs to packed mode");
    }
    SSR_REQUIRE(p->v_rows || (p->v_screen.xy && p->v_screen.depth && p->v_screen.conic && p->v_screen.opac && p->v_screen.rgb),
                "ssr_projection_bwd", "null v_screen buffer");
    const ssr_world& v = p->v_world;
    SSR_REQUIRE(v.means && v.quats && v.log_scales && v.opacity_logits && v.features_dc && v.features_sh,
                "ssr_projection_bwd", "null v_world buffer");
    SSR_REQUIRE(v.sh_stride >= 3 * p->sh_degree * (p->sh_degree + 2), "ssr_projection_bwd", "v_world.sh_stride too small");
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->aabb) & 15) == 0 && (reinterpret_cast<uintptr_t>(p->world.quats) & 15) == 0 &&
                (reinterpret_cast<uintptr_t>(v.quats) & 15) == 0, "ssr_projection_bwd", "aabb and quats must be 16-byte aligned");
    if (p->visible_ids) {
        SSR_REQUIRE(p->n_visible >= 0 && p->n_visible <= p->num_splats, "ssr_projection_bwd", "visible count out of range");
        if (p->n_visible == 0) return 0;
    }
    const int64_t work = packed ? p->num_packed : (p->visible_ids ? p->n_visible : p->num_splats);
    const dim3 grid((unsigned)ceil_div(work, kProjBlock)), block(kProjBlock);
    hipStream_t s = as_stream(stream);
    const bool lens = camera_needs_lens_path(p->camera.camera_model, p->camera.distortion);
    // accumulating over packed rows: a caller's id list may name a splat more than once (rows of several
    // cameras), so add atomically unless the caller vouches for unique ids
    const int put_mode = !p->accumulate ? kPutStore : ((packed && !p->packed_ids_unique) ? kPutAtomic : kPutAdd);
#define SSR_LAUNCH_BWD_L(D, L)                                                                                          \
    switch (put_mode) {                                                                                                 \
        case kPutStore: hipLaunchKernelGGL((projection_bwd_kernel<D, kPutStore, L>), grid, block, 0, s, *p); break;       \
        case kPutAdd: hipLaunchKernelGGL((projection_bwd_kernel<D, kPutAdd, L>), grid, block, 0, s, *p); break;           \
        default: hipLaunchKernelGGL((projection_bwd_kernel<D, kPutAtomic, L>), grid, block, 0, s, *p); break;             \
    }
#define SSR_LAUNCH_BWD(D) if (lens) { SSR_LAUNCH_BWD_L(D, true) } else { SSR_LAUNCH_BWD_L(D, false) }
    // degree 3 into gradient rows of 45 floats, 16-byte aligned: the kernel that stages those rows through LDS
    const bool staged = p->sh_degree == 3 && v.sh_stride == kShRow && put_mode != kPutAtomic &&
                        (reinterpret_cast<uintptr_t>(v.features_sh) & 15) == 0;
    if (staged) {
        if (put_mode == kPutStore) {
            if (lens) hipLaunchKernelGGL((projection_bwd_staged_kernel<kPutStore, true>), grid, block, 0, s, *p);
            else hipLaunchKernelGGL((projection_bwd_staged_kernel<kPutStore, false>), grid, block, 0, s, *p);
        } else {
            if (lens) hipLaunchKernelGGL((projection_bwd_staged_kernel<kPutAdd, true>), grid, block, 0, s, *p);
            else hipLaunchKernelGGL((projection_bwd_staged_kernel<kPutAdd, false>), grid, block, 0, s, *p);
        }
    } else
    switch (p->sh_degree) {
        case 0: SSR_LAUNCH_BWD(0); break;
        case 1: SSR_LAUNCH_BWD(1); break;
        case 2: SSR_LAUNCH_BWD(2); break;
        default: SSR_LAUNCH_BWD(3); break;
    }
#undef SSR_LAUNCH_BWD
#undef SSR_LAUNCH_BWD_L
    SSR_CHECK_LAUNCH("ssr_projection_bwd");
    if (p->v_viewmat) {
#define SSR_LAUNCH_POSE(D)                                                                            \
    if (lens) hipLaunchKernelGGL((projection_pose_bwd_kernel<D, true>), grid, block, 0, s, *p);        \
    else hipLaunchKernelGGL((projection_pose_bwd_kernel<D, false>), grid, block, 0, s, *p);
        switch (p->sh_degree) {
            case 0: SSR_LAUNCH_POSE(0); break;
            case 1: SSR_LAUNCH_POSE(1); break;
            case 2: SSR_LAUNCH_POSE(2); break;
            default: SSR_LAUNCH_POSE(3); break;
        }
#undef SSR_LAUNCH_POSE
        SSR_CHECK_LAUNCH("ssr_projection_bwd (camera pose)");
    }
    return 0;
}

extern "C" int ssr_packed_row_map(const int32_t* gaussian_ids, int64_t nnz, int64_t num_splats, int32_t* row_of,
                                  ssr_stream_t stream) {
    const char* where = "ssr_packed_row_map";
    SSR_REQUIRE(num_splats >= 0 && num_splats < (int64_t)1 << 31 && nnz >= 0 && nnz <= num_splats, where, "counts out of range");
    if (num_splats == 0) return 0;
    SSR_REQUIRE(row_of && (nnz == 0 || gaussian_ids), where, "null buffer");
    if (ssr_fill_u32(row_of, 0xffffffffu, num_splats, stream)) return 1;
    if (nnz == 0) return 0;
    hipLaunchKernelGGL(packed_row_map_kernel, dim3((unsigned)ceil_div(nnz, kProjBlock)), dim3(kProjBlock), 0, as_stream(stream),
                       gaussian_ids, nnz, num_splats, row_of);
    SSR_CHECK_LAUNCH(where);
    return 0;
}

extern "C" int ssr_fused_projection_bwd_optimizer(const ssr_fpbo_params* p, ssr_stream_t stream) {
    const char* where = "ssr_fused_projection_bwd_optimizer";
    SSR_REQUIRE(p, where, "null params");
    ssr_sh_quant none;
    memset(&none, 0, sizeof(none));
    if (p->sh_state_packed) {   // the coefficients are read from the 16-bit value codes
        none.codec = SSR_SH_REF_Q16; none.packed = p->sh_value_packed; none.bounds = p->sh_value_bounds;
        none.num_sh_buffer = p->num_sh_buffer;
    }
    int e = check_common(where, p->num_splats, p->sh_degree, p->world, none, p->camera);
    if (e) return e;
    if (p->num_splats == 0) return 0;
    SSR_REQUIRE(p->aabb && (reinterpret_cast<uintptr_t>(p->aabb) & 15) == 0, where, "aabb must be non-null and 16-byte aligned");
    SSR_REQUIRE(p->v_rows || (p->v_screen.xy && p->v_screen.depth && p->v_screen.conic && p->v_screen.opac && p->v_screen.rgb), where,
                "null v_screen buffer");
    const bool quant = p->sh_state_packed != nullptr;
    int n_ns = 0;
    for (int t = 0; t < 5; t++) n_ns += (p->non_sh_packed[t] != nullptr) + (p->non_sh_bounds[t] != nullptr);
    SSR_REQUIRE(n_ns == 0 || n_ns == 10, where, "the quantized non-SH state needs all five packed and all five bounds arrays");
    const bool nsq = n_ns == 10;
    SSR_REQUIRE(!nsq || quant, where, "the quantized non-SH state is built together with the quantized SH state only");
    for (const ssr_world* w : {&p->world, &p->g1, &p->g2}) {
        SSR_REQUIRE((nsq && w != &p->world) || (w->means && w->quats && w->log_scales && w->opacity_logits && w->features_dc), where,
                    "null parameter or moment buffer");
        SSR_REQUIRE(quant || p->sh_degree == 0 || (w->features_sh && w->sh_stride >= 3 * p->sh_degree * (p->sh_degree + 2)), where,
                    "features_sh missing or sh_stride too small");
    }
    if (quant) {
        SSR_REQUIRE(p->sh_state_bounds && p->sh_value_packed && p->sh_value_bounds, where, "null quantized SH state buffer");
        SSR_REQUIRE((int)p->num_sh_buffer >= p->sh_degree * (p->sh_degree + 2) && p->num_sh_buffer <= 15u, where,
                    "num_sh_buffer must cover the SH degree (at most 15)");
    }
    SSR_REQUIRE((reinterpret_cast<uintptr_t>(p->world.quats) & 15) == 0, where, "quats must be 16-byte aligned");
    SSR_REQUIRE(p->steps || p->step >= 1, where, "Adam step must be >= 1");
    AdamD ad;
    ad.b1c = ssr_adam_inv_bias1((float)p->step);
    ad.b2c = ssr_adam_inv_bias2((float)p->step);
    const dim3 grid((unsigned)ceil_div(p->num_splats, kProjBlock)), block(kProjBlock);
    hipStream_t s = as_stream(stream);
    const bool lens = camera_needs_lens_path(p->camera.camera_model, p->camera.distortion);
#define SSR_LAUNCH_FPBO_Q(D, L)                                                                                             \
    if (nsq) hipLaunchKernelGGL((fused_projection_bwd_optimizer_kernel<D, L, true, true>), grid, block, 0, s, *p, ad);          \
    else if (quant) hipLaunchKernelGGL((fused_projection_bwd_optimizer_kernel<D, L, true, false>), grid, block, 0, s, *p, ad);  \
    else hipLaunchKernelGGL((fused_projection_bwd_optimizer_kernel<D, L, false, false>), grid, block, 0, s, *p, ad);
#define SSR_LAUNCH_FPBO(D)           \
    if (lens) {                      \
        SSR_LAUNCH_FPBO_Q(D, true)   \
    } else {                         \
        SSR_LAUNCH_FPBO_Q(D, false)  \
    }
    switch (p->sh_degree) {
        case 0: SSR_LAUNCH_FPBO(0); break;
        case 1: SSR_LAUNCH_FPBO(1); break;
        case 2: SSR_LAUNCH_FPBO(2); break;
        default: SSR_LAUNCH_FPBO(3); break;
    }
#undef SSR_LAUNCH_FPBO
#undef SSR_LAUNCH_FPBO_Q
    SSR_CHECK_LAUNCH(where);
    return 0;
}

extern "C" int ssr_zero_world_rows(const ssr_world* v_world, const int32_t* ids, int64_t n, const float* skip_visible_aabb,
                                   const int32_t* skip_sorted_ids, int64_t n_skip, ssr_stream_t stream) {
    SSR_REQUIRE(v_world, "ssr_zero_world_rows", "null world");
    SSR_REQUIRE(n >= 0 && n < (int64_t)1 << 31, "ssr_zero_world_rows", "count out of range");
    if (n == 0) return 0;
    SSR_REQUIRE(ids, "ssr_zero_world_rows", "null ids");
    SSR_REQUIRE(n_skip >= 0 && (n_skip == 0 || skip_sorted_ids), "ssr_zero_world_rows", "skip list: negative count or null ids");
    const ssr_world& v = *v_world;
    SSR_REQUIRE(v.means && v.quats && v.log_scales && v.opacity_logits && v.features_dc && (v.features_sh || v.sh_stride == 0),
                "ssr_zero_world_rows", "null buffer");
    hipLaunchKernelGGL(zero_world_rows_kernel, dim3((unsigned)ceil_div(n, kProjBlock)), dim3(kProjBlock), 0, as_stream(stream),
                       v, ids, n, reinterpret_cast<const float4*>(skip_visible_aabb), skip_sorted_ids, n_skip);
    SSR_CHECK_LAUNCH("ssr_zero_world_rows");
    return 0;
}
