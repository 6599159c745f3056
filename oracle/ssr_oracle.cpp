// ssr_oracle.cpp -- CPU restatement of the reference's Gaussian-splat raster hot path.
//
// TEST INFRASTRUCTURE ONLY: used by tests, the smoke check and the benchmark's cpu_baseline leg
// to check and to time against; never linked into or called from the product library.
//
// Arithmetic policy: IEEE binary32, no contraction (`-ffp-contract=off`), no fast-math; fused
// multiply-adds only where written as ssr_fma(); exp/log/atan2 from include/ssr_math.h. Each
// function names the reference source it follows.
#include "ssr_oracle.h"
#include "../include/ssr_math.h"
#include "../include/ssr_camera.h"
#include "../include/ssr_quant.h"
#include "../include/ssr_colour.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>
#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

constexpr float kAlphaThreshold = 1.0f / 255.0f;   // src/core/Common.cuh:47
constexpr int kTile = 16;                          // TILE_SIZE_X * MACRO_TILE_SIZE_X, Common.cuh:36-39
constexpr int kMicro = 8;                          // TILE_SIZE_X

struct Cam {
    int model;
    uint32_t W, H;
    float R[3][3];
    float t[3];
    float fx, fy, cx, cy;
    int tier;
    float dc[8];
    bool aa;   // antialiased ("mip") variant
};

// PINHOLE without lens distortion and EQUIRECTANGULAR are written out by hand below; the other
// (model, tier) pairs use the differentiated model functions of include/ssr_camera.h.
bool lens_path(const Cam& c) { return !((c.model == OR_CAM_PINHOLE && c.tier == OR_LENS_NONE) || c.model == OR_CAM_EQUIRECT); }

Cam load_cam(const or_camera* c) {
    // src/kernels/projection/ProjectionFwd_kernel.cuh:52-60
    Cam k;
    k.model = c->model; k.W = c->width; k.H = c->height;
    for (int i = 0; i < 3; i++) {
        for (int j = 0; j < 3; j++) k.R[i][j] = c->viewmat[4 * i + j];
        k.t[i] = c->viewmat[4 * i + 3];
    }
    k.fx = c->fx; k.fy = c->fy; k.cx = c->cx; k.cy = c->cy;
    k.tier = c->distortion;
    for (int i = 0; i < 8; i++) k.dc[i] = (c->distortion != OR_LENS_NONE) ? c->dist_coeffs[i] : 0.0f;
    k.aa = c->antialiased != 0;
    return k;
}

float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h >> 15) << 31;
    uint32_t e = (h >> 10) & 0x1f, m = h & 0x3ff;
    if (e == 0) {
        if (m == 0) return ssr_u2f(sign);
        float f = (float)m * 5.9604644775390625e-8f;  // m * 2^-24, exact
        return (sign ? -f : f);
    }
    if (e == 31) return ssr_u2f(sign | 0x7f800000u | (m << 13));
    return ssr_u2f(sign | ((e + 112) << 23) | (m << 13));
}

uint16_t float_to_half_rn(float f) {
    uint32_t u = ssr_f2u(f);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t au = u & 0x7fffffffu;
    if (au >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | ((au > 0x7f800000u) ? 0x200u : 0));
    if (au >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);          // rounds to inf
    if (au < 0x33000001u) return (uint16_t)sign;                        // rounds to zero
    int e = (int)(au >> 23) - 127;
    uint32_t m = (au & 0x7fffffu) | 0x800000u;
    int shift = (e < -14) ? (13 + (-14 - e)) : 13;
    uint32_t hm = m >> shift;
    uint32_t rem = m & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (hm & 1))) hm++;
    uint32_t he = (e < -14) ? 0 : (uint32_t)(e + 15);
    // hm carries the implicit bit when normal; adding handles mantissa overflow into exponent
    uint32_t h = (e < -14) ? hm : ((he << 10) + (hm - 0x400u));
    return (uint16_t)(sign | h);
}

// src/shaders/harmonics.slang:114-140 (_sh_load_q8/_q16); int8*fp16-scale is the benchmark codec.
void decode_sh(int64_t gid, const or_sh_source* sh, int n_coef, float* out /* [n_coef*3] */) {
    if (sh->codec == OR_SH_F32) {
        const float* p = sh->sh_f32 + gid * 45;
        for (int i = 0; i < n_coef * 3; i++) out[i] = p[i];
        return;
    }
    if (sh->codec == OR_SH_I8_F16SCALE) {
        const int8_t* p = reinterpret_cast<const int8_t*>(sh->packed) + gid * 45;
        float s = half_to_float(sh->scale_f16[gid]);
        for (int i = 0; i < n_coef * 3; i++) out[i] = (float)p[i] * s;
        return;
    }
    const int64_t base = (int64_t)3 * (int64_t)sh->num_sh_buffer * gid;
    const int64_t stride = sh->bounds_stride > 0 ? sh->bounds_stride
                                                 : (int64_t)256 * 3 * (int64_t)sh->num_sh_buffer;
    const bool q16 = sh->codec == OR_SH_REF_Q16;
    const float inv = q16 ? (1.0f / 65535.0f) : (1.0f / 255.0f);
    for (int i = 0; i < n_coef * 3; i++) {
        int64_t cell = base + i;
        const float* mm = sh->bounds + 2 * (cell / stride);
        float q = q16 ? (float)reinterpret_cast<const uint16_t*>(sh->packed)[cell]
                      : (float)sh->packed[cell];
        out[i] = mm[0] + (mm[1] - mm[0]) * (q * inv);
    }
}

// Real SH basis values for degree <= 3 (excluding DC), src/shaders/harmonics.slang:154-223.
struct ShBasis { float Y[15]; float x, y, z, inorm; };

ShBasis sh_basis(int degree, const float dir[3]) {
    ShBasis b;
    for (float& v : b.Y) v = 0.0f;
    b.inorm = 1.0f / ssr_sqrt((dir[0] * dir[0] + dir[1] * dir[1]) + dir[2] * dir[2]);
    float x = dir[0] * b.inorm, y = dir[1] * b.inorm, z = dir[2] * b.inorm;
    b.x = x; b.y = y; b.z = z;
    if (degree < 1) return b;
    b.Y[0] = -0.48860251190292f * y;
    b.Y[1] = 0.48860251190292f * z;
    b.Y[2] = -0.48860251190292f * x;
    if (degree < 2) return b;
    float z2 = z * z;
    float fTmp0B = -1.092548430592079f * z;
    float fC1 = x * x - y * y;
    float fS1 = 2.f * x * y;
    b.Y[3] = 0.5462742152960395f * fS1;
    b.Y[4] = fTmp0B * y;
    b.Y[5] = 0.9461746957575601f * z2 - 0.3153915652525201f;
    b.Y[6] = fTmp0B * x;
    b.Y[7] = 0.5462742152960395f * fC1;
    if (degree < 3) return b;
    float fTmp0C = -2.285228997322329f * z2 + 0.4570457994644658f;
    float fTmp1B = 1.445305721320277f * z;
    float fC2 = x * fC1 - y * fS1;
    float fS2 = x * fS1 + y * fC1;
    b.Y[8] = -0.5900435899266435f * fS2;
    b.Y[9] = fTmp1B * fS1;
    b.Y[10] = fTmp0C * y;
    b.Y[11] = z * (1.865881662950577f * z2 - 1.119528997770346f);
    b.Y[12] = fTmp0C * x;
    b.Y[13] = fTmp1B * fC1;
    b.Y[14] = -0.5900435899266435f * fC2;
    return b;
}

// colour before the +0.5 shift; src/shaders/harmonics.slang:154-223. The degree-1 band is
// written there as fTmp0A * (-y*c0 + z*c1 - x*c2); the higher bands as sums of Y_j * c_j.
void sh_color_raw(int degree, const ShBasis& b, const float dc[3], const float* c, float out[3]) {
    for (int ch = 0; ch < 3; ch++) {
        float col = 0.2820947917738781f * dc[ch];
        if (degree >= 1) {
            col = col + 0.48860251190292f *
                            (((-b.y) * c[0 * 3 + ch] + b.z * c[1 * 3 + ch]) - b.x * c[2 * 3 + ch]);
        }
        if (degree >= 2) {
            float s = b.Y[3] * c[3 * 3 + ch] + b.Y[4] * c[4 * 3 + ch];
            s = s + b.Y[5] * c[5 * 3 + ch];
            s = s + b.Y[6] * c[6 * 3 + ch];
            s = s + b.Y[7] * c[7 * 3 + ch];
            col = col + s;
        }
        if (degree >= 3) {
            float s = b.Y[8] * c[8 * 3 + ch] + b.Y[9] * c[9 * 3 + ch];
            for (int j = 10; j < 15; j++) s = s + b.Y[j] * c[j * 3 + ch];
            col = col + s;
        }
        out[ch] = col;
    }
}

// mean + R^T t, src/shaders/harmonics.slang:145-149
void view_dir(const Cam& cam, const float m[3], float dir[3]) {
    for (int i = 0; i < 3; i++)
        dir[i] = m[i] + ((cam.R[0][i] * cam.t[0] + cam.R[1][i] * cam.t[1]) + cam.R[2][i] * cam.t[2]);
}

struct Proj {
    bool valid;
    float aabb[4];
    float sort_depth, radius;
    float xy[2], depth, conic[3], opac;
    // intermediates reused by the VJP
    float mc[3], qn[4], qinv, s[3], Rq[3][3], M[3][3], J[2][3], covc[3][3];
    float c2[2][2];   // blurred 2D covariance
    float sig, comp, det_orig, det_blur, c2o[2];   // antialiased variant: sigmoid(logit), compensation, determinants, pre-blur diagonal
    bool clamp_lo[2], clamp_hi[2];
};

void quat_to_rot(const float q[4], float R[3][3]) {
    // src/shaders/projection_utils.slang:69-87
    float w = q[0], x = q[1], y = q[2], z = q[3];
    float x2 = x * x, y2 = y * y, z2 = z * z;
    float xy = x * y, xz = x * z, yz = y * z;
    float wx = w * x, wy = w * y, wz = w * z;
    R[0][0] = 1.f - 2.f * (y2 + z2); R[0][1] = 2.f * (xy - wz); R[0][2] = 2.f * (xz + wy);
    R[1][0] = 2.f * (xy + wz); R[1][1] = 1.f - 2.f * (x2 + z2); R[1][2] = 2.f * (yz - wx);
    R[2][0] = 2.f * (xz - wy); R[2][1] = 2.f * (yz + wx); R[2][2] = 1.f - 2.f * (x2 + y2);
}

inline float dot3(const float a[3], const float b[3]) { return (a[0] * b[0] + a[1] * b[1]) + a[2] * b[2]; }

// src/shaders/projection_utils.slang:1033-1043
float view_radius(const float mean[3], const float ls[3], float logit, const float campos[3]) {
    float extend = ssr_sqrt(2.0f * ssr_log(ssr_max(255.0f / (1.0f + ssr_exp(-logit)), 1.0f)));
    float radius = ssr_exp(ssr_max(ls[0], ssr_max(ls[1], ls[2]))) * extend;
    float d[3] = {mean[0] - campos[0], mean[1] - campos[1], mean[2] - campos[2]};
    float dist = ssr_sqrt(dot3(d, d));
    return radius / (ssr_max(dist, radius) + ssr_sqrt(ssr_max(dist * dist - radius * radius, 0.0f)));
}

// projection_3dgs<camera_model, DistNone, assume_valid, eval3d=false>,
// src/shaders/primitive_3dgs.slang:419-578. With assume_valid the cull branches are skipped
// (the form the backward differentiates, :644-653).
Proj project(const Cam& cam, const float mean[3], const float quat[4], const float ls[3],
             float logit, bool assume_valid) {
    Proj p;
    std::memset(&p, 0, sizeof(p));
    p.valid = false;
    for (int i = 0; i < 3; i++)
        p.mc[i] = ((cam.R[i][0] * mean[0] + cam.R[i][1] * mean[1]) + cam.R[i][2] * mean[2]) + cam.t[i];
    const float x = p.mc[0], y = p.mc[1], z = p.mc[2];
    float len = ssr_sqrt(dot3(p.mc, p.mc));
    float cull_z = (cam.model == OR_CAM_PINHOLE) ? z : len;
    p.depth = len;
    if (!assume_valid && cull_z <= 0.0f) return p;

    p.opac = 1.0f / (1.0f + ssr_exp(-logit));

    // quat_scale_to_covar(normalize(quat), exp(scale)), projection_utils.slang:112-124
    p.qinv = 1.0f / ssr_sqrt(((quat[0] * quat[0] + quat[1] * quat[1]) + quat[2] * quat[2]) + quat[3] * quat[3]);
    for (int i = 0; i < 4; i++) p.qn[i] = quat[i] * p.qinv;
    for (int i = 0; i < 3; i++) p.s[i] = ssr_exp(ls[i]);
    quat_to_rot(p.qn, p.Rq);
    for (int i = 0; i < 3; i++)
        for (int j = 0; j < 3; j++) p.M[i][j] = p.Rq[i][j] * p.s[j];
    float cov[3][3], tmp[3][3];
    for (int i = 0; i < 3; i++)
        for (int j = 0; j < 3; j++)
            cov[i][j] = (p.M[i][0] * p.M[j][0] + p.M[i][1] * p.M[j][1]) + p.M[i][2] * p.M[j][2];
    // covarW2C: R * cov * R^T, projection_utils.slang:100-108
    for (int i = 0; i < 3; i++)
        for (int j = 0; j < 3; j++)
            tmp[i][j] = (cam.R[i][0] * cov[0][j] + cam.R[i][1] * cov[1][j]) + cam.R[i][2] * cov[2][j];
    for (int i = 0; i < 3; i++)
        for (int j = 0; j < 3; j++)
            p.covc[i][j] = (tmp[i][0] * cam.R[j][0] + tmp[i][1] * cam.R[j][1]) + tmp[i][2] * cam.R[j][2];

    float (*J)[3] = p.J;
    if (lens_path(cam)) {
        // persp / fisheye / equisolid _proj<D, assume_valid> and _proj_jac<D>
        // (projection_utils.slang:345-358,414-427,446-459 and :362-375,463-493): the point is
        // dropped when the lens map is not locally invertible there (is_valid_distortion, :310-321);
        // otherwise uv and its Jacobian come from one first-order evaluation of the model.
        typedef SsrJet<3, 1> Jet;
        Jet u, v, du, dv;
        ssr_model_normalised<Jet>(cam.model, ssr_jet_seed<3, 1>(x, 0), ssr_jet_seed<3, 1>(y, 1), ssr_jet_seed<3, 1>(z, 2), u, v);
        if (!assume_valid && !ssr_distortion_valid(cam.tier, cam.dc, u.v, v.v)) return p;
        ssr_distort<Jet>(cam.tier, cam.dc, u, v, du, dv);
        const Jet px = du * cam.fx + cam.cx, py = dv * cam.fy + cam.cy;
        p.xy[0] = px.v; p.xy[1] = py.v;
        for (int k = 0; k < 3; k++) { J[0][k] = px.d[k]; J[1][k] = py.d[k]; }
        if (cam.model == OR_CAM_PINHOLE) {   // the clamp of persp_proj_3dgs, primitive_3dgs.slang:84-95
            float Wf = (float)cam.W;
            float lim_pos = Wf + 0.3f * (0.5f * Wf);
            float lim_neg = 0.3f * (0.5f * Wf);
            float rz = 1.f / z;
            float max_x = (-((-lim_neg) - cam.cx)) * rz, min_x = (-(lim_pos - cam.cx)) * rz;
            float max_y = (-((-lim_neg) - cam.cy)) * rz, min_y = (-(lim_pos - cam.cy)) * rz;
            p.clamp_lo[0] = J[0][2] < min_x; p.clamp_hi[0] = !p.clamp_lo[0] && J[0][2] > max_x;
            p.clamp_lo[1] = J[1][2] < min_y; p.clamp_hi[1] = !p.clamp_lo[1] && J[1][2] > max_y;
            J[0][2] = ssr_min(ssr_max(J[0][2], min_x), max_x);
            J[1][2] = ssr_min(ssr_max(J[1][2], min_y), max_y);
        }
    } else if (cam.model == OR_CAM_PINHOLE) {
        // persp_proj_3dgs, primitive_3dgs.slang:63-99; persp_proj_uv / _jac,
        // projection_utils.slang:331-375. The valid test (z < 0) is covered by the z <= 0 cull.
        float z2 = z * z;
        p.xy[0] = cam.fx * (x / z) + cam.cx;
        p.xy[1] = cam.fy * (y / z) + cam.cy;
        J[0][0] = (z / z2) * cam.fx; J[0][1] = 0.0f; J[0][2] = ((0.0f - x) / z2) * cam.fx;
        J[1][0] = 0.0f; J[1][1] = (z / z2) * cam.fy; J[1][2] = ((0.0f - y) / z2) * cam.fy;
        float Wf = (float)cam.W;
        float lim_pos = Wf + 0.3f * (0.5f * Wf);
        float lim_neg = 0.3f * (0.5f * Wf);
        float rz = 1.f / z;
        // the y limits reuse the x limits, as written at primitive_3dgs.slang:92-93
        float max_x = (-((-lim_neg) - cam.cx)) * rz, min_x = (-(lim_pos - cam.cx)) * rz;
        float max_y = (-((-lim_neg) - cam.cy)) * rz, min_y = (-(lim_pos - cam.cy)) * rz;
        p.clamp_lo[0] = J[0][2] < min_x; p.clamp_hi[0] = !p.clamp_lo[0] && J[0][2] > max_x;
        p.clamp_lo[1] = J[1][2] < min_y; p.clamp_hi[1] = !p.clamp_lo[1] && J[1][2] > max_y;
        J[0][2] = ssr_min(ssr_max(J[0][2], min_x), max_x);
        J[1][2] = ssr_min(ssr_max(J[1][2], min_y), max_y);
    } else {
        // equirect_proj_3dgs, primitive_3dgs.slang:194-211; projection_utils.slang:505-548
        float h2 = x * x + z * z;
        float h = ssr_sqrt(h2);
        float r2 = h2 + y * y;
        p.xy[0] = cam.fx * ssr_atan2(x, z) + cam.cx;
        p.xy[1] = cam.fy * ssr_atan2(y, h) + cam.cy;
        float hr2 = h * r2;
        J[0][0] = (z / h2) * cam.fx; J[0][1] = 0.0f; J[0][2] = ((0.0f - x) / h2) * cam.fx;
        J[1][0] = ((0.0f - x * y) / hr2) * cam.fy; J[1][1] = (h / r2) * cam.fy;
        J[1][2] = ((0.0f - z * y) / hr2) * cam.fy;
    }
    // cov2d = J covc J^T
    float jc[2][3];
    for (int i = 0; i < 2; i++)
        for (int j = 0; j < 3; j++)
            jc[i][j] = (J[i][0] * p.covc[0][j] + J[i][1] * p.covc[1][j]) + J[i][2] * p.covc[2][j];
    for (int i = 0; i < 2; i++)
        for (int j = 0; j < 2; j++)
            p.c2[i][j] = (jc[i][0] * J[j][0] + jc[i][1] * J[j][1]) + jc[i][2] * J[j][2];
    if (!assume_valid && (cam.model == OR_CAM_FISHEYE || cam.model == OR_CAM_EQUISOLID)) {
        // primitive_3dgs.slang:509-514: behind the lens (z < 0) yet still visibly opaque at the image
        // centre -- dropped; evaluated on the covariance before the blur
        const float m0 = p.xy[0] - cam.cx, m1 = p.xy[1] - cam.cy;
        const float idet = 1.0f / (p.c2[0][0] * p.c2[1][1] - p.c2[0][1] * p.c2[1][0]);
        const float i00 = p.c2[1][1] * idet, i01 = (-p.c2[0][1]) * idet, i10 = (-p.c2[1][0]) * idet, i11 = p.c2[0][0] * idet;
        const float q = (i00 * m0 + i01 * m1) * m0 + (i10 * m0 + i11 * m1) * m1;
        const float seen = p.opac * ssr_exp(-0.5f * q);
        if (z < 0.0f && seen > kAlphaThreshold) return p;
    }
    // add_blur, primitive_3dgs.slang:398-405,528-543: eps 0.3, or 0.1 in the antialiased variant, which also scales
    // the opacity by sqrt(max(0, det before / det after))
    const float eps2d = cam.aa ? 0.1f : 0.3f;
    p.det_orig = p.c2[0][0] * p.c2[1][1] - p.c2[0][1] * p.c2[1][0];
    p.c2o[0] = p.c2[0][0]; p.c2o[1] = p.c2[1][1];
    p.c2[0][0] = p.c2[0][0] + eps2d;
    p.c2[1][1] = p.c2[1][1] + eps2d;
    float det = p.c2[0][0] * p.c2[1][1] - p.c2[0][1] * p.c2[1][0];
    p.det_blur = det;
    if (!assume_valid && det <= 0.f) return p;
    p.sig = p.opac; p.comp = 1.0f;
    if (cam.aa) {
        p.comp = ssr_sqrt(ssr_max(0.0f, p.det_orig / det));
        p.opac = p.opac * p.comp;
    }
    float invdet = 1.0f / det;   // inverse(), projection_utils.slang:164-174
    p.conic[0] = p.c2[1][1] * invdet;
    p.conic[1] = (-p.c2[0][1]) * invdet;
    p.conic[2] = p.c2[0][0] * invdet;
    if (!assume_valid && p.opac < kAlphaThreshold) return p;
    float extend = ssr_min(3.33f, ssr_sqrt(2.0f * ssr_log(p.opac / kAlphaThreshold)));
    float rx = extend * ssr_sqrt(p.c2[0][0]);
    float ry = extend * ssr_sqrt(p.c2[1][1]);
    float xmin = p.xy[0] - rx, xmax = p.xy[0] + rx, ymin = p.xy[1] - ry, ymax = p.xy[1] + ry;
    if (!assume_valid && (xmax <= 0 || xmin >= (float)cam.W || ymax <= 0 || ymin >= (float)cam.H))
        return p;
    p.aabb[0] = xmin; p.aabb[1] = ymin; p.aabb[2] = xmax; p.aabb[3] = ymax;
    // get_sorting_depth, projection_utils.slang:1012-1029
    if (cam.model == OR_CAM_PINHOLE) p.sort_depth = z;
    else if (cam.model == OR_CAM_EQUIRECT) p.sort_depth = dot3(p.mc, p.mc);
    else p.sort_depth = ((z * z) * z) * z + ((1.0f / 512.0f) * (x * x + y * y)) * (x * x + y * y);
    float campos[3];
    for (int i = 0; i < 3; i++)
        campos[i] = -((cam.R[0][i] * cam.t[0] + cam.R[1][i] * cam.t[1]) + cam.R[2][i] * cam.t[2]);
    p.radius = view_radius(mean, ls, logit, campos);
    p.valid = true;
    return p;
}

// src/kernels/tile/IntersectTile.cu:34-53
inline void ellipse_range_bound(const float ic[3], float y0, float y1, float out[2]) {
    float a = ic[0], b = ic[1], c = ic[2];
    float ym = ((-b) / c) * ssr_sqrt(c / (a * c - b * b));
    float v0 = ssr_min(ssr_max(-ym, y0), y1);   // clamp(x,a,b) = x<a ? a : x>b ? b : x
    float v1 = ssr_min(ssr_max(ym, y0), y1);
    float bv0 = (-b) * v0, bv1 = (-b) * v1;
    float inv_a = 1.0f / a;
    out[0] = inv_a * (bv0 - ssr_sqrt(bv0 * bv0 - a * ((c * v0) * v0 - 1.f)));
    out[1] = inv_a * (bv1 + ssr_sqrt(bv1 * bv1 - a * ((c * v1) * v1 - 1.f)));
}

inline int clampi(int x, int a, int b) { return x < a ? a : (x > b ? b : x); }

struct TileGeom {
    bool visible;
    float xy[2];
    float ic[3];
    int xmin, xmax, ymin, ymax;   // tile range [min, max)
    bool by_rows;
};

// shared prologue of the count and write passes, IntersectTile.cu:124-164
TileGeom tile_geom(const float aabb[4], const float xy[2], const float conic[3], float opac,
                   int tile_w, int tile_h) {
    TileGeom g;
    g.visible = !(aabb[2] <= aabb[0] || aabb[3] <= aabb[1]);
    if (!g.visible) return g;
    g.xy[0] = xy[0]; g.xy[1] = xy[1];
    float k = 0.5f / ssr_log(opac / kAlphaThreshold);
    for (int i = 0; i < 3; i++) g.ic[i] = conic[i] * k;
    g.xmin = std::min(std::max(0, ssr_f2i_sat(ssr_floor((aabb[0] + 0.5f) / (float)kTile))), tile_w);
    g.ymin = std::min(std::max(0, ssr_f2i_sat(ssr_floor((aabb[1] + 0.5f) / (float)kTile))), tile_h);
    g.xmax = std::min(std::max(0, ssr_f2i_sat(ssr_ceil((aabb[2] + 0.5f) / (float)kTile))), tile_w);
    g.ymax = std::min(std::max(0, ssr_f2i_sat(ssr_ceil((aabb[3] + 0.5f) / (float)kTile))), tile_h);
    g.by_rows = (g.ymax - g.ymin) * kTile <= (g.xmax - g.xmin) * kTile;
    return g;
}

// Calls emit(tile_x, tile_y) for every tile the ellipse touches, in the reference's order.
// Count pass: IntersectTile.cu:55-101 (int casts); write pass: :198-247 (unsigned casts). With
// saturating NaN->0 conversion and the clamp to [min,max] both give the same interval.
template <class F>
void for_each_tile(const TileGeom& g, F&& emit) {
    float ic[3] = {g.ic[0], g.ic[1], g.ic[2]};
    if (g.by_rows) {
        for (int y = g.ymin; y < g.ymax; y++) {
            float y0 = (float)(y * kTile) - g.xy[1];
            float y1 = y0 + (float)kTile;
            float bd[2];
            ellipse_range_bound(ic, y0, y1, bd);
            int x0 = clampi(ssr_f2i_sat(ssr_floor((bd[0] + g.xy[0]) / (float)kTile)), g.xmin, g.xmax);
            int x1 = clampi(ssr_f2i_sat(ssr_ceil((bd[1] + g.xy[0]) / (float)kTile)), g.xmin, g.xmax);
            for (int x = x0; x < x1; x++) emit(x, y);
        }
    } else {
        float sw[3] = {ic[2], ic[1], ic[0]};
        for (int x = g.xmin; x < g.xmax; x++) {
            float x0 = (float)(x * kTile) - g.xy[0];
            float x1 = x0 + (float)kTile;
            float bd[2];
            ellipse_range_bound(sw, x0, x1, bd);
            int y0 = clampi(ssr_f2i_sat(ssr_floor((bd[0] + g.xy[1]) / (float)kTile)), g.ymin, g.ymax);
            int y1 = clampi(ssr_f2i_sat(ssr_ceil((bd[1] + g.xy[1]) / (float)kTile)), g.ymin, g.ymax);
            for (int y = y0; y < y1; y++) emit(x, y);
        }
    }
}

// src/core/Common.cuh:55-77
inline bool ellipse_box_overlap(const float ic[3], float x0, float x1, float y0, float y1) {
    float a = ic[0], b = ic[1], c = ic[2];
    float wx = (-b) / c, wy = (-b) / a;
    float u0 = ssr_min(ssr_max(x0 * wx, y0), y1);
    float u1 = ssr_min(ssr_max(x1 * wx, y0), y1);
    float v0 = ssr_min(ssr_max(y0 * wy, x0), x1);
    float v1 = ssr_min(ssr_max(y1 * wy, x0), x1);
    b = b * 2.0f;
    float mx = ssr_min(((a * x0) * x0 + (b * x0) * u0) + (c * u0) * u0,
                       ((a * x1) * x1 + (b * x1) * u1) + (c * u1) * u1);
    float my = ssr_min(((a * v0) * v0 + (b * v0) * y0) + (c * y0) * y0,
                       ((a * v1) * v1 + (b * v1) * y1) + (c * y1) * y1);
    float mc = ssr_max(ssr_max(x0, -x1), ssr_max(y0, -y1));
    return ssr_min(mc, ssr_min(mx, my) - 1.0f) < 0.f;
}

// micro-tile footprint test, RasterizationEval3DFwd_kernel.cuh:203-209 / ...Bwd_kernel.cuh:336-342
inline bool micro_hit(const float xy[2], const float conic[3], float opac, float bx0, float by0) {
    if (!(opac > kAlphaThreshold)) return false;
    float kk = 0.5f / ssr_log(opac / kAlphaThreshold);
    float ic[3] = {conic[0] * kk, conic[1] * kk, conic[2] * kk};
    return ellipse_box_overlap(ic, bx0 - xy[0], (bx0 + (float)kMicro) - xy[0], by0 - xy[1],
                               (by0 + (float)kMicro) - xy[1]);
}

struct Frag { float x, y, hx, cy, hz, cx, cz, opac, r, g, b, d; };

inline Frag load_frag(int32_t g, const float* xy, const float* depth, const float* conic,
                      const float* opac, const float* rgb) {
    Frag f;
    f.x = xy[2 * g]; f.y = xy[2 * g + 1];
    f.cx = conic[3 * g]; f.cy = conic[3 * g + 1]; f.cz = conic[3 * g + 2];
    f.hx = 0.5f * f.cx; f.hz = 0.5f * f.cz;
    f.opac = opac[g];
    f.r = rgb[3 * g]; f.g = rgb[3 * g + 1]; f.b = rgb[3 * g + 2];
    f.d = depth[g];
    return f;
}

// FragmentFwd::evaluate_alpha, src/primitives/Primitive3DGS.cuh:250-260.
// sigma = 0.5*(a dx^2 + c dy^2) + b dx dy, with the fused operations fixed as written here.
inline float eval_alpha(const Frag& f, float px, float py, float& dx, float& dy, float& vis,
                        float& sigma) {
    dx = f.x - px; dy = f.y - py;
    sigma = ssr_fma(f.hx * dx, dx, ssr_fma(f.hz * dy, dy, (f.cy * dx) * dy));
    vis = ssr_exp(-sigma);
    float alpha = ssr_min(0.999f, f.opac * vis);
    return sigma < 0.f ? 0.f : alpha;
}

}  // namespace

extern "C" {

int or_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
void or_set_num_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n > 0 ? n : 1);
#else
    (void)n;
#endif
}

void or_math(int op, int64_t n, const float* a, const float* b, float* out) {
    for (int64_t i = 0; i < n; i++) {
        switch (op) {
            case 0: out[i] = ssr_exp(a[i]); break;
            case 1: out[i] = ssr_log(a[i]); break;
            case 2: out[i] = ssr_atan2(a[i], b[i]); break;
            case 4: out[i] = ssr_adam_inv_bias1(a[i]); break;
            case 5: out[i] = ssr_adam_inv_bias2(a[i]); break;
            default: out[i] = ssr_sigmoid(a[i]); break;
        }
    }
}

void or_decode_sh(int64_t gid, const or_sh_source* sh, float* out45) { decode_sh(gid, sh, 15, out45); }

// Fused projection backward + Adam, fp32 state (src/kernels/optim/FusedProjectionBwdOptim_kernel.cuh:232-710
// with BLOCK_SIZE == 0, VALUE_BITS == 32, use_scale_agnostic_mean = color_trust_linear = false).
// The data gradient is or_projection_bwd's; the regularizers are the closed-form derivatives of
// src/shaders/per_splat_losses.slang:30-81; the effective-rank term (:3-15) is differentiated with the
// first-order arithmetic of include/ssr_camera.h (ssr_erank_reg_grad).
float or_erank_reg(const float* log_scales, float w, float w3, float* grad) {
    return ssr_erank_reg_grad(log_scales, w, w3, grad);
}

void or_quant_codec(int op, int64_t n, float* a, float* b, const float* mm, uint32_t* codes) {
    for (int64_t i = 0; i < n; i++) {
        if (op == 0) codes[i] = ssr_adamq_encode(a[i], b[i], mm);
        else if (op == 1) ssr_adamq_decode(codes[i], mm, a + i, b + i);
        else if (op == 2) codes[i] = ssr_q16_encode(a[i], mm[0], mm[1]);
        else if (op == 3) a[i] = ssr_q16_decode(codes[i], mm[0], mm[1]);
        else if (op == 4) codes[i] = ssr_adamq16_encode(a[i], b[i], mm);
        else ssr_adamq16_decode(codes[i], mm, a + i, b + i);
    }
}

void or_colour_map(int op, int64_t n, const float* x, float* y) {
    for (int64_t i = 0; i < n; i++)
        y[i] = op == 0 ? ssr_srgb_slope(x[i]) : op == 1 ? ssr_splat_dc_encode(x[i]) : ssr_splat_dc_decode(x[i]);
}

static void fused_optimizer_impl(int64_t N, int sh_degree,
    float* means, float* quats, float* log_scales, float* opacity_logits, float* features_dc, float* features_sh,
    const or_sh_quant_state* q, const or_non_sh_quant_state* nq,
    const or_camera* cam, const float* aabb,
    const float* v_xy, const float* v_sdepth, const float* v_conic, const float* v_opac, const float* v_srgb,
    const float* const* v_in, float* const* g1_in, float* const* g2_in, float* densify_score,
    const float* hyper, int32_t step, const int32_t* steps, const float* radii) {
    const int n_coef = sh_degree * (sh_degree + 2);
    // Quantized non-SH state (NonShQuantState, FusedProjectionBwdOptim_kernel.cuh:97-143,373-638): the moments of the
    // five non-SH tensors are decoded against each block's OLD bounds into fp32, the step below runs on those, and
    // afterwards each block's min / max of the new (u, log_s) become its NEW bounds, against which they are encoded.
    static const int kPrims[5] = {3, 4, 3, 1, 3};
    const int64_t n_blocks_ns = (N + 255) / 256;
    std::vector<float> dq1[5], dq2[5];
    float* g1[6];
    float* g2[6];
    for (int t = 0; t < 6; t++) { g1[t] = g1_in ? g1_in[t] : nullptr; g2[t] = g2_in ? g2_in[t] : nullptr; }
    if (nq) {
        for (int t = 0; t < 5; t++) {
            dq1[t].resize((size_t)N * kPrims[t]); dq2[t].resize((size_t)N * kPrims[t]);
            for (int64_t g = 0; g < N; g++)
                for (int i = 0; i < kPrims[t]; i++)
                    ssr_adamq16_decode(nq->packed[t][kPrims[t] * g + i], nq->bounds[t] + 4 * (g / 256), &dq1[t][kPrims[t] * g + i],
                                       &dq2[t][kPrims[t] * g + i]);
            g1[t] = dq1[t].data(); g2[t] = dq2[t].data();
        }
    }
    std::vector<float> vm((size_t)N * 3), vq((size_t)N * 4), vs((size_t)N * 3), vo((size_t)N), vd((size_t)N * 3),
        vsh((size_t)N * 45);
    or_sh_source src;
    memset(&src, 0, sizeof(src));
    src.codec = OR_SH_F32; src.sh_f32 = features_sh; src.num_sh_buffer = 15;
    if (q) {
        // the view-direction gradient is taken against the decoded coefficients
        // (FusedProjectionBwdOptim_kernel.cuh:289-310)
        src.codec = OR_SH_REF_Q16; src.sh_f32 = nullptr; src.packed = reinterpret_cast<const uint8_t*>(q->value_packed); src.bounds = q->value_bounds;
        src.num_sh_buffer = q->num_sh_buffer; src.bounds_stride = (int64_t)256 * 3 * q->num_sh_buffer;
    }
    or_projection_bwd(N, sh_degree, means, quats, log_scales, opacity_logits, features_dc, &src, cam, aabb, v_xy, v_sdepth,
                      v_conic, v_opac, v_srgb, vm.data(), vq.data(), vs.data(), vo.data(), vd.data(), vsh.data());
    const float lr_means = hyper[0], lr_quats = hyper[1], lr_scales = hyper[2], lr_opacs = hyper[3], lr_dc = hyper[4],
                lr_sh = hyper[5], max_ratio = hyper[6], scale_w = hyper[7], mcmc_o = hyper[8], mcmc_s = hyper[9],
                qnorm_w = hyper[10], sh_w = hyper[11], erank_w = hyper[12], erank_w3 = hyper[13];
    // colour trust region (FusedProjectionBwdOptim_kernel.cuh:551-596,651-705,774-794): per splat the slope of the
    // sRGB curve at its DC colour and the clip of its SH steps, from the parameters as they were
    const bool ctl = hyper[14] != 0.0f;
    const float eps_tr = hyper[15];
    // hyper[16] != 0: v_in[5] holds SH-gradient contributions that are already there (the other cameras of a batch,
    // which the reference sums inside its kernel, FusedProjectionBwdOptim_kernel.cuh:262-330) and is added; the
    // reference's own v_splats_world input carries none for SH, so the default leaves it unread
    const bool sh_in = hyper[16] != 0.0f && v_in && v_in[5];
    const float kSh0 = 0.28209479177387814f;
    std::vector<float> ctl_slope(ctl ? (size_t)N * 3 : 0), ctl_clip(ctl ? (size_t)N * 3 : 0);
    auto clip_step = [](float delta, float clip) {
        delta = ssr_min(ssr_max(delta, -clip), clip);
        return ssr_isfinite(delta) ? delta : 0.0f;
    };
    const float kBeta1 = 0.9f, kBeta2 = 0.999f, kEps = 1e-15f;
    const float sh_reg = sh_w * (1.0f / (float)(n_coef > 0 ? n_coef : 1));
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < N; g++) {
        float b1c, b2c;
        if (steps) {
            const float t = (float)steps[g];
            b1c = ssr_adam_inv_bias1(t);   // FusedProjectionBwdOptim_kernel.cuh:369-370, float constants
            b2c = ssr_adam_inv_bias2(t);
        } else {
            b1c = ssr_adam_inv_bias1((float)step);
            b2c = ssr_adam_inv_bias2((float)step);
        }
        auto adam = [&](float x, float v, float lr, float* g1p, float* g2p) {
            const float a = kBeta1 * *g1p + (1.f - kBeta1) * v;
            const float b = kBeta2 * *g2p + (1.f - kBeta2) * (v * v);
            *g1p = a; *g2p = b;
            return x - ((lr * b1c) * a) / (ssr_sqrt(b * b2c) + kEps);
        };
        auto vin = [&](int k, int64_t i) { return v_in && v_in[k] ? v_in[k][i] : 0.0f; };
        float gm[3], gq[4], gs[3], go, gd[3];
        for (int i = 0; i < 3; i++) {
            gm[i] = vin(0, 3 * g + i) + vm[3 * g + i];
            gs[i] = vin(2, 3 * g + i) + vs[3 * g + i];
            gd[i] = vin(4, 3 * g + i) + vd[3 * g + i];
        }
        for (int i = 0; i < 4; i++) gq[i] = vin(1, 4 * g + i) + vq[4 * g + i];
        go = vin(3, g) + vo[g];
        if (ctl) {
            const float inv_opac = 1.0f / ssr_max(ssr_sigmoid(opacity_logits[g]), 1e-12f);
            for (int c = 0; c < 3; c++) {
                const float c_dc = kSh0 * features_dc[3 * g + c] + 0.5f;
                ctl_slope[3 * g + c] = ssr_srgb_slope(c_dc);
                const float cc = ssr_max(c_dc, (1.0f / 255.0f) * (1.0f / 255.0f));
                ctl_clip[3 * g + c] = kSh0 * ssr_sqrt(((4.0f * eps_tr) * cc) * inv_opac);
            }
        }
        // SH (fp32 state; the quantized state is updated block by block below)
        for (int i = 0; !q && i < 3 * n_coef; i++) {
            float* x = features_sh + 45 * g + i;
            float v = (vsh[45 * g + i] + (sh_in ? v_in[5][45 * g + i] : 0.0f)) + sh_reg * *x;
            if (ctl) {
                v = v / ctl_slope[3 * g + i % 3];
                const float delta = adam(0.0f, v, lr_sh, g1[5] + 45 * g + i, g2[5] + 45 * g + i);
                *x = *x + clip_step(delta, ctl_clip[3 * g + i % 3]);
            } else {
                *x = adam(*x, v, lr_sh, g1[5] + 45 * g + i, g2[5] + 45 * g + i);
            }
        }
        const float* ls = log_scales + 3 * g;
        const float* q0 = quats + 4 * g;
        const float logit = opacity_logits[g];
        // regularizers
        const float sg = ssr_sigmoid(logit);
        go += mcmc_o * (sg * (1.0f - sg));
        const float ms = (mcmc_s * 1e-2f) / 3.0f;
        const float e[3] = {ssr_exp(ls[0]), ssr_exp(ls[1]), ssr_exp(ls[2])};
        int imax = 0, imin = 0;
        for (int i = 1; i < 3; i++) { if (e[i] > e[imax]) imax = i; if (e[i] < e[imin]) imin = i; }
        const float ratio = e[imax] / e[imin];
        const float rg = ratio > max_ratio ? scale_w * ratio : 0.0f;
        for (int i = 0; i < 3; i++) gs[i] += ms + (i == imax ? rg : 0.f) - (i == imin ? rg : 0.f);
        if (erank_w != 0.0f || erank_w3 != 0.0f) {   // erank_reg_3dgs, per_splat_losses.slang:3-15,101
            float ge[3];
            ssr_erank_reg_grad(ls, erank_w, erank_w3, ge);
            for (int i = 0; i < 3; i++) gs[i] += ge[i];
        }
        const float qn = ssr_sqrt((q0[0] * q0[0] + q0[1] * q0[1]) + (q0[2] * q0[2] + q0[3] * q0[3]));
        const float qg = qnorm_w * ((1.0f - 1.0f / qn) / qn);
        for (int i = 0; i < 4; i++) gq[i] += qg * q0[i];
        const float lim = 0.5f / 0.28209479177387814f;
        for (int i = 0; i < 3; i++)
            gd[i] += sh_w * (ssr_max(features_dc[3 * g + i] - lim, 0.0f) + ssr_min(features_dc[3 * g + i] + lim, 0.0f));
        const float smax = ssr_max(ssr_max(ls[0], ls[1]), ls[2]);
        // use_scale_agnostic_mean (FusedProjectionBwdOptim_kernel.cuh:519-534), from the parameters as they were:
        // num = apply_covar_to_vec(quat, exp(0.5 log_scale), v_mean) * sqrt(2 log(max(255 sigmoid(opacity), 1.00001)))
        // (projection_utils.slang:151-162, the rotation from the stored quaternion as it is), den = 0.6 radii
        float sa_num[3] = {0.f, 0.f, 0.f}, sa_den = 0.f;
        if (radii) {
            float Rm[3][3], M[3][3], cov[3][3];
            quat_to_rot(q0, Rm);
            const float hs[3] = {ssr_exp(0.5f * ls[0]), ssr_exp(0.5f * ls[1]), ssr_exp(0.5f * ls[2])};
            for (int i = 0; i < 3; i++)
                for (int j = 0; j < 3; j++) M[i][j] = Rm[i][j] * hs[j];
            for (int i = 0; i < 3; i++)
                for (int j = 0; j < 3; j++) cov[i][j] = (M[i][0] * M[j][0] + M[i][1] * M[j][1]) + M[i][2] * M[j][2];
            const float extent = ssr_sqrt(2.0f * ssr_log(ssr_max(255.0f * ssr_sigmoid(logit), 1.00001f)));
            for (int i = 0; i < 3; i++) sa_num[i] = ((cov[i][0] * gm[0] + cov[i][1] * gm[1]) + cov[i][2] * gm[2]) * extent;
            sa_den = radii[g] * 0.6f;
        }
        // scales
        float new_ls[3];
        for (int i = 0; i < 3; i++) new_ls[i] = adam(ls[i], gs[i], lr_scales, g1[2] + 3 * g + i, g2[2] + 3 * g + i);
        // quats, Riemannian
        {
            const float inv = 1.0f / qn;
            float q[4], v[4];
            for (int i = 0; i < 4; i++) q[i] = q0[i] * inv;
            const float d = (q[0] * gq[0] + q[1] * gq[1]) + (q[2] * gq[2] + q[3] * gq[3]);
            for (int i = 0; i < 4; i++) v[i] = gq[i] - d * q[i];
            for (int i = 0; i < 4; i++) q[i] = adam(q[i], v[i], lr_quats, g1[1] + 4 * g + i, g2[1] + 4 * g + i);
            const float minv = 1.0f / ssr_sqrt((q[0] * q[0] + q[1] * q[1]) + (q[2] * q[2] + q[3] * q[3]));
            for (int i = 0; i < 4; i++) quats[4 * g + i] = q[i] * minv;
        }
        for (int i = 0; i < 3; i++) log_scales[3 * g + i] = new_ls[i];
        opacity_logits[g] = adam(logit, go, lr_opacs, g1[3] + g, g2[3] + g);
        if (densify_score) densify_score[g] = ssr_exp(smax) * ssr_sqrt(dot3(gm, gm));
        for (int i = 0; i < 3; i++) {
            if (radii) {
                float* g1p = g1[0] + 3 * g + i;
                float* g2p = g2[0] + 3 * g + i;
                const float a = kBeta1 * *g1p + (1.f - kBeta1) * sa_num[i];
                const float b = kBeta2 * *g2p + (1.f - kBeta2) * (((gm[i] * gm[i]) * sa_den) * sa_den);
                *g1p = a; *g2p = b;
                means[3 * g + i] = means[3 * g + i] - ((lr_means * b1c) * a) / (ssr_sqrt(b * b2c) + kEps);
            } else {
                means[3 * g + i] = adam(means[3 * g + i], gm[i], lr_means, g1[0] + 3 * g + i, g2[0] + 3 * g + i);
            }
        }
        for (int i = 0; i < 3; i++) {
            if (ctl) {
                const float dc = features_dc[3 * g + i];
                const float delta = adam(0.0f, gd[i] / ctl_slope[3 * g + i], lr_dc, g1[4] + 3 * g + i, g2[4] + 3 * g + i);
                const float clip = kSh0 * ssr_sqrt((2.0f * eps_tr) / ssr_max(sg, 1e-12f));
                features_dc[3 * g + i] = ssr_splat_dc_decode(ssr_splat_dc_encode(dc) + clip_step(delta, clip));
            } else {
                features_dc[3 * g + i] = adam(features_dc[3 * g + i], gd[i], lr_dc, g1[4] + 3 * g + i, g2[4] + 3 * g + i);
            }
        }
    }
    if (nq) {
        for (int t = 0; t < 5; t++)
            for (int64_t blk = 0; blk < n_blocks_ns; blk++) {
                const int64_t c0 = blk * 256 * kPrims[t], c1 = std::min<int64_t>(N, blk * 256 + 256) * kPrims[t];
                float mm[4] = {1e30f, -1e30f, 1e30f, -1e30f};
                for (int64_t c = c0; c < c1; c++) {
                    float u, ls;
                    ssr_adamq_to_us(dq1[t][c], dq2[t][c], &u, &ls);
                    mm[0] = ssr_min(mm[0], u); mm[1] = ssr_max(mm[1], u);
                    mm[2] = ssr_min(mm[2], ls); mm[3] = ssr_max(mm[3], ls);
                }
                for (int k = 0; k < 4; k++) nq->bounds[t][4 * blk + k] = mm[k];
                for (int64_t c = c0; c < c1; c++) nq->packed[t][c] = ssr_adamq16_encode(dq1[t][c], dq2[t][c], mm);
            }
    }
    if (!q) return;
    // ---- SH coefficients and moments in the quantized state, FusedProjectionBwdOptim_kernel.cuh:709-1030 ----
    // Per block of 256 splats: decode moments and values against the block's OLD bounds, take the Adam step in
    // fp32, reduce min / max of the new (u, log_s) and of the new values over the block, store those as the NEW
    // bounds, encode against them. Coefficients above the active degree are re-encoded as zeros, and the new
    // bounds are widened to contain zero when there are any (:842-861, :925-938).
    const int64_t R = 3 * (int64_t)q->num_sh_buffer;
    const int64_t n_blocks = (N + 255) / 256;
#pragma omp parallel for schedule(static)
    for (int64_t blk = 0; blk < n_blocks; blk++) {
        const int64_t g0 = blk * 256, g1e = (g0 + 256 < N) ? g0 + 256 : N;
        const int n_here = (int)(g1e - g0);
        float old_mm[4], new_mm[4] = {1e30f, -1e30f, 1e30f, -1e30f};
        for (int k = 0; k < 4; k++) old_mm[k] = q->state_bounds[4 * blk + k];
        const float old_lo = q->value_bounds[2 * blk], old_hi = q->value_bounds[2 * blk + 1];
        float new_lo = 1e30f, new_hi = -1e30f;
        std::vector<float> ng1((size_t)n_here * 3 * n_coef), ng2(ng1.size()), nx(ng1.size());
        for (int s = 0; s < n_here; s++) {
            const int64_t g = g0 + s;
            float b1c, b2c;
            if (steps) {
                const float t = (float)steps[g];
                b1c = ssr_adam_inv_bias1(t);
                b2c = ssr_adam_inv_bias2(t);
            } else {
                b1c = ssr_adam_inv_bias1((float)step);
                b2c = ssr_adam_inv_bias2((float)step);
            }
            for (int i = 0; i < 3 * n_coef; i++) {
                const int64_t cell = R * g + i;
                float m1, m2;
                ssr_adamq_decode(q->state_packed[cell], old_mm, &m1, &m2);
                const float x = ssr_q16_decode(q->value_packed[cell], old_lo, old_hi);
                float v = (vsh[45 * g + i] + (sh_in ? v_in[5][45 * g + i] : 0.0f)) + sh_reg * x;
                if (ctl) v = v / ctl_slope[3 * g + i % 3];
                const float a = kBeta1 * m1 + (1.f - kBeta1) * v;
                const float b = kBeta2 * m2 + (1.f - kBeta2) * (v * v);
                float delta = 0.0f - ((lr_sh * b1c) * a) / (ssr_sqrt(b * b2c) + kEps);
                if (ctl) delta = clip_step(delta, ctl_clip[3 * g + i % 3]);
                const float xn = x + delta;
                const size_t o = (size_t)s * 3 * n_coef + i;
                ng1[o] = a; ng2[o] = b; nx[o] = xn;
                float u, ls;
                ssr_adamq_to_us(a, b, &u, &ls);
                new_mm[0] = ssr_min(new_mm[0], u); new_mm[1] = ssr_max(new_mm[1], u);
                new_mm[2] = ssr_min(new_mm[2], ls); new_mm[3] = ssr_max(new_mm[3], ls);
                new_lo = ssr_min(new_lo, xn); new_hi = ssr_max(new_hi, xn);
            }
            if (R > 3 * n_coef) {
                new_lo = ssr_min(new_lo, 0.0f); new_hi = ssr_max(new_hi, 0.0f);
                new_mm[0] = ssr_min(new_mm[0], 0.0f); new_mm[1] = ssr_max(new_mm[1], 0.0f);
                new_mm[2] = ssr_min(new_mm[2], 0.0f);
            }
        }
        for (int k = 0; k < 4; k++) q->state_bounds[4 * blk + k] = new_mm[k];
        q->value_bounds[2 * blk] = new_lo; q->value_bounds[2 * blk + 1] = new_hi;
        for (int s = 0; s < n_here; s++) {
            const int64_t g = g0 + s;
            for (int64_t i = 0; i < R; i++) {
                const int64_t cell = R * g + i;
                if (i < 3 * n_coef) {
                    const size_t o = (size_t)s * 3 * n_coef + (size_t)i;
                    q->state_packed[cell] = (uint16_t)ssr_adamq_encode(ng1[o], ng2[o], new_mm);
                    q->value_packed[cell] = (uint16_t)ssr_q16_encode(nx[o], new_lo, new_hi);
                } else {
                    q->state_packed[cell] = (uint16_t)ssr_adamq_encode(0.0f, 0.0f, new_mm);
                    q->value_packed[cell] = (uint16_t)ssr_q16_encode(0.0f, new_lo, new_hi);
                }
            }
        }
    }
}

void or_fused_projection_bwd_optimizer(int64_t N, int sh_degree,
    float* means, float* quats, float* log_scales, float* opacity_logits, float* features_dc, float* features_sh,
    const or_camera* cam, const float* aabb,
    const float* v_xy, const float* v_sdepth, const float* v_conic, const float* v_opac, const float* v_srgb,
    const float* const* v_in, float* const* g1, float* const* g2, float* densify_score,
    const float* hyper, int32_t step, const int32_t* steps, const float* radii) {
    fused_optimizer_impl(N, sh_degree, means, quats, log_scales, opacity_logits, features_dc, features_sh, nullptr, nullptr, cam, aabb,
                         v_xy, v_sdepth, v_conic, v_opac, v_srgb, v_in, g1, g2, densify_score, hyper, step, steps, radii);
}

void or_fused_projection_bwd_optimizer_q(int64_t N, int sh_degree,
    float* means, float* quats, float* log_scales, float* opacity_logits, float* features_dc, const or_sh_quant_state* q,
    const or_non_sh_quant_state* nq,
    const or_camera* cam, const float* aabb,
    const float* v_xy, const float* v_sdepth, const float* v_conic, const float* v_opac, const float* v_srgb,
    const float* const* v_in, float* const* g1, float* const* g2, float* densify_score,
    const float* hyper, int32_t step, const int32_t* steps, const float* radii) {
    fused_optimizer_impl(N, sh_degree, means, quats, log_scales, opacity_logits, features_dc, nullptr, q, nq, cam, aabb,
                         v_xy, v_sdepth, v_conic, v_opac, v_srgb, v_in, g1, g2, densify_score, hyper, step, steps, radii);
}


// QuantizedTensor<BITS,256>::encode_v with block-reduced bounds, src/core/Tensor.h:1364-1392
void or_quantize_ref(int bits, int64_t n_cells, int64_t stride, const float* v, uint8_t* packed,
                     float* bounds) {
    const float qmax = bits == 16 ? 65535.0f : 255.0f;
    int64_t nb = (n_cells + stride - 1) / stride;
    for (int64_t b = 0; b < nb; b++) {
        int64_t lo_i = b * stride, hi_i = std::min(n_cells, lo_i + stride);
        float lo = v[lo_i], hi = v[lo_i];
        for (int64_t i = lo_i; i < hi_i; i++) { lo = std::min(lo, v[i]); hi = std::max(hi, v[i]); }
        bounds[2 * b] = lo; bounds[2 * b + 1] = hi;
        float range = ssr_max(hi - lo, 1e-30f);
        for (int64_t i = lo_i; i < hi_i; i++) {
            float qf = std::round(qmax * (v[i] - lo) / range);
            qf = ssr_min(ssr_max(qf, 0.0f), qmax);
            if (bits == 16) reinterpret_cast<uint16_t*>(packed)[i] = (uint16_t)qf;
            else packed[i] = (uint8_t)qf;
        }
    }
}

void or_quantize_i8_f16(int64_t N, int cells, const float* v, int8_t* codes, uint16_t* scale_f16) {
    for (int64_t g = 0; g < N; g++) {
        float amax = 0.0f;
        for (int i = 0; i < cells; i++) amax = std::max(amax, std::fabs(v[g * cells + i]));
        uint16_t h = float_to_half_rn(amax / 127.0f);
        if ((h & 0x7fff) == 0 && amax > 0.0f) h = 1;   // smallest subnormal rather than zero
        scale_f16[g] = h;
        float s = half_to_float(h);
        for (int i = 0; i < cells; i++) {
            float q = s > 0.0f ? std::nearbyint(v[g * cells + i] / s) : 0.0f;
            q = std::min(std::max(q, -127.0f), 127.0f);
            codes[g * cells + i] = (int8_t)q;
        }
    }
}

// projection_fused_fwd_kernel, src/kernels/projection/ProjectionFwd_kernel.cuh:17-111, with
// World::project (src/primitives/Primitive3DGS.cuh:56-110) inlined.
int64_t or_projection_fwd(int64_t N, int sh_degree, const float* means, const float* quats,
    const float* log_scales, const float* opacity_logits, const float* features_dc,
    const or_sh_source* sh, const or_camera* camera, float* aabb, float* sort_depth, float* radii,
    float* xy, float* depth, float* conic, float* opac, float* rgb) {
    const Cam cam = load_cam(camera);
    const int n_coef = sh_degree * (sh_degree + 2);
    int64_t visible = 0;
#pragma omp parallel for schedule(static) reduction(+ : visible)
    for (int64_t g = 0; g < N; g++) {
        Proj p = project(cam, means + 3 * g, quats + 4 * g, log_scales + 3 * g, opacity_logits[g], false);
        float col[3] = {0, 0, 0};
        float bb[4] = {p.aabb[0], p.aabb[1], p.aabb[2], p.aabb[3]};
        if (bb[2] > bb[0] && bb[3] > bb[1]) {
            float coef[45];
            decode_sh(g, sh, n_coef, coef);
            float dir[3];
            view_dir(cam, means + 3 * g, dir);
            ShBasis b = sh_basis(sh_degree, dir);
            float raw[3];
            sh_color_raw(sh_degree, b, features_dc + 3 * g, coef, raw);
            // max(rgb + 0.5, 0), harmonics.slang:1055-1066
            for (int c = 0; c < 3; c++) col[c] = ssr_max(raw[c] + 0.5f, 0.0f);
        }
        bb[0] = ssr_min(ssr_max(bb[0], 0.0f), (float)cam.W - 1.0f);
        bb[1] = ssr_min(ssr_max(bb[1], 0.0f), (float)cam.H - 1.0f);
        bb[2] = ssr_min(ssr_max(bb[2], 0.0f), (float)cam.W - 1.0f);
        bb[3] = ssr_min(ssr_max(bb[3], 0.0f), (float)cam.H - 1.0f);
        if (bb[2] - bb[0] > 1e-3f && bb[3] - bb[1] > 1e-3f) {
            xy[2 * g] = p.xy[0]; xy[2 * g + 1] = p.xy[1];
            depth[g] = p.depth;
            for (int c = 0; c < 3; c++) { conic[3 * g + c] = p.conic[c]; rgb[3 * g + c] = col[c]; }
            opac[g] = p.opac;
            for (int c = 0; c < 4; c++) aabb[4 * g + c] = bb[c];
            sort_depth[g] = p.sort_depth;
            radii[g] = ssr_max(radii[g], p.radius);   // atomicMax over cameras
            visible++;
        } else {
            for (int c = 0; c < 4; c++) aabb[4 * g + c] = 0.0f;
            sort_depth[g] = 0.0f;
        }
    }
    return visible;
}

// intersect_tile_kernel<count=true, ellipse=true>, src/kernels/tile/IntersectTile.cu:104-186;
// tile_active (may be NULL): tiles marked 0 are not counted (:62,76-80,95-98)
void or_tile_count_masked(int64_t N, const float* aabb, const float* xy, const float* conic,
    const float* opac, uint32_t width, uint32_t height, const int32_t* tile_active, int64_t* tiles_per_splat) {
    const int tw = (int)((width + kTile - 1) / kTile), th = (int)((height + kTile - 1) / kTile);
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < N; g++) {
        TileGeom tg = tile_geom(aabb + 4 * g, xy + 2 * g, conic + 3 * g, opac[g], tw, th);
        int64_t n = 0;
        if (tg.visible) for_each_tile(tg, [&](int x, int y) { if (!tile_active || tile_active[(int64_t)y * tw + x]) n++; });
        tiles_per_splat[g] = n;
    }
}
void or_tile_count(int64_t N, const float* aabb, const float* xy, const float* conic,
    const float* opac, uint32_t width, uint32_t height, int64_t* tiles_per_splat) {
    or_tile_count_masked(N, aabb, xy, conic, opac, width, height, nullptr, tiles_per_splat);
}

// tile_active_kernel, src/kernels/tile/IntersectTile.cu:316-347, with nearest_sample_b
// (src/core/Interpolation.cuh:108-120); kMaskPad = 1 (IntersectTile.cu:311)
void or_compute_tile_active(const uint8_t* mask, int32_t h_mask, int32_t w_mask, uint32_t width, uint32_t height,
    int32_t* tile_active) {
    const int tw = (int)((width + kTile - 1) / kTile), th = (int)((height + kTile - 1) / kTile);
    const int W = (int)width, H = (int)height;
    for (int ty = 0; ty < th; ty++)
        for (int tx = 0; tx < tw; tx++) {
            bool live = false;
            for (int dy = -1; dy < kTile + 1 && !live; ++dy) {
                const int y = ty * kTile + dy;
                if (y >= H) break;
                if (y < 0) continue;
                for (int dx = -1; dx < kTile + 1; ++dx) {
                    const int x = tx * kTile + dx;
                    if (x >= W) break;
                    if (x < 0) continue;
                    const float u = (((float)x + 0.5f) * (float)w_mask) / (float)W - 0.5f;
                    const float v = (((float)y + 0.5f) * (float)h_mask) / (float)H - 0.5f;
                    const int sx = std::max(0, std::min(w_mask - 1, ssr_f2i_sat(ssr_floor(u + 0.5f))));
                    const int sy = std::max(0, std::min(h_mask - 1, ssr_f2i_sat(ssr_floor(v + 0.5f))));
                    if (mask[(size_t)sy * w_mask + sx]) { live = true; break; }
                }
            }
            tile_active[ty * tw + tx] = live ? 1 : 0;
        }
}

void or_inclusive_sum_i64(int64_t n, const int64_t* in, int64_t* out) {
    int64_t s = 0;
    for (int64_t i = 0; i < n; i++) { s += in[i]; out[i] = s; }
}

// intersect_tile_kernel<count=false, ellipse=true>, IntersectTile.cu:188-267
int64_t or_tile_write(int64_t N, const float* aabb, const float* sort_depth, const float* xy,
    const float* conic, const float* opac, const int64_t* cum, uint32_t width, uint32_t height,
    int64_t* isect_ids, int32_t* flatten_ids) {
    return or_tile_write_masked(N, aabb, sort_depth, xy, conic, opac, cum, width, height, nullptr, isect_ids, flatten_ids);
}
// tile_active (may be NULL): skipped tiles are left out (IntersectTile.cu:225,240)
int64_t or_tile_write_masked(int64_t N, const float* aabb, const float* sort_depth, const float* xy,
    const float* conic, const float* opac, const int64_t* cum, uint32_t width, uint32_t height,
    const int32_t* tile_active, int64_t* isect_ids, int32_t* flatten_ids) {
    const int tw = (int)((width + kTile - 1) / kTile), th = (int)((height + kTile - 1) / kTile);
    int64_t pads = 0;
#pragma omp parallel for schedule(static) reduction(+ : pads)
    for (int64_t g = 0; g < N; g++) {
        int64_t cur = g == 0 ? 0 : cum[g - 1];
        const int64_t end = cum[g];
        TileGeom tg = tile_geom(aabb + 4 * g, xy + 2 * g, conic + 3 * g, opac[g], tw, th);
        if (tg.visible) {
            uint32_t du = ssr_f2u(ssr_fabs(sort_depth[g]));
            du = (du >> 31) ? ~du : (du ^ 0x80000000u);
            for_each_tile(tg, [&](int x, int y) {
                if (tile_active && !tile_active[(int64_t)y * tw + x]) return;
                if (cur < end) {
                    int64_t tile_id = (int64_t)y * tw + (int64_t)x;
                    isect_ids[cur] = (int64_t)(((uint64_t)tile_id << 32) | (uint64_t)du);
                    flatten_ids[cur] = (int32_t)g;
                    cur++;
                }
            });
        }
        while (cur < end) {   // IntersectTile.cu:261-266
            isect_ids[cur] = (int64_t)0xffffffffull;
            flatten_ids[cur] = (int32_t)g;
            cur++; pads++;
        }
    }
    return pads;
}

// sort_pairs contract, src/backend/common/SortScan.h:53-56; checked in the reference against
// std::stable_sort on the masked key (src/backend/vulkan/tests/vk_sortscan_test.cpp:67-80).
void or_sort_pairs(int64_t n, const int64_t* keys_in, const int32_t* vals_in, int begin_bit,
    int end_bit, int64_t* keys_out, int32_t* vals_out) {
    std::vector<int64_t> idx((size_t)n);
    std::iota(idx.begin(), idx.end(), (int64_t)0);
    const int nb = end_bit - begin_bit;
    const uint64_t mask = nb >= 64 ? ~0ull : (((1ull << nb) - 1) << begin_bit);
    std::stable_sort(idx.begin(), idx.end(), [&](int64_t a, int64_t b) {
        return ((uint64_t)keys_in[a] & mask) < ((uint64_t)keys_in[b] & mask);
    });
    for (int64_t i = 0; i < n; i++) { keys_out[i] = keys_in[idx[i]]; vals_out[i] = vals_in[idx[i]]; }
}

// intersect_offset_kernel, IntersectTile.cu:271-307; zero-filled when n_isects == 0 (:448-451)
void or_tile_offsets(int64_t n, const int64_t* ids, uint32_t n_tiles, int32_t* offsets) {
    if (n == 0) { for (uint32_t i = 0; i < n_tiles; i++) offsets[i] = 0; return; }
    for (int64_t idx = 0; idx < n; idx++) {
        int64_t tile = ids[idx] >> 32;
        if (idx == 0) for (int64_t i = 0; i < tile + 1; i++) offsets[i] = 0;
        if (idx == n - 1) for (int64_t i = tile + 1; i < (int64_t)n_tiles; i++) offsets[i] = (int32_t)n;
        if (idx > 0) {
            int64_t prev = ids[idx - 1] >> 32;
            if (prev != tile) for (int64_t i = prev + 1; i < tile + 1; i++) offsets[i] = (int32_t)idx;
        }
    }
}

// rasterize_to_pixels_fwd_kernel (IS_EVAL3D=0, dist_type=None, no median),
// src/kernels/raster/RasterizationEval3DFwd_kernel.cuh:86-313
void or_raster_fwd(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    float* out_rgb, float* out_depth, float* out_T, int32_t* out_last_ids, int64_t* stats) {
    or_raster_fwd_ex(N, xy, depth, conic, opac, rgb, width, height, tile_offsets, flatten_ids, n_isects, out_rgb, out_depth,
                     out_T, out_last_ids, stats, 0, nullptr, nullptr, nullptr);
}

// The same kernel with its variants (RasterizationEval3DFwd_kernel.cuh:143-148,245-307):
// dist_type 1 (D) / 2 (RGB_D): the depth channel is accumulated as ln(max(z, 1e-6)), second moments
// S = sum w c^2 are accumulated next to C = sum w c, the distortion image D = W S - C^2 (W = 1 - T)
// is written for the active channels and the rendered depth becomes exp(C_lnz / W).
// out_median (non-NULL): depth at which the post-splat transmittance crosses 1/2, interpolated
// linearly in ln T between the two bracketing splats (0 when it never does).
void or_raster_fwd_ex(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    float* out_rgb, float* out_depth, float* out_T, int32_t* out_last_ids, int64_t* stats,
    int dist_type, float* out_dist_rgb, float* out_dist_depth, float* out_median) {
    (void)N;
    const bool dist = dist_type != 0, dist_rgb = dist_type == 2;
    const int tw = (int)((width + kTile - 1) / kTile), th = (int)((height + kTile - 1) / kTile);
    const int n_tiles = tw * th;
    int64_t kf = 0, kb = 0, vis_f = 0, vis_b = 0, prod_b = 0;
#pragma omp parallel for schedule(dynamic, 4) reduction(+ : kf, kb, vis_f, vis_b, prod_b)
    for (int tile = 0; tile < n_tiles; tile++) {
        const int ty = tile / tw, tx = tile % tw;
        const int32_t start = tile_offsets[tile];
        const int32_t end = (tile == n_tiles - 1) ? (int32_t)n_isects : tile_offsets[tile + 1];
        std::vector<Frag> frags((size_t)std::max(0, end - start));
        std::vector<uint8_t> hits(frags.size());
        for (int32_t i = start; i < end; i++) {
            int32_t g = flatten_ids[i];
            frags[i - start] = load_frag(g, xy, depth, conic, opac, rgb);
            uint8_t m = 0;
            for (int mt = 0; mt < 4; mt++) {
                float bx0 = (float)(tx * kTile + (mt & 1) * kMicro), by0 = (float)(ty * kTile + (mt >> 1) * kMicro);
                if (micro_hit(xy + 2 * g, conic + 3 * g, opac[g], bx0, by0)) m |= (uint8_t)(1u << mt);
            }
            hits[i - start] = m;
        }
        int32_t max_eval = start - 1, max_last = start - 1;
        bool any_pixel = false;
        int32_t mt_eval[4] = {start - 1, start - 1, start - 1, start - 1}, mt_last[4] = {-1, -1, -1, -1};
        std::vector<uint8_t> used(frags.size(), 0);   // bit m: some pixel of sub-tile m composited it
        for (int py_ = 0; py_ < kTile; py_++) {
            for (int px_ = 0; px_ < kTile; px_++) {
                const uint32_t i = ty * kTile + py_, j = tx * kTile + px_;
                if (i >= height || j >= width) continue;
                any_pixel = true;
                const int mt = (py_ / kMicro) * 2 + (px_ / kMicro);
                const float px = (float)j + 0.5f, py = (float)i + 0.5f;
                float T = 1.0f, cr = 0, cg = 0, cb = 0, cd = 0;
                float s2r = 0, s2g = 0, s2b = 0, s2d = 0;
                float median = 0.0f, med_prev_z = 0.0f, med_prev_T = 1.0f;
                uint32_t cur_idx = 0;
                int32_t last_eval = start - 1;
                for (int32_t k = start; k < end; k++) {
                    if (!((hits[k - start] >> mt) & 1)) continue;
                    const Frag& f = frags[k - start];
                    float dx, dy, vis, sigma;
                    float alpha = eval_alpha(f, px, py, dx, dy, vis, sigma);
                    last_eval = k;
                    if (alpha <= kAlphaThreshold) continue;
                    const float next_T = T * (1.0f - alpha);
                    if (out_median) {   // before the 1e-4 early-out, RasterizationEval3DFwd_kernel.cuh:245-259
                        if (med_prev_T >= 0.5f && next_T < 0.5f) {
                            const float a = ssr_log(med_prev_T), b = ssr_log(next_T), d = b - a;
                            const float fr = (ssr_fabs(d) > 1e-20f) ? (-0.6931471805599453f - a) / d : 0.0f;
                            median = med_prev_z + (f.d - med_prev_z) * fr;
                        }
                        med_prev_T = next_T;
                        med_prev_z = f.d;
                    }
                    if (next_T > 1e-4f) {
                        const float w = alpha * T;
                        const float zd = dist ? ssr_log(ssr_max(f.d, 1e-6f)) : f.d;
                        if (dist) {
                            if (dist_rgb) {
                                s2r = ssr_fma(f.r * f.r, w, s2r); s2g = ssr_fma(f.g * f.g, w, s2g); s2b = ssr_fma(f.b * f.b, w, s2b);
                            }
                            s2d = ssr_fma(zd * zd, w, s2d);
                        }
                        cr = ssr_fma(f.r, w, cr); cg = ssr_fma(f.g, w, cg); cb = ssr_fma(f.b, w, cb);
                        cd = ssr_fma(zd, w, cd);
                        cur_idx = (uint32_t)k;
                        T = next_T;
                        used[k - start] |= (uint8_t)(1u << mt);
                    } else {
                        break;   // done: the crossing splat is not added
                    }
                }
                // a pixel that never terminates looks at the whole range
                const int64_t pid = (int64_t)i * width + j;
                out_T[pid] = T;
                const float invW = 1.0f / ssr_max(1.0f - T, 1e-10f);
                out_rgb[3 * pid] = cr; out_rgb[3 * pid + 1] = cg; out_rgb[3 * pid + 2] = cb;
                if (out_median) out_median[pid] = median;
                if (dist) {   // D = W S - C^2 on the raw accumulators, :291-295
                    const float W = 1.0f - T;
                    if (dist_rgb) {
                        out_dist_rgb[3 * pid] = s2r * W - cr * cr;
                        out_dist_rgb[3 * pid + 1] = s2g * W - cg * cg;
                        out_dist_rgb[3 * pid + 2] = s2b * W - cb * cb;
                    }
                    out_dist_depth[pid] = s2d * W - cd * cd;
                    out_depth[pid] = ssr_exp(cd * invW);
                } else {
                    out_depth[pid] = cd * invW;
                }
                out_last_ids[pid] = (int32_t)cur_idx;
                max_eval = std::max(max_eval, last_eval);
                max_last = std::max(max_last, (int32_t)cur_idx);
                mt_eval[mt] = std::max(mt_eval[mt], last_eval);
                mt_last[mt] = std::max(mt_last[mt], (int32_t)cur_idx);
            }
        }
        for (int32_t k = start; k < end; k++)
            for (int mt = 0; mt < 4; mt++) {
                if (!((hits[k - start] >> mt) & 1)) continue;
                if (k <= mt_eval[mt]) vis_f++;
                if (k <= mt_last[mt]) vis_b++;
                if ((used[k - start] >> mt) & 1) prod_b++;
            }
        if (any_pixel && end > start) {
            kf += std::max(0, max_eval - start + 1);
            kb += std::max(0, std::min(max_last, end - 1) - start + 1);
        }
    }
    // [2..4]: (splat, 8x8 sub-tile) visits of the forward, of the backward, and those of the
    // backward in which at least one pixel composited the splat
    if (stats) { stats[0] = kf; stats[1] = kb; stats[2] = vis_f; stats[3] = vis_b; stats[4] = prod_b; }
}

// Lane statistics of the compositing backward (a measurement aid, not a restatement of the reference):
// how many of the pixels a (splat, pixel-block) visit covers actually composite the splat (alpha > 1/255
// and sorted index <= the pixel's last_id), for square blocks of 8, 4 and 2 pixels inside the 8x8
// sub-tiles the reference's footprint test keeps. A block is visited when the sub-tile test passes,
// the sorted index does not exceed the largest last_id of the block's sub-tile, and the ellipse
// alpha >= 1/255 reaches the box of the block's pixel centres.
// out[0..2] = visits at block size 8, 4, 2; out[3] = compositing (pixel, splat) pairs;
// out[4..6] = visits with at least one compositing pixel, per block size.
void or_raster_lane_stats(const float* xy, const float* depth, const float* conic, const float* opac, const float* rgb,
    uint32_t width, uint32_t height, const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    const int32_t* last_ids, int64_t* out) {
    const int tw = (int)((width + kTile - 1) / kTile), th = (int)((height + kTile - 1) / kTile);
    const int n_tiles = tw * th;
    int64_t v8 = 0, v4 = 0, v2 = 0, pairs = 0, p8 = 0, p4 = 0, p2 = 0;
#pragma omp parallel for schedule(dynamic, 4) reduction(+ : v8, v4, v2, pairs, p8, p4, p2)
    for (int tile = 0; tile < n_tiles; tile++) {
        const int ty = tile / tw, tx = tile % tw;
        const int32_t start = tile_offsets[tile];
        const int32_t end = (tile == n_tiles - 1) ? (int32_t)n_isects : tile_offsets[tile + 1];
        int32_t mt_last[4] = {-1, -1, -1, -1};
        for (int py_ = 0; py_ < kTile; py_++)
            for (int px_ = 0; px_ < kTile; px_++) {
                const uint32_t i = ty * kTile + py_, j = tx * kTile + px_;
                if (i >= height || j >= width) continue;
                const int mt = (py_ / kMicro) * 2 + (px_ / kMicro);
                mt_last[mt] = std::max(mt_last[mt], last_ids[(int64_t)i * width + j]);
            }
        for (int32_t k = start; k < end; k++) {
            const int32_t g = flatten_ids[k];
            const Frag f = load_frag(g, xy, depth, conic, opac, rgb);
            if (!(f.opac > kAlphaThreshold)) continue;
            const float kk = 0.5f / ssr_log(f.opac / kAlphaThreshold);
            const float ic[3] = {f.cx * kk, f.cy * kk, f.cz * kk};
            for (int mt = 0; mt < 4; mt++) {
                if (k > mt_last[mt]) continue;
                const int ox = tx * kTile + (mt & 1) * kMicro, oy = ty * kTile + (mt >> 1) * kMicro;
                if (!micro_hit(xy + 2 * g, conic + 3 * g, f.opac, (float)ox, (float)oy)) continue;
                bool act[8][8];
                for (int y = 0; y < 8; y++)
                    for (int x = 0; x < 8; x++) {
                        const uint32_t i = oy + y, j = ox + x;
                        act[y][x] = false;
                        if (i >= height || j >= width) continue;
                        float dx, dy, vis, sigma;
                        const float alpha = eval_alpha(f, (float)j + 0.5f, (float)i + 0.5f, dx, dy, vis, sigma);
                        act[y][x] = alpha > kAlphaThreshold && k <= last_ids[(int64_t)i * width + j];
                    }
                for (int bs = 8; bs >= 2; bs >>= 1) {
                    for (int by = 0; by < 8; by += bs)
                        for (int bx = 0; bx < 8; bx += bs) {
                            const float x0 = (float)(ox + bx) + 0.5f - f.x, y0 = (float)(oy + by) + 0.5f - f.y;
                            if (bs < 8 && !ellipse_box_overlap(ic, x0, x0 + (float)(bs - 1), y0, y0 + (float)(bs - 1))) continue;
                            int n_act = 0;
                            for (int y = by; y < by + bs; y++)
                                for (int x = bx; x < bx + bs; x++) n_act += act[y][x] ? 1 : 0;
                            if (bs == 8) { v8++; pairs += n_act; p8 += n_act > 0; }
                            else if (bs == 4) { v4++; p4 += n_act > 0; }
                            else { v2++; p2 += n_act > 0; }
                        }
                }
            }
        }
    }
    out[0] = v8; out[1] = v4; out[2] = v2; out[3] = pairs; out[4] = p8; out[5] = p4; out[6] = p2;
}

// rasterize_to_pixels_bwd_kernel (IS_EVAL3D=0, dist_type=None, no median, no accum weights),
// src/kernels/raster/RasterizationEval3DBwd_kernel.cuh:107-584, fragment VJPs from
// src/primitives/Primitive3DGS.cuh:262-300. Partial sums are formed per (splat, 8x8 sub-tile)
// as the reference does before its atomics, then added in sorted-pair order.
void or_raster_bwd(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    const float* render_T, const int32_t* last_ids, const float* render_depth,
    const float* v_rgb, const float* v_depth, const float* v_T,
    float* v_xy, float* v_sdepth, float* v_conic, float* v_opac, float* v_srgb, double* abs_terms) {
    or_raster_bwd_ex(N, xy, depth, conic, opac, rgb, width, height, tile_offsets, flatten_ids, n_isects, render_T, last_ids,
                     render_depth, v_rgb, v_depth, v_T, v_xy, v_sdepth, v_conic, v_opac, v_srgb, abs_terms,
                     0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, nullptr, nullptr, 0, nullptr);
}

// The same kernel with its variants (RasterizationEval3DBwd_kernel.cuh:150-172,207-257,268-279,433-550,574-585):
// depth distortion / median / per-splat accumulation of a pixel weight map. gaussian_ids (packed
// mode, may be NULL) maps a screen row to the world row that accum_weight is indexed by; with
// accum_mode 3 (Avg) accum_weight holds n_world numerators followed by n_world denominators.
void or_raster_bwd_ex(int64_t N, const float* xy, const float* depth, const float* conic,
    const float* opac, const float* rgb, uint32_t width, uint32_t height,
    const int32_t* tile_offsets, const int32_t* flatten_ids, int64_t n_isects,
    const float* render_T, const int32_t* last_ids, const float* render_depth,
    const float* v_rgb, const float* v_depth, const float* v_T,
    float* v_xy, float* v_sdepth, float* v_conic, float* v_opac, float* v_srgb, double* abs_terms,
    int dist_type, const float* render_rgb, const float* dist_rgb_img, const float* dist_depth_img,
    const float* v_dist_rgb, const float* v_dist_depth, const float* v_median,
    int accum_mode, const float* accum_map, const int32_t* gaussian_ids, int64_t n_world, float* accum_weight) {
    const bool dist = dist_type != 0, dist_rgb = dist_type == 2;
    std::vector<float> awpart(accum_mode ? (size_t)n_isects * 2 : 0, 0.0f);
    const int tw = (int)((width + kTile - 1) / kTile), th = (int)((height + kTile - 1) / kTile);
    const int n_tiles = tw * th;
    std::vector<float> part((size_t)n_isects * 10, 0.0f);
    std::vector<double> apart(abs_terms ? (size_t)n_isects * 10 : 0, 0.0);
#pragma omp parallel for schedule(dynamic, 4)
    for (int tile = 0; tile < n_tiles; tile++) {
        const int ty = tile / tw, tx = tile % tw;
        const int32_t start = tile_offsets[tile];
        const int32_t end = (tile == n_tiles - 1) ? (int32_t)n_isects : tile_offsets[tile + 1];
        if (end <= start) continue;
        for (int mt = 0; mt < 4; mt++) {
            const int bx = tx * kTile + (mt & 1) * kMicro, by = ty * kTile + (mt >> 1) * kMicro;
            // per-pixel state, RasterizationEval3DBwd_kernel.cuh:186-232
            float T1[64], vT1[64], vc[64][4];
            int32_t bin_final[64];
            float Cc[64][4], Sc[64][4], vD[64][4], Wd[64], amap[64];
            float med_v[64], pend_zgrad[64], pend_zfar[64], pend_Tfar[64];
            int undo_steps[64] = {0};   // per pixel: how many times T has been divided by (1 - alpha) so far
            for (int p = 0; p < 64; p++) {
                const int pxi = bx + p % kMicro, pyi = by + p / kMicro;
                const bool inside = pxi < (int)width && pyi < (int)height;
                const int64_t pid = (int64_t)pyi * width + pxi;
                bin_final[p] = inside ? last_ids[pid] : -1;
                float Tf = inside ? render_T[pid] : 0.0f;
                float vT = inside ? v_T[pid] : 0.0f;
                float vr = inside ? v_rgb[3 * pid] : 0.f, vg = inside ? v_rgb[3 * pid + 1] : 0.f,
                      vb = inside ? v_rgb[3 * pid + 2] : 0.f, vd = inside ? v_depth[pid] : 0.f;
                float inv_alpha = 1.0f / ssr_max(1.0f - Tf, 1e-10f);
                float exp_depth = inside ? render_depth[pid] : 0.0f;
                if (dist) {   // log-depth render: depth = exp(C_lnz / W), RasterizationEval3DBwd_kernel.cuh:212-218
                    const float m = ssr_log(ssr_max(exp_depth, 1e-6f));
                    vT = vT + ((exp_depth * vd) * m) * inv_alpha;
                    vd = vd * (exp_depth * inv_alpha);
                } else {
                    vT = vT + (exp_depth * vd) * inv_alpha;
                    vd = vd * inv_alpha;
                }
                T1[p] = Tf; vT1[p] = vT;
                vc[p][0] = vr; vc[p][1] = vg; vc[p][2] = vb; vc[p][3] = vd;
                if (dist) {   // :228-257
                    for (int q = 0; q < 3; q++) Cc[p][q] = (inside && dist_rgb) ? render_rgb[3 * pid + q] : 0.0f;
                    Cc[p][3] = ssr_log(ssr_max(exp_depth, 1e-6f)) * ssr_max(1.0f - Tf, 1e-10f);
                    const float W = inside ? (1.0f - Tf) : 0.0f;
                    const float invW = W > 1e-10f ? (1.0f / W) : 0.0f;
                    float Dv[4] = {0, 0, 0, 0};
                    for (int q = 0; q < 4; q++) vD[p][q] = 0.0f;
                    if (inside) {
                        if (dist_rgb) for (int q = 0; q < 3; q++) { Dv[q] = dist_rgb_img[3 * pid + q]; vD[p][q] = v_dist_rgb[3 * pid + q]; }
                        Dv[3] = dist_depth_img[pid]; vD[p][3] = v_dist_depth[pid];
                    }
                    for (int q = 0; q < 4; q++) Sc[p][q] = (Dv[q] + Cc[p][q] * Cc[p][q]) * invW;
                    Wd[p] = W;
                }
                amap[p] = (accum_mode && accum_map && inside) ? accum_map[pid] : 0.0f;
                med_v[p] = (v_median && inside) ? v_median[pid] : 0.0f;
                pend_zgrad[p] = pend_zfar[p] = pend_Tfar[p] = 0.0f;
            }
            for (int32_t k = end - 1; k >= start; k--) {
                const int32_t g = flatten_ids[k];
                if (!micro_hit(xy + 2 * g, conic + 3 * g, opac[g], (float)bx, (float)by)) continue;
                const Frag f = load_frag(g, xy, depth, conic, opac, rgb);
                float acc[10] = {0};   // xy(2) depth conic(3) opac rgb(3)
                double aacc[10] = {0};
                bool any = false;
                float aw = 0.0f, aw_den = 0.0f;
                for (int p = 0; p < 64; p++) {
                    if (k > bin_final[p]) continue;
                    const float px = (float)(bx + p % kMicro) + 0.5f, py = (float)(by + p / kMicro) + 0.5f;
                    float dx, dy, vis, sigma;
                    const float alpha = eval_alpha(f, px, py, dx, dy, vis, sigma);
                    if (alpha <= kAlphaThreshold) continue;
                    any = true;
                    const float ra = 1.0f / (1.0f - alpha);
                    const float T0 = T1[p] * ra;
                    const float* c = vc[p];
                    float vT1p = vT1[p];
                    float v_depth_median = 0.0f;
                    if (v_median) {   // :433-470
                        const float vm = med_v[p];
                        if (pend_Tfar[p] > 0.0f) {   // this splat is the near member of the crossing found one step ago
                            v_depth_median += pend_zgrad[p];
                            const float a_ln = ssr_log(T1[p]), b_ln = ssr_log(pend_Tfar[p]);
                            const float dba = b_ln - a_ln;
                            const float inv = (ssr_fabs(dba) > 1e-20f) ? (-1.0f / dba) : 0.0f;
                            const float Sg = (vm * (pend_zfar[p] - f.d)) * inv;
                            vT1p += Sg / T1[p];
                            pend_Tfar[p] = 0.0f;
                        }
                        if (T0 >= 0.5f && T1[p] < 0.5f) {   // far member: the post-splat T drops below 1/2 here
                            const float a = ssr_log(T0), b = ssr_log(T1[p]), d = b - a;
                            const float fr = (ssr_fabs(d) > 1e-20f) ? (-0.6931471805599453f - a) / d : 0.0f;
                            v_depth_median += fr * vm;
                            pend_zgrad[p] = (1.0f - fr) * vm;
                            pend_zfar[p] = f.d;
                            pend_Tfar[p] = T1[p];
                        }
                    }
                    const float zd = dist ? ssr_log(ssr_max(f.d, 1e-6f)) : f.d;
                    const float dotcv = ssr_fma(zd, c[3], ssr_fma(f.b, c[2], ssr_fma(f.g, c[1], f.r * c[0])));
                    float v_alpha = T0 * dotcv - vT1p * T0;
                    const float w = alpha * T0;
                    float v_T0 = alpha * dotcv + vT1p * (1.0f - alpha);
                    float vcol[4] = {c[0] * w, c[1] * w, c[2] * w, c[3] * w};
                    if (dist) {   // closed form D = W S - C^2, :497-517
                        const float col[4] = {f.r, f.g, f.b, zd};
                        float gsum = 0.0f;
                        for (int q = dist_rgb ? 0 : 3; q < 4; q++) {
                            vcol[q] += ((col[q] * Wd[p] - Cc[p][q]) * vD[p][q]) * (2.0f * w);
                            gsum += ((Sc[p][q] + (col[q] * col[q]) * Wd[p]) - (col[q] * Cc[p][q]) * 2.0f) * vD[p][q];
                        }
                        v_alpha += T0 * gsum;
                        v_T0 += alpha * gsum;
                        vcol[3] *= 1.0f / ssr_max(f.d, 1e-6f);
                    }
                    vcol[3] += v_depth_median;
                    float t[10] = {0};
                    // v_alpha is a difference, T0 (c . v_c) - v_T1 T0, often of nearly equal numbers: what rounding
                    // moves in it scales with the two products, not with what is left of them. For the magnitude sums
                    // the six channels that are linear in v_alpha are therefore taken at |T0 (c . v_c)| + |v_T1 T0|.
                    const float v_alpha_mag = ssr_fabs(T0 * dotcv) + ssr_fabs(vT1p * T0);
                    float tmag[10] = {0};
                    if (sigma >= 0.f && f.opac * vis <= 0.999f) {
                        const float v_sigma = (-f.opac) * vis * v_alpha;
                        t[3] = 0.5f * v_sigma * dx * dx;
                        t[4] = v_sigma * dx * dy;
                        t[5] = 0.5f * v_sigma * dy * dy;
                        t[0] = v_sigma * (f.cx * dx + f.cy * dy);
                        t[1] = v_sigma * (f.cy * dx + f.cz * dy);
                        t[6] = vis * v_alpha;
                        const float m_sigma = f.opac * vis * v_alpha_mag;
                        tmag[3] = 0.5f * m_sigma * dx * dx;
                        tmag[4] = ssr_fabs(m_sigma * dx * dy);
                        tmag[5] = 0.5f * m_sigma * dy * dy;
                        tmag[0] = m_sigma * (ssr_fabs(f.cx * dx) + ssr_fabs(f.cy * dy));
                        tmag[1] = m_sigma * (ssr_fabs(f.cy * dx) + ssr_fabs(f.cz * dy));
                        tmag[6] = vis * v_alpha_mag;
                    }
                    t[7] = vcol[0]; t[8] = vcol[1]; t[9] = vcol[2]; t[2] = vcol[3];
                    tmag[7] = ssr_fabs(vcol[0]); tmag[8] = ssr_fabs(vcol[1]); tmag[9] = ssr_fabs(vcol[2]); tmag[2] = ssr_fabs(vcol[3]);
                    for (int q = 0; q < 10; q++) acc[q] += t[q];
                    // Every term carries the rounding of the undo steps that produced its T0 and v_T1 (a division and
                    // a product each, about two ulp a step, 1.2e-7): with the 2e-6 of the magnitude sum that tests
                    // allow for summation order, a term n steps deep counts (1 + 0.06 n) times.
                    if (abs_terms) {
                        const double deep = 1.0 + 0.06 * undo_steps[p];
                        for (int q = 0; q < 10; q++) aacc[q] += (double)ssr_max(ssr_fabs(t[q]), tmag[q]) * deep;
                    }
                    undo_steps[p]++;
                    if (accum_mode == 1) aw = ssr_max(aw, amap[p] * w);   // :553-562
                    else if (accum_mode) { aw += amap[p] * w; if (accum_mode == 3) aw_den += w; }
                    T1[p] = T0; vT1[p] = v_T0;
                }
                if (any) {
                    for (int q = 0; q < 10; q++) {
                        float v = ssr_isfinite(acc[q]) ? acc[q] : 0.0f;   // atomicAddFVec, Common.cuh:791-856
                        part[(size_t)k * 10 + q] += v;
                        if (abs_terms) apart[(size_t)k * 10 + q] += aacc[q];
                    }
                    if (accum_mode == 1) awpart[(size_t)k * 2] = ssr_max(awpart[(size_t)k * 2], aw);
                    else if (accum_mode) { awpart[(size_t)k * 2] += aw; awpart[(size_t)k * 2 + 1] += aw_den; }
                }
            }
        }
    }
    for (int64_t k = 0; k < n_isects; k++) {
        const int32_t g = flatten_ids[k];
        const float* p = &part[(size_t)k * 10];
        v_xy[2 * g] += p[0]; v_xy[2 * g + 1] += p[1];
        v_sdepth[g] += p[2];
        v_conic[3 * g] += p[3]; v_conic[3 * g + 1] += p[4]; v_conic[3 * g + 2] += p[5];
        v_opac[g] += p[6];
        v_srgb[3 * g] += p[7]; v_srgb[3 * g + 1] += p[8]; v_srgb[3 * g + 2] += p[9];
        if (abs_terms) for (int q = 0; q < 10; q++) abs_terms[(size_t)g * 10 + q] += apart[(size_t)k * 10 + q];
        if (accum_mode) {
            const int64_t wid = gaussian_ids ? gaussian_ids[g] : g;
            if (accum_mode == 1) accum_weight[wid] = ssr_max(accum_weight[wid], awpart[(size_t)k * 2]);
            else {
                accum_weight[wid] += awpart[(size_t)k * 2];
                if (accum_mode == 3) accum_weight[n_world + wid] += awpart[(size_t)k * 2 + 1];
            }
        }
    }
}

// projection_fused_bwd_kernel, src/kernels/projection/ProjectionBwd_kernel.cuh:16-130, with
// World::project_vjp (src/primitives/Primitive3DGS.cuh:119-201). The projection VJP is derived by
// hand from projection_3dgs (assume_valid form); its autodiff conventions follow
// src/generated/primitive_3dgs.cuh:12782-13230: a clamped Jacobian entry passes its gradient to
// the violated bound (which depends on z), v_conic enters as [[vx, vy],[0, vz]], normalize(quat)
// and length() are differentiated, and extend/aabb/sorting depth/radius carry no gradient.
void or_projection_bwd(int64_t N, int sh_degree, const float* means, const float* quats,
    const float* log_scales, const float* opacity_logits, const float* features_dc,
    const or_sh_source* sh, const or_camera* camera, const float* aabb, const float* v_xy,
    const float* v_sdepth, const float* v_conic, const float* v_opac, const float* v_srgb,
    float* v_means, float* v_quats, float* v_scales, float* v_opacities, float* v_dc, float* v_sh) {
    or_projection_bwd_pose(N, sh_degree, means, quats, log_scales, opacity_logits, features_dc, sh, camera, aabb, v_xy, v_sdepth,
                           v_conic, v_opac, v_srgb, v_means, v_quats, v_scales, v_opacities, v_dc, v_sh, nullptr);
}

void or_projection_bwd_pose(int64_t N, int sh_degree, const float* means, const float* quats,
    const float* log_scales, const float* opacity_logits, const float* features_dc,
    const or_sh_source* sh, const or_camera* camera, const float* aabb, const float* v_xy,
    const float* v_sdepth, const float* v_conic, const float* v_opac, const float* v_srgb,
    float* v_means, float* v_quats, float* v_scales, float* v_opacities, float* v_dc, float* v_sh, float* v_viewmat) {
    const Cam cam = load_cam(camera);
    const int n_coef = sh_degree * (sh_degree + 2);
    auto fin = [](float v) { return ssr_isfinite(v) ? v : 0.0f; };
    std::vector<float> pose(v_viewmat ? (size_t)N * 12 : 0, 0.0f);   // per-splat dL/dR (9) and dL/dt (3), summed below
#pragma omp parallel for schedule(static)
    for (int64_t g = 0; g < N; g++) {
        const float* bb = aabb + 4 * g;
        if (bb[2] <= bb[0] || bb[3] <= bb[1]) continue;   // ProjectionBwd_kernel.cuh:58
        const float* mean = means + 3 * g;
        Proj p = project(cam, mean, quats + 4 * g, log_scales + 3 * g, opacity_logits[g], true);
        const float x = p.mc[0], y = p.mc[1], z = p.mc[2];
        float vmc[3] = {0, 0, 0};
        // --- conic = inverse(cov2d) ---
        const float c00 = p.c2[0][0], c01 = p.c2[0][1], c10 = p.c2[1][0], c11 = p.c2[1][1];
        const float det = c00 * c11 - c01 * c10, inv = 1.0f / det;
        const float g00 = v_conic[3 * g], g01 = v_conic[3 * g + 1], g11 = v_conic[3 * g + 2];
        const float v_inv = (c11 * g00 - c01 * g01) + c00 * g11;
        const float v_det = -(v_inv / (det * det));
        float vC[2][2];
        vC[0][0] = inv * g11 + c11 * v_det;
        vC[1][1] = inv * g00 + c00 * v_det;
        vC[0][1] = -(inv * g01) - c10 * v_det;
        vC[1][0] = -(c01 * v_det);
        if (cam.aa) {
            // opacity = sigmoid(logit) * sqrt(max(0, det_orig / det_blur)): through both determinants to the 2D covariance
            const float ratio = p.det_orig / p.det_blur;
            const float v_comp = v_opac[g] * p.sig;
            const float v_ratio = ratio > 0.0f ? v_comp * (0.5f / ssr_sqrt(ssr_max(1e-7f, ratio))) : 0.0f;
            const float v_do = v_ratio / p.det_blur;
            const float v_db = -((v_ratio * p.det_orig) / (p.det_blur * p.det_blur));
            vC[0][0] += v_do * p.c2o[1] + v_db * c11;
            vC[1][1] += v_do * p.c2o[0] + v_db * c00;
            vC[0][1] += (v_do + v_db) * (-c10);
            vC[1][0] += (v_do + v_db) * (-c01);
        }
        // --- cov2d = J covc J^T ---
        float vJ[2][3], vS[3][3];
        for (int i = 0; i < 2; i++)
            for (int k = 0; k < 3; k++) {
                float s = 0.0f;
                for (int j = 0; j < 2; j++)
                    for (int l = 0; l < 3; l++)
                        s += vC[i][j] * p.J[j][l] * p.covc[k][l] + vC[j][i] * p.J[j][l] * p.covc[l][k];
                vJ[i][k] = s;
            }
        for (int k = 0; k < 3; k++)
            for (int l = 0; l < 3; l++) {
                float s = 0.0f;
                for (int i = 0; i < 2; i++)
                    for (int j = 0; j < 2; j++) s += p.J[i][k] * vC[i][j] * p.J[j][l];
                vS[k][l] = s;
            }
        const float vm0 = v_xy[2 * g], vm1 = v_xy[2 * g + 1];
        if (lens_path(cam)) {
            // bwd_diff of *_proj_uv and of its forward-mode Jacobian (projection_utils.slang:362-375,
            // 463-493): v_p = J^T v_uv + sum_ij v_J[i][j] dJ[i][j]/dp, with dJ/dp the Hessians of the
            // two pixel coordinates; a clamped J[i][2] (perspective only) depends on z through its bound.
            typedef SsrJet<3, 2> Jet;
            Jet px, py;
            ssr_model_pixel<Jet>(cam.model, cam.tier, cam.dc, cam.fx, cam.fy, cam.cx, cam.cy, ssr_jet_seed<3, 2>(x, 0),
                                 ssr_jet_seed<3, 2>(y, 1), ssr_jet_seed<3, 2>(z, 2), px, py);
            const float iz2 = 1.0f / (z * z);
            const float Wf = (float)cam.W;
            const float lim_pos = Wf + 0.3f * (0.5f * Wf), lim_neg = 0.3f * (0.5f * Wf);
            const float bound_lo[2] = {-(lim_pos - cam.cx), -(lim_pos - cam.cy)}, bound_hi[2] = {lim_neg + cam.cx, lim_neg + cam.cy};
            for (int i = 0; i < 2; i++) {
                const Jet& f = i == 0 ? px : py;
                const float vm = i == 0 ? vm0 : vm1;
                for (int k = 0; k < 3; k++) vmc[k] += vm * f.d[k];
                for (int j = 0; j < 3; j++) {
                    if (j == 2 && p.clamp_lo[i]) { vmc[2] += vJ[i][2] * bound_lo[i] * (-iz2); continue; }
                    if (j == 2 && p.clamp_hi[i]) { vmc[2] += vJ[i][2] * bound_hi[i] * (-iz2); continue; }
                    for (int k = 0; k < 3; k++) vmc[k] += vJ[i][j] * f.h[j <= k ? ssr_jet_idx<3>(j, k) : ssr_jet_idx<3>(k, j)];
                }
            }
        } else if (cam.model == OR_CAM_PINHOLE) {
            const float z2 = z * z, iz = 1.0f / z, iz2 = 1.0f / z2;
            vmc[2] += vJ[0][0] * (-cam.fx * iz2) + vJ[1][1] * (-cam.fy * iz2);
            const float Wf = (float)cam.W;
            const float lim_pos = Wf + 0.3f * (0.5f * Wf), lim_neg = 0.3f * (0.5f * Wf);
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
        // --- depth = length(mean_c), sqrt derivative guarded at 1e-7 ---
        {
            const float s2 = dot3(p.mc, p.mc);
            const float vs = v_sdepth[g] * (0.5f / ssr_sqrt(ssr_max(1e-7f, s2)));
            for (int i = 0; i < 3; i++) vmc[i] += 2.0f * p.mc[i] * vs;
        }
        float vmean[3];
        for (int i = 0; i < 3; i++) vmean[i] = (cam.R[0][i] * vmc[0] + cam.R[1][i] * vmc[1]) + cam.R[2][i] * vmc[2];
        // --- covc = R cov R^T  ->  v_cov = R^T vS R ; cov = M M^T ---
        float t1[3][3], vcov[3][3], vM[3][3];
        for (int i = 0; i < 3; i++)
            for (int j = 0; j < 3; j++)
                t1[i][j] = (cam.R[0][i] * vS[0][j] + cam.R[1][i] * vS[1][j]) + cam.R[2][i] * vS[2][j];
        for (int i = 0; i < 3; i++)
            for (int j = 0; j < 3; j++)
                vcov[i][j] = (t1[i][0] * cam.R[0][j] + t1[i][1] * cam.R[1][j]) + t1[i][2] * cam.R[2][j];
        for (int i = 0; i < 3; i++)
            for (int j = 0; j < 3; j++) {
                float s = 0.0f;
                for (int k = 0; k < 3; k++) s += (vcov[i][k] + vcov[k][i]) * p.M[k][j];
                vM[i][j] = s;
            }
        float vRq[3][3], vscale[3];
        for (int j = 0; j < 3; j++) {
            float s = 0.0f;
            for (int i = 0; i < 3; i++) { vRq[i][j] = vM[i][j] * p.s[j]; s += vM[i][j] * p.Rq[i][j]; }
            vscale[j] = s * p.s[j];   // through exp(log_scale)
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
        for (int i = 0; i < 4; i++) vquat[i] = (vqn[i] - p.qn[i] * qd) * p.qinv;
        const float vlogit = (v_opac[g] * p.comp) * (p.sig * (1.0f - p.sig));

        // --- SH colour VJP, harmonics.slang:373-649,1087-1126 ---
        float coef[45];
        decode_sh(g, sh, n_coef, coef);
        float dir[3];
        view_dir(cam, mean, dir);
        ShBasis b = sh_basis(sh_degree, dir);
        float raw[3];
        sh_color_raw(sh_degree, b, features_dc + 3 * g, coef, raw);
        float vc[3];
        for (int c = 0; c < 3; c++) vc[c] = v_srgb[3 * g + c] * (raw[c] >= -0.5f ? 1.0f : 0.0f);
        float vdcl[3];
        for (int c = 0; c < 3; c++) vdcl[c] = 0.2820947917738781f * vc[c];
        float vdir[3] = {0, 0, 0};
        if (sh_degree >= 1) {
            for (int j = 0; j < n_coef; j++) {
                float tv[3] = {b.Y[j] * vc[0], b.Y[j] * vc[1], b.Y[j] * vc[2]};
                float d2 = dot3(tv, tv);
                if (ssr_isfinite(d2) && d2 != 0.0f)   // harmonics.slang:397-403
                    for (int c = 0; c < 3; c++) v_sh[g * 45 + j * 3 + c] += tv[c];
            }
            auto cd = [&](int j) { return (coef[3 * j] * vc[0] + coef[3 * j + 1] * vc[1]) + coef[3 * j + 2] * vc[2]; };
            const float X = b.x, Y = b.y, Z = b.z;
            float vx = -0.48860251190292f * cd(2), vy = -0.48860251190292f * cd(0), vz = 0.48860251190292f * cd(1);
            if (sh_degree >= 2) {
                const float z2 = Z * Z;
                const float fTmp0B = -1.092548430592079f * Z;
                const float fC1 = X * X - Y * Y, fS1 = 2.f * X * Y;
                const float fC1_x = 2.f * X, fC1_y = -2.f * Y, fS1_x = 2.f * Y, fS1_y = 2.f * X;
                const float pSH6_z = 2.f * 0.9461746957575601f * Z;
                const float pSH7_x = fTmp0B, pSH7_z = -1.092548430592079f * X;
                const float pSH5_y = fTmp0B, pSH5_z = -1.092548430592079f * Y;
                const float pSH8_x = 0.5462742152960395f * fC1_x, pSH8_y = 0.5462742152960395f * fC1_y;
                const float pSH4_x = 0.5462742152960395f * fS1_x, pSH4_y = 0.5462742152960395f * fS1_y;
                vx += pSH4_x * cd(3) + pSH8_x * cd(7) + pSH7_x * cd(6);
                vy += pSH4_y * cd(3) + pSH8_y * cd(7) + pSH5_y * cd(4);
                vz += pSH6_z * cd(5) + pSH7_z * cd(6) + pSH5_z * cd(4);
                if (sh_degree >= 3) {
                    const float fTmp0C = -2.285228997322329f * z2 + 0.4570457994644658f;
                    const float fTmp1B = 1.445305721320277f * Z;
                    const float fC2 = X * fC1 - Y * fS1, fS2 = X * fS1 + Y * fC1;
                    (void)fC2; (void)fS2;
                    const float fTmp0C_z = -2.285228997322329f * 2.f * Z;
                    const float fTmp1B_z = 1.445305721320277f;
                    const float fC2_x = fC1 + X * fC1_x - Y * fS1_x;
                    const float fC2_y = X * fC1_y - fS1 - Y * fS1_y;
                    const float fS2_x = fS1 + X * fS1_x + Y * fC1_x;
                    const float fS2_y = X * fS1_y + fC1 + Y * fC1_y;
                    const float pSH12_z = 3.f * 1.865881662950577f * z2 - 1.119528997770346f;
                    const float pSH13_x = fTmp0C, pSH13_z = fTmp0C_z * X;
                    const float pSH11_y = fTmp0C, pSH11_z = fTmp0C_z * Y;
                    const float pSH14_x = fTmp1B * fC1_x, pSH14_y = fTmp1B * fC1_y, pSH14_z = fTmp1B_z * fC1;
                    const float pSH10_x = fTmp1B * fS1_x, pSH10_y = fTmp1B * fS1_y, pSH10_z = fTmp1B_z * fS1;
                    const float pSH15_x = -0.5900435899266435f * fC2_x, pSH15_y = -0.5900435899266435f * fC2_y;
                    const float pSH9_x = -0.5900435899266435f * fS2_x, pSH9_y = -0.5900435899266435f * fS2_y;
                    vx += pSH9_x * cd(8) + pSH15_x * cd(14) + pSH10_x * cd(9) + pSH14_x * cd(13) + pSH13_x * cd(12);
                    vy += pSH9_y * cd(8) + pSH15_y * cd(14) + pSH10_y * cd(9) + pSH14_y * cd(13) + pSH11_y * cd(10);
                    vz += pSH12_z * cd(11) + pSH13_z * cd(12) + pSH11_z * cd(10) + pSH14_z * cd(13) + pSH10_z * cd(9);
                }
            }
            const float dn = (vx * X + vy * Y) + vz * Z;
            vdir[0] = (vx - dn * X) * b.inorm;
            vdir[1] = (vy - dn * Y) * b.inorm;
            vdir[2] = (vz - dn * Z) * b.inorm;
        }
        if (v_viewmat) {
            // mean_c = R mean + t, cov_c = R cov R^T, view direction = mean + R^T t (primitive_3dgs.slang:434-436,
            // harmonics.slang:145-149): dL/dt = v_mean_c + R v_dir, dL/dR = v_mean_c mean^T + (vS + vS^T) R cov + t v_dir^T
            float cov[3][3], RS[3][3];
            for (int a = 0; a < 3; a++)
                for (int j = 0; j < 3; j++) cov[a][j] = (p.M[a][0] * p.M[j][0] + p.M[a][1] * p.M[j][1]) + p.M[a][2] * p.M[j][2];
            for (int k = 0; k < 3; k++)
                for (int j = 0; j < 3; j++) RS[k][j] = (cam.R[k][0] * cov[0][j] + cam.R[k][1] * cov[1][j]) + cam.R[k][2] * cov[2][j];
            float* out = pose.data() + 12 * g;
            for (int i = 0; i < 3; i++) {
                out[9 + i] = vmc[i] + ((cam.R[i][0] * vdir[0] + cam.R[i][1] * vdir[1]) + cam.R[i][2] * vdir[2]);
                for (int j = 0; j < 3; j++) {
                    float s = vmc[i] * mean[j] + cam.t[i] * vdir[j];
                    for (int k = 0; k < 3; k++) s += (vS[i][k] + vS[k][i]) * RS[k][j];
                    out[3 * i + j] = s;
                }
            }
        }
        // World::atomicStore, PrimitiveBase3DGS.cuh:75-83: per-component finite filter
        for (int i = 0; i < 3; i++) v_means[3 * g + i] += fin(vmean[i] + vdir[i]);
        for (int i = 0; i < 4; i++) v_quats[4 * g + i] += fin(vquat[i]);
        for (int i = 0; i < 3; i++) v_scales[3 * g + i] += fin(vscale[i]);
        v_opacities[g] += fin(vlogit);
        for (int i = 0; i < 3; i++) v_dc[3 * g + i] += fin(vdcl[i]);
    }
    if (v_viewmat) {   // summed in double, in splat order (the kernels add floats in an unspecified order)
        double acc[12] = {0};
        for (int64_t g = 0; g < N; g++)
            for (int k = 0; k < 12; k++) acc[k] += pose[12 * g + k];
        for (int i = 0; i < 3; i++) {
            for (int j = 0; j < 3; j++) v_viewmat[4 * i + j] += (float)acc[3 * i + j];
            v_viewmat[4 * i + 3] += (float)acc[9 + i];
        }
    }
}

}  // extern "C"
