"""Independent float64 restatements (numpy) used to pin the oracle: matrix-form projection,
textbook real spherical harmonics, brute-force per-pixel compositing. None of this code is shared
with the oracle or the kernels; finite differences of these functions pin the backward passes."""
from __future__ import annotations

import math

import numpy as np

ALPHA_T = 1.0 / 255.0


def quat_rot(q):
    w, x, y, z = q / np.linalg.norm(q)
    return np.array([
        [1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
        [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
        [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]])


def lens_distort(tier, c, u, v):
    """The distortion tiers of src/shaders/projection_utils.slang:235-295, written from the COLMAP model
    definitions (OPENCV, THIN_PRISM_FISHEYE radial-first, FULL_OPENCV); works on complex numbers."""
    if tier == 0:
        return u, v
    r2 = u * u + v * v
    if tier == 1:
        k1, k2, p1, p2 = c[:4]
        radial, sx, sy = 1 + k1 * r2 + k2 * r2 ** 2, 0.0, 0.0
    elif tier == 2:
        k1, k2, k3, k4, p1, p2, sx, sy = c[:8]
        radial = 1 + k1 * r2 + k2 * r2 ** 2 + k3 * r2 ** 3 + k4 * r2 ** 4
    else:
        k1, k2, k3, k4, k5, k6, p1, p2 = c[:8]
        radial = (1 + k1 * r2 + k2 * r2 ** 2 + k3 * r2 ** 3) / (1 + k4 * r2 + k5 * r2 ** 2 + k6 * r2 ** 3)
        sx = sy = 0.0
    du = u * radial + 2 * p1 * u * v + p2 * (r2 + 2 * u * u) + sx * r2
    dv = v * radial + 2 * p2 * u * v + p1 * (r2 + 2 * v * v) + sy * r2
    return du, dv


def model_normalised(model, x, y, z):
    """(x/z, y/z); equidistant fisheye theta * (x, y)/r; equisolid 2 sin(theta/2) * (x, y)/r. Complex-safe:
    inputs may carry an infinitesimal imaginary part (complex-step differentiation)."""
    import cmath
    if model == 0:
        return x / z, y / z
    r = cmath.sqrt(x * x + y * y)
    # atan2 under complex-step differentiation: the real angle, plus i times its differential
    rr, zr = complex(r).real, complex(z).real
    theta = complex(math.atan2(rr, zr), (zr * complex(r).imag - rr * complex(z).imag) / (rr * rr + zr * zr))
    if abs(r) < 1e-12:
        k = 1.0 / z
    elif model == 1:
        k = theta / r
    else:
        k = 2 * cmath.sin(0.5 * theta) / r
    return x * k, y * k


def model_pixel(model, tier, coeffs, intr, p):
    fx, fy, cx, cy = [float(v) for v in intr]
    u, v = model_normalised(model, p[0], p[1], p[2])
    du, dv = lens_distort(tier, [float(c) for c in coeffs], u, v)
    return fx * du + cx, fy * dv + cy


def model_jacobian(model, tier, coeffs, intr, p):
    """d pixel / d p by complex-step differentiation (no subtraction, so exact to rounding)."""
    J = np.zeros((2, 3))
    h = 1e-30
    for k in range(3):
        q = [complex(v) for v in p]
        q[k] += 1j * h
        a, b = model_pixel(model, tier, coeffs, intr, q)
        J[0, k], J[1, k] = a.imag / h, b.imag / h
    return J


def lens_valid(tier, coeffs, u, v):
    """is_valid_distortion (src/shaders/projection_utils.slang:310-321), with central differences."""
    if tier == 0:
        return True, 1.0
    c = [float(x) for x in coeffs]
    h = 1e-6
    a1, b1 = lens_distort(tier, c, u + h, v); a0, b0 = lens_distort(tier, c, u - h, v)
    c1, d1 = lens_distort(tier, c, u, v + h); c0, d0 = lens_distort(tier, c, u, v - h)
    j00, j10, j01, j11 = (a1 - a0) / (2 * h), (b1 - b0) / (2 * h), (c1 - c0) / (2 * h), (d1 - d0) / (2 * h)
    jdet = min(j00 * j11 - j01 * j10, j00, j11)
    du, dv = lens_distort(tier, c, u, v)
    return (0.25 < jdet < 4.0) and (u * du + v * dv >= 0), jdet


def project(mean, quat, log_scale, logit, viewmat, intr, width, model, f32_consts=True, tier=0, coeffs=None, antialiased=False):
    """Returns xy(2), depth, conic(3), opac, plus cov2d (blurred) and the tile extents."""
    R, t = viewmat[:3, :3].astype(np.float64), viewmat[:3, 3].astype(np.float64)
    fx, fy, cx, cy = [float(v) for v in intr]
    pc = R @ mean + t
    x, y, z = pc
    Rq = quat_rot(quat)
    S = np.diag(np.exp(log_scale))
    cov = Rq @ S @ S @ Rq.T
    covc = R @ cov @ R.T
    coeffs = np.zeros(8) if coeffs is None else np.asarray(coeffs, np.float64)
    extra = {}
    if model in (1, 2) or tier != 0:
        a, b = model_pixel(model, tier, coeffs, intr, [complex(v) for v in pc])
        xy = np.array([a.real, b.real])
        J = model_jacobian(model, tier, coeffs, intr, pc)
        u, v = model_normalised(model, complex(x), complex(y), complex(z))
        extra["lens_valid"], extra["lens_jdet"] = lens_valid(tier, coeffs, u.real, v.real)
    elif model == 0:
        xy = np.array([fx * x / z + cx, fy * y / z + cy])
        J = np.array([[fx / z, 0, -fx * x / z ** 2], [0, fy / z, -fy * y / z ** 2]])
    else:
        h = math.hypot(x, z)
        r2 = x * x + y * y + z * z
        xy = np.array([fx * math.atan2(x, z) + cx, fy * math.atan2(y, h) + cy])
        J = np.array([[fx * z / h ** 2, 0, -fx * x / h ** 2],
                      [-fy * x * y / (h * r2), fy * h / r2, -fy * z * y / (h * r2)]])
    if model == 0:
        c03 = float(np.float32(0.3)) if f32_consts else 0.3
        lim_pos = width + c03 * (0.5 * width)
        lim_neg = c03 * (0.5 * width)
        # y limits reuse the x limits (src/shaders/primitive_3dgs.slang:92-93)
        J[0, 2] = min(max(J[0, 2], -(lim_pos - cx) / z), (lim_neg + cx) / z)
        J[1, 2] = min(max(J[1, 2], -(lim_pos - cy) / z), (lim_neg + cy) / z)
    c2 = J @ covc @ J.T
    opac = 1.0 / (1.0 + math.exp(-logit))
    if model in (1, 2):
        # the weight the unblurred splat still has at the image centre (src/shaders/primitive_3dgs.slang:509-514)
        m = xy - np.array([cx, cy])
        extra["centre_weight"] = opac * math.exp(-0.5 * float(m @ np.linalg.inv(c2) @ m))
    # screen-space blur; the antialiased ("mip") variant blurs less and rescales the opacity by the square root of
    # the ratio of the determinants, so that a splat keeps its integrated weight (src/shaders/primitive_3dgs.slang:398-405,528-543)
    blur = 0.1 if antialiased else 0.3
    eps = float(np.float32(blur)) if f32_consts else blur
    det_before = float(np.linalg.det(c2))
    c2 = c2 + eps * np.eye(2)
    if antialiased:
        opac = opac * math.sqrt(max(0.0, det_before / float(np.linalg.det(c2))))
    inv = np.linalg.inv(c2)
    depth = float(np.linalg.norm(pc))
    return dict(xy=xy, depth=depth, conic=np.array([inv[0, 0], inv[0, 1], inv[1, 1]]), opac=opac,
                cov2d=c2, pc=pc, **extra)


def real_sh_deg3(d):
    """Textbook real spherical harmonics l=1..3 (Cartesian forms, unit vector d), multiplied by the
    Condon-Shortley sign (-1)^m that the reference's basis carries
    (src/shaders/harmonics.slang:172-217). Order: l=1 m=-1,0,1; l=2 m=-2..2; l=3 m=-3..3."""
    x, y, z = d / np.linalg.norm(d)
    pi = math.pi
    Y = [
        -math.sqrt(3 / (4 * pi)) * y, math.sqrt(3 / (4 * pi)) * z, -math.sqrt(3 / (4 * pi)) * x,
        0.5 * math.sqrt(15 / pi) * x * y, -0.5 * math.sqrt(15 / pi) * y * z,
        0.25 * math.sqrt(5 / pi) * (3 * z * z - 1), -0.5 * math.sqrt(15 / pi) * x * z,
        0.25 * math.sqrt(15 / pi) * (x * x - y * y),
        -0.25 * math.sqrt(35 / (2 * pi)) * y * (3 * x * x - y * y),
        0.5 * math.sqrt(105 / pi) * x * y * z,
        -0.25 * math.sqrt(21 / (2 * pi)) * y * (5 * z * z - 1),
        0.25 * math.sqrt(7 / pi) * (5 * z ** 3 - 3 * z),
        -0.25 * math.sqrt(21 / (2 * pi)) * x * (5 * z * z - 1),
        0.25 * math.sqrt(105 / pi) * (x * x - y * y) * z,
        -0.25 * math.sqrt(35 / (2 * pi)) * x * (x * x - 3 * y * y),
    ]
    return np.array(Y)


def sh_color(mean, viewmat, dc, coeffs, degree=3, clamp=True):
    R, t = viewmat[:3, :3].astype(np.float64), viewmat[:3, 3].astype(np.float64)
    d = mean + R.T @ t            # mean - campos
    Y = real_sh_deg3(d)
    ncoef = degree * (degree + 2)
    col = 0.5 * math.sqrt(1 / math.pi) * dc + (Y[:ncoef, None] * coeffs[:ncoef]).sum(axis=0)
    col = col + 0.5
    return np.maximum(col, 0.0) if clamp else col


def composite(px, py, frags, with_state=False):
    """Front-to-back compositing of one pixel over `frags` (already in sorted order):
    dict arrays xy[K,2], conic[K,3], opac[K], rgb[K,3], depth[K]. Returns rgb, depth, T, last."""
    T = 1.0
    rgb = np.zeros(3)
    dsum = 0.0
    last = 0
    for k in range(len(frags["opac"])):
        dx = frags["xy"][k, 0] - px
        dy = frags["xy"][k, 1] - py
        a, b, c = frags["conic"][k]
        sigma = 0.5 * (a * dx * dx + c * dy * dy) + b * dx * dy
        if sigma < 0:
            continue
        alpha = min(0.999, frags["opac"][k] * math.exp(-sigma))
        if alpha <= ALPHA_T:
            continue
        nT = T * (1 - alpha)
        if nT <= 1e-4:
            break
        w = alpha * T
        rgb = rgb + w * frags["rgb"][k]
        dsum += w * frags["depth"][k]
        T = nT
        last = k
    depth = dsum / max(1 - T, 1e-10)
    return rgb, depth, T, last


def composite_ex(px, py, frags, dist_type=0):
    """composite() plus the variant outputs, each from its definition rather than from the kernel's
    accumulators: per-splat weights w_k = alpha_k T_k; with distortion on, the depth channel is
    c = ln(max(z, 1e-6)), rendered depth = exp(sum w c / W), and the distortion image is
    1/2 sum_ij w_i w_j (c_i - c_j)^2 per channel (which equals W S - C^2); the median depth is where
    the post-splat transmittance first drops below 1/2, interpolated linearly in ln T from the
    previous splat (virtual first point z = 0, T = 1). Returns a dict."""
    K = len(frags["opac"])
    T = 1.0
    ws, ks = [], []
    median, prev_T, prev_z, found = 0.0, 1.0, 0.0, False
    for k in range(K):
        dx = frags["xy"][k, 0] - px
        dy = frags["xy"][k, 1] - py
        a, b, c = frags["conic"][k]
        sigma = 0.5 * (a * dx * dx + c * dy * dy) + b * dx * dy
        if sigma < 0:
            continue
        alpha = min(0.999, frags["opac"][k] * math.exp(-sigma))
        if alpha <= ALPHA_T:
            continue
        nT = T * (1 - alpha)
        if not found and prev_T >= 0.5 and nT < 0.5:
            la, lb = math.log(prev_T), math.log(nT)
            f = (math.log(0.5) - la) / (lb - la) if abs(lb - la) > 1e-20 else 0.0
            median = prev_z + (frags["depth"][k] - prev_z) * f
            found = True
        prev_T, prev_z = nT, frags["depth"][k]
        if nT <= 1e-4:
            break
        ws.append(alpha * T)
        ks.append(k)
        T = nT
    w = np.array(ws)
    ks = np.array(ks, int)
    rgbs = frags["rgb"][ks] if len(ks) else np.zeros((0, 3))
    z = frags["depth"][ks] if len(ks) else np.zeros(0)
    W = max(1 - T, 1e-10)
    out = dict(T=T, last=int(ks[-1]) if len(ks) else 0, rgb=(w[:, None] * rgbs).sum(axis=0), median=median, w=w, ks=ks)
    if dist_type:
        lz = np.log(np.maximum(z, 1e-6))
        out["depth"] = math.exp((w * lz).sum() / W)
        pair = lambda c: 0.5 * (w[:, None] * w[None, :] * (c[:, None] - c[None, :]) ** 2).sum()
        out["dist_depth"] = pair(lz)
        out["dist_rgb"] = np.array([pair(rgbs[:, q]) for q in range(3)]) if len(ks) else np.zeros(3)
    else:
        out["depth"] = (w * z).sum() / W
    return out


def median_plan(px, py, frags):
    """What the median-depth backward of the reference freezes at one pixel (RasterizationEval3DBwd_kernel.cuh:433-470):
    the composited splats in order, the far member of the crossing of T = 1/2 (first composited splat after which
    T < 1/2), the near member (the composited splat before it, None when the far one is the first) and
    d0 = ln(1 - alpha_far). None when T never crosses 1/2 among the composited splats (a crossing splat that also
    ends the pixel is not composited, and the backward never visits it)."""
    K = len(frags["opac"])
    T, chain = 1.0, []
    for k in range(K):
        dx, dy = frags["xy"][k, 0] - px, frags["xy"][k, 1] - py
        a, b, c = frags["conic"][k]
        sigma = 0.5 * (a * dx * dx + c * dy * dy) + b * dx * dy
        if sigma < 0:
            continue
        alpha = min(0.999, frags["opac"][k] * math.exp(-sigma))
        if alpha <= ALPHA_T:
            continue
        nT = T * (1 - alpha)
        if nT <= 1e-4:
            break
        if T >= 0.5 and nT < 0.5:
            return dict(chain=list(chain), near=chain[-1] if chain else None, far=k, d0=math.log(1 - alpha))
        chain.append(k)
        T = nT
    return None


def median_surrogate(px, py, frags, plan):
    """The function whose gradient the reference's median backward is: z_near + (z_far - z_near) (ln 1/2 - a) / d0 with
    a = sum over the composited splats up to the near one of ln(1 - alpha_j), and d0 (the far splat's own ln(1 - alpha))
    held at its value of the unperturbed scene -- "the far splat's own opacity term is omitted"."""
    a = 0.0
    for k in plan["chain"]:
        dx, dy = frags["xy"][k, 0] - px, frags["xy"][k, 1] - py
        ca, cb, cc = frags["conic"][k]
        sigma = 0.5 * (ca * dx * dx + cc * dy * dy) + cb * dx * dy
        a += math.log(1 - min(0.999, frags["opac"][k] * math.exp(-sigma)))
    z_n = frags["depth"][plan["near"]] if plan["near"] is not None else 0.0
    z_f = frags["depth"][plan["far"]]
    return z_n + (z_f - z_n) * (math.log(0.5) - a) / plan["d0"]
