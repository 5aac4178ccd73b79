// Device-side math shared by the gfx950 kernels.
//
// Everything here is float32 written as explicit single operations; the
// translation units are compiled with -ffp-contract=off so that a fused
// multiply-add appears only where __builtin_fmaf is spelled out.  That fixed
// operation order is what makes the integer outputs of the pipeline (radii,
// tile counts, sort keys) reproducible against a CPU evaluation of the same
// formulas.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/d3gs_hip.h"
#include <type_traits>

namespace d3gs {

constexpr int kDepthStepBits = 18;  // depth bits of the 32-bit sort key (render.py:737, 768)
constexpr int kTile = 16;          // tile edge in pixels (config tile_size, config_def.py:79)
constexpr int kBlock = 256;        // threads per tile / per 1-D block (csrc/inliner.py:38)

// exp with a fixed operation sequence (Cephes single-precision scheme): the
// same sequence on any IEEE-754 machine gives the same bits.  The reference
// calls CUDA's approximate __expf here (render.py:1768); its rounding is
// unspecified, this one is < 1 ulp from the true value.
__device__ __forceinline__ float det_expf(float x) {
    if (!(x == x)) return x;
    if (x < -86.0f) return 0.0f;
    if (x > 88.0f) return __builtin_inff();
    float kf = __builtin_rintf(x * 1.44269504088896341f);
    float r = __builtin_fmaf(kf, -0.693359375f, x);
    r = __builtin_fmaf(kf, 2.12194440e-4f, r);
    float z = r * r;
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    float e = __builtin_fmaf(p, z, r) + 1.0f;
    return __builtin_ldexpf(e, (int)kf);
}

// exp of the blend kernels: arguments known to lie in [-80, 80] and not NaN (a power that passed the cull
// threshold).  The same polynomial as det_expf with a cheaper range reduction, fixed like the rest of the
// sequence: k = round(x log2 e) comes out of one fused multiply-add with 1.5 * 2^23 (the sum's low mantissa bits
// are k), the reduced argument uses t - 1.5 * 2^23 = k, and 2^k is applied by adding k to the exponent field
// (the result stays normal in this range).  Two full-rate operations and an integer add in place of a multiply, a
// round, a convert and an ldexp, which issue at half rate.
__device__ __forceinline__ float det_expf_inrange(float x) {
    const float t = __builtin_fmaf(x, 1.44269504088896341f, 12582912.0f);
    const float kf = t - 12582912.0f;
    float r = __builtin_fmaf(kf, -0.693359375f, x);
    r = __builtin_fmaf(kf, 2.12194440e-4f, r);
    float z = r * r;
    float p = 1.9875691500e-4f;
    p = __builtin_fmaf(p, r, 1.3981999507e-3f);
    p = __builtin_fmaf(p, r, 8.3334519073e-3f);
    p = __builtin_fmaf(p, r, 4.1665795894e-2f);
    p = __builtin_fmaf(p, r, 1.6666665459e-1f);
    p = __builtin_fmaf(p, r, 5.0000001201e-1f);
    float e = __builtin_fmaf(p, z, r) + 1.0f;
    return __uint_as_float(__float_as_uint(e) + (__float_as_uint(t) << 23));
}

__device__ __forceinline__ float det_logf(float x) {
    if (!(x > 0.0f)) return -__builtin_inff();
    if (x < 1.17549435e-38f) x = 1.17549435e-38f;
    uint32_t ix = __float_as_uint(x);
    int e = (int)(ix >> 23) - 126;
    float m = __uint_as_float((ix & 0x007fffffu) | 0x3f000000u);
    if (m < 0.707106781186547524f) {
        e -= 1;
        m = (m + m) - 1.0f;
    } else {
        m = m - 1.0f;
    }
    float z = m * m;
    float y = 7.0376836292e-2f;
    y = __builtin_fmaf(y, m, -1.1514610310e-1f);
    y = __builtin_fmaf(y, m, 1.1676998740e-1f);
    y = __builtin_fmaf(y, m, -1.2420140846e-1f);
    y = __builtin_fmaf(y, m, 1.4249322787e-1f);
    y = __builtin_fmaf(y, m, -1.6668057665e-1f);
    y = __builtin_fmaf(y, m, 2.0000714765e-1f);
    y = __builtin_fmaf(y, m, -2.4999993993e-1f);
    y = __builtin_fmaf(y, m, 3.3333331174e-1f);
    y = (y * m) * z;
    float fe = (float)e;
    y = y + (-2.12194440e-4f * fe);
    y = y + (-0.5f * z);
    float r = m + y;
    r = r + (0.693359375f * fe);
    return r;
}

__device__ __forceinline__ float det_sigmoid(float x) { return 1.0f / (1.0f + det_expf(-x)); }

__device__ __forceinline__ float dot3(const float* a, const float* b) { return (a[0] * b[0] + a[1] * b[1]) + a[2] * b[2]; }

// Tile coordinate from a pixel-space float: truncate toward zero like the
// reference's cast (render.py:472-473), clamped to [0, hi].  The float clamp
// first keeps the conversion defined for huge or non-finite inputs.
__device__ __forceinline__ int tile_coord(float v, int hi) {
    v = fminf(fmaxf(v, -1.0f), 1.0e6f);
    int t = (int)v;
    return t < 0 ? 0 : (t > hi ? hi : t);
}

// Unit quaternion in (x,y,z,w) memory order -> rotation matrix, row major.
__device__ __forceinline__ void quat_to_rot(const float q[4], float R[9]) {
    float x = q[0], y = q[1], z = q[2], w = q[3];
    float xx = x * x, yy = y * y, zz = z * z;
    float xy = x * y, xz = x * z, yz = y * z;
    float wx = w * x, wy = w * y, wz = w * z;
    R[0] = 1.0f - 2.0f * (yy + zz);
    R[1] = 2.0f * (xy - wz);
    R[2] = 2.0f * (xz + wy);
    R[3] = 2.0f * (xy + wz);
    R[4] = 1.0f - 2.0f * (xx + zz);
    R[5] = 2.0f * (yz - wx);
    R[6] = 2.0f * (xz - wy);
    R[7] = 2.0f * (yz + wx);
    R[8] = 1.0f - 2.0f * (xx + yy);
}

// Sigma3 = (R diag s)(R diag s)^T as [00,01,02,11,12,22]   (gs3d.py:368-385)
__device__ __forceinline__ void cov3d_from_scale_rot(const float s[3], const float R[9], float c6[6]) {
    float M[9];
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
        for (int j = 0; j < 3; ++j) M[i * 3 + j] = R[i * 3 + j] * s[j];
    c6[0] = dot3(M + 0, M + 0);
    c6[1] = dot3(M + 0, M + 3);
    c6[2] = dot3(M + 0, M + 6);
    c6[3] = dot3(M + 3, M + 3);
    c6[4] = dot3(M + 3, M + 6);
    c6[5] = dot3(M + 6, M + 6);
}

__device__ __forceinline__ void sym3_mv(const float c6[6], const float v[3], float out[3]) {
    out[0] = (c6[0] * v[0] + c6[1] * v[1]) + c6[2] * v[2];
    out[1] = (c6[1] * v[0] + c6[3] * v[1]) + c6[4] * v[2];
    out[2] = (c6[2] * v[0] + c6[4] * v[1]) + c6[5] * v[2];
}

// Rows of T = J W for the EWA projection (gs3d.py:436-456); tx,ty are the
// frustum-clamped camera-space x,y.
__device__ __forceinline__ void ewa_rows(const d3gs_params& P, const float pc[3], float t0[3], float t1[3], float& tx,
                                         float& ty) {
    float limx = fabsf((P.tan_fovx * P.clamp_factor) * pc[2]);
    float limy = fabsf((P.tan_fovy * P.clamp_factor) * pc[2]);
    tx = fminf(fmaxf(pc[0], -limx), limx);
    ty = fminf(fmaxf(pc[1], -limy), limy);
    float zz = pc[2] * pc[2];
    float j00 = P.fx / pc[2];
    float j11 = P.fy / pc[2];
    float j02 = -(tx * P.fx) / zz;
    float j12 = -(ty * P.fy) / zz;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        t0[k] = j00 * P.w2c[0 + k] + j02 * P.w2c[6 + k];
        t1[k] = j11 * P.w2c[3 + k] + j12 * P.w2c[6 + k];
    }
}

// ---------------------------------------------------------------------------
// Tiles touched by one gaussian (render.py:1017-1327).
//
// tile_walk_setup() evaluates, once per gaussian, everything the per-tile test
// needs; tile_keep() is the per-tile predicate.  The preprocess kernel counts
// kept tiles and the key-expansion kernel emits them, both from the same stored
// (uv, radius, conic, opacity), in row-major order (y outer, x inner), so both
// make identical decisions.
//
// Tile counts per gaussian are heavy-tailed (median 4, maximum ~1000 at the
// benchmark scene), so a plain one-thread-per-gaussian loop leaves 63 lanes idle
// behind the largest gaussian of each wavefront.  wave_tile_count()/wave_tile_emit()
// let each lane walk its own gaussian only when it is small, and process the
// large ones cooperatively: the owner's setup is broadcast with v_readlane and
// the 64 lanes test 64 candidate tiles per step.
// ---------------------------------------------------------------------------
struct TileWalkIn {
    float u, v;
    float radius;
    float conic0, conic1, conic2;
    float opacity;
};

struct TileWalk {
    int rminx, rminy, rmaxx, rmaxy;  // 3-sigma tile rect
    int lx0, ly0, lx1, ly1;          // the same rect in candidate-rect coordinates (what the per-tile test compares)
    int bminx, bminy, bw, bh;        // candidate rect (origin, size); the 3-sigma rect when no filter
    float uo, vo, bx, by;            // centre relative to the candidate rect origin, AABB half extents
    float ow, oh, os, oc;            // OBB: axis radii r1, r2 (ow, oh) and sin, cos; ELLIPSE: conic a, b, c and the bound
    float or3, or4;                  // OBB: axis radii r3, r4
};

// Separating-axis test of a 16x16 tile box against the oriented box of a gaussian
// (gs3d.py:1254-1322).  With l1 = (8, 8) the tile half extents, l2 = (w/2, h/2) the box half
// extents and (c, s) the box direction, the four projected-radius sums do not depend on the tile:
// they are formed once per gaussian, in the operation order of the reference's expression
// ((r1 + r2) + r3) + r4, and the per-tile work is the projection of the centre offset on each
// axis.  With NaN sin/cos every "<=" is false, so the tile is kept.
struct ObbAxes { float r1, r2, r3, r4, s, c; };
__device__ __forceinline__ ObbAxes obb_axes(float w, float h, float s, float c) {
    const float l1x = 8.0f, l1y = 8.0f, l2x = w / 2.0f, l2y = h / 2.0f;
    ObbAxes a;
    a.r1 = ((l1x * 1.0f + l1y * 0.0f) + l2x * fabsf(c)) + l2y * fabsf(-s);
    a.r2 = ((l1x * 0.0f + l1y * 1.0f) + l2x * fabsf(s)) + l2y * fabsf(c);
    a.r3 = ((l1x * fabsf(c) + l1y * fabsf(s)) + l2x * fabsf(c * c + s * s)) + l2y * fabsf((-s) * c + c * s);
    a.r4 = ((l1x * fabsf(-s) + l1y * fabsf(c)) + l2x * fabsf(c * (-s) + s * c)) + l2y * fabsf((-s) * (-s) + c * c);
    a.s = s;
    a.c = c;
    return a;
}
__device__ __forceinline__ bool obb_overlaps_tile(float bx0, float by0, const ObbAxes& a, float cu, float cv) {
    const float lx = (bx0 + 8.0f) - cu, ly = (by0 + 8.0f) - cv;   // (bx1 + bx0) / 2 is exactly bx0 + 8
    // all four axes, no early way out: in a wavefront some lane nearly always needs every one of them
    const bool s1 = a.r1 <= fabsf(lx), s2 = a.r2 <= fabsf(ly);
    const bool s3 = a.r3 <= fabsf(lx * a.c + ly * a.s), s4 = a.r4 <= fabsf(lx * (-a.s) + ly * a.c);
    return !(s1 | s2 | s3 | s4);
}

// Where the level set {conic form = -bound} crosses a horizontal (axis = 1) or vertical (axis = 0)
// line (gs3d.py:1149-1178, 1210-1240; coordinates relative to the centre).  lo = hi = -1 on a miss.
struct EllipseCut { float lo, hi; };
__device__ __forceinline__ EllipseCut ellipse_cut(int axis, float line, float cu, float cv, float cx, float cy,
                                                  float cz, float bound) {
    const float own = axis ? cv : cu, other = axis ? cu : cv, lead = axis ? cx : cz;
    const float t = line - own;
    const float val = (((-bound) * lead) - ((cx * cz) * t) * t) + ((cy * cy) * t) * t;
    EllipseCut r{-1.0f, -1.0f};
    if (val >= 0.0f) {
        const float sq = sqrtf(fmaxf(0.0f, val));
        r.lo = other + ((-cy) * t - sq) / lead;
        r.hi = other + ((-cy) * t + sq) / lead;
    }
    return r;
}

// gs3d.py:1078-1117: an edge line cuts the ellipse inside the edge, or the ellipse covers the box,
// or its centre lies in the box.
__device__ __forceinline__ bool ellipse_overlaps_box(float bx0, float by0, float bx1, float by1, float cx, float cy,
                                                     float cz, float bound, float cu, float cv) {
    const EllipseCut x0 = ellipse_cut(0, bx0, cu, cv, cx, cy, cz, bound), x1 = ellipse_cut(0, bx1, cu, cv, cx, cy, cz, bound);
    const EllipseCut y0 = ellipse_cut(1, by0, cu, cv, cx, cy, cz, bound), y1 = ellipse_cut(1, by1, cu, cv, cx, cy, cz, bound);
    auto in = [](float v, float lo, float hi) { return v >= lo && v <= hi; };
    const bool valid = in(x0.lo, by0, by1) || in(x0.hi, by0, by1) || in(x1.lo, by0, by1) || in(x1.hi, by0, by1) ||
                       in(y0.lo, bx0, bx1) || in(y0.hi, bx0, bx1) || in(y1.lo, bx0, bx1) || in(y1.hi, bx0, bx1);
    const bool cover = x0.lo <= by0 && x0.hi >= by1 && x1.lo <= by0 && x1.hi >= by1 && y0.lo <= bx0 && y0.hi >= bx1 &&
                       y1.lo <= bx0 && y1.hi >= bx1;
    const bool centre = bx0 <= cu && bx1 >= cu && by0 <= cv && by1 >= cv;
    return valid || cover || centre;
}

__device__ __forceinline__ TileWalk tile_walk_setup(const d3gs_params& P, const TileWalkIn& g) {
    const int TX = P.tiles_x, TY = P.tiles_y;
    TileWalk w;
    w.rminx = tile_coord((g.u - g.radius) / 16.0f, TX);
    w.rminy = tile_coord((g.v - g.radius) / 16.0f, TY);
    w.rmaxx = tile_coord((((g.u + g.radius) + 16.0f) - 1.0f) / 16.0f, TX);
    w.rmaxy = tile_coord((((g.v + g.radius) + 16.0f) - 1.0f) / 16.0f, TY);
    w.uo = w.vo = w.bx = w.by = w.ow = w.oh = w.os = w.oc = w.or3 = w.or4 = 0.0f;
    if (P.filter_algo == D3GS_FILTER_NONE) {
        w.bminx = w.rminx;
        w.bminy = w.rminy;
        w.bw = w.rmaxx - w.rminx;
        w.bh = w.rmaxy - w.rminy;
        w.lx0 = w.ly0 = 0;
        w.lx1 = w.bw;
        w.ly1 = w.bh;
        return w;
    }
    // half extents of the exact alpha >= alpha_eps ellipse (gs3d.py:710-742)
    float bound = 2.0f * det_logf(P.alpha_eps / g.opacity);
    float D = g.conic0 * g.conic2 - g.conic1 * g.conic1;
    float vx = ((-bound) * g.conic2) * D;
    float vy = ((-bound) * g.conic0) * D;
    float bx = sqrtf(fmaxf(0.0f, vx)) / D;
    float by = sqrtf(fmaxf(0.0f, vy)) / D;
    bx = vx > 0.0f ? bx : 0.0f;
    by = vy > 0.0f ? by : 0.0f;
    bx = fabsf(bx);
    by = fabsf(by);
    w.bx = bx;
    w.by = by;
    w.bminx = tile_coord((g.u - bx) / 16.0f, TX);
    w.bminy = tile_coord((g.v - by) / 16.0f, TY);
    int bmaxx = tile_coord(ceilf((g.u + bx) / 16.0f), TX);
    int bmaxy = tile_coord(ceilf((g.v + by) / 16.0f), TY);
    w.bw = max(bmaxx - w.bminx, 0);
    w.bh = max(bmaxy - w.bminy, 0);
    w.uo = g.u - (float)w.bminx * 16.0f;
    w.vo = g.v - (float)w.bminy * 16.0f;
    w.lx0 = w.rminx - w.bminx;
    w.lx1 = w.rmaxx - w.bminx;
    w.ly0 = w.rminy - w.bminy;
    w.ly1 = w.rmaxy - w.bminy;
    if (P.filter_algo == D3GS_FILTER_OBB || P.filter_algo == D3GS_FILTER_OBB_DFVT) {
        // oriented bounding box of the ellipse x^T Q x = 1, Q = -conic / bound (gs3d.py:761-791, 981-987)
        float eA = (-g.conic0) / bound, eC = (-g.conic2) / bound, eB = (-g.conic1) / bound;
        float det = eA * eC - eB * eB;
        float mid = 0.5f * (eA + eC);
        float sq = sqrtf(fmaxf(0.0f, mid * mid - det));
        float e1 = mid + sq, e2 = mid - sq;
        float s1 = e1 > 0.0f ? 1.0f : -1.0f, s2 = e2 > 0.0f ? 1.0f : -1.0f;
        float v2x = e2 - eC, v2y = eB;
        float len = sqrtf(v2x * v2x + v2y * v2y);
        v2x = v2x / len;
        v2y = v2y / len;
        float minor = 1.0f / sqrtf(e1 * s1);
        float major = 1.0f / sqrtf(e2 * s2);
        const ObbAxes ax = obb_axes(major * 2.0f, minor * 2.0f, v2y, v2x);
        w.ow = ax.r1;
        w.oh = ax.r2;
        w.or3 = ax.r3;
        w.or4 = ax.r4;
        w.os = v2y;
        w.oc = v2x;
    } else if (P.filter_algo == D3GS_FILTER_ELLIPSE) {
        w.ow = g.conic0;
        w.oh = g.conic1;
        w.os = g.conic2;
        w.oc = bound;
    }
    return w;
}

// Does the filter keep the candidate tile whose pixel origin, relative to the candidate rect's, is (px0, py0)?
// The filter is a template argument: the walks below run their loops once per filter instead of choosing the
// test anew for every tile.  tile_keep() adds the 3-sigma rect for a tile given by its coordinates (lx, ly).
template <int kFilter>
__device__ __forceinline__ bool tile_test(const TileWalk& w, float px0, float py0) {
    if constexpr (kFilter == D3GS_FILTER_NONE) return true;
    if constexpr (kFilter == D3GS_FILTER_AABB) {
        const float px1 = px0 + 16.0f, py1 = py0 + 16.0f;
        const bool xo = (w.uo - w.bx) <= px1 && (w.uo + w.bx) >= px0;
        const bool yo = (w.vo - w.by) <= py1 && (w.vo + w.by) >= py0;
        return xo && yo;
    } else if constexpr (kFilter == D3GS_FILTER_ELLIPSE) {
        const float px1 = px0 + 16.0f, py1 = py0 + 16.0f;
        return ellipse_overlaps_box(px0, py0, px1, py1, w.ow, w.oh, w.os, w.oc, w.uo, w.vo);
    } else {
        const ObbAxes ax{w.ow, w.oh, w.or3, w.or4, w.os, w.oc};
        return obb_overlaps_tile(px0, py0, ax, w.uo, w.vo);
    }
}
template <int kFilter>
__device__ __forceinline__ bool tile_keep(const TileWalk& w, int lx, int ly) {
    const bool keep = tile_test<kFilter>(w, (float)(lx * 16), (float)(ly * 16));
    return keep && lx >= w.lx0 && lx < w.lx1 && ly >= w.ly0 && ly < w.ly1;      // inside the 3-sigma rect
}

// A lane's walk over its own small candidate rect, row by row: calls visit(t, px0, py0, kept) once per candidate
// tile t.  The
// tile's pixel origin is stepped as a float (multiples of 16, exact), and the 3-sigma rect is compared in the
// same units, so the loop carries no integer coordinates and converts nothing.
template <int kFilter, class Visit>
__device__ __forceinline__ void small_walk(const TileWalk& w, int area, Visit&& visit) {
    const float x_end = (float)(w.bw * 16);
    const float fx0 = (float)(w.lx0 * 16), fx1 = (float)(w.lx1 * 16);
    const float fy0 = (float)(w.ly0 * 16), fy1 = (float)(w.ly1 * 16);
    float px0 = 0.0f, py0 = 0.0f;
    for (int t = 0; t < area; ++t) {
        visit(t, px0, py0, tile_test<kFilter>(w, px0, py0) && px0 >= fx0 && px0 < fx1 && py0 >= fy0 && py0 < fy1);
        px0 += 16.0f;
        const bool wrap = px0 == x_end;
        px0 = wrap ? 0.0f : px0;
        py0 += wrap ? 16.0f : 0.0f;
    }
}

// Runs f(std::integral_constant<int, filter>) for the filter named at run time (OBB_DFVT is computed as OBB).
template <class F>
__device__ __forceinline__ void with_filter(const int filter_algo, F&& f) {
    switch (filter_algo) {
        case D3GS_FILTER_NONE: f(std::integral_constant<int, D3GS_FILTER_NONE>{}); break;
        case D3GS_FILTER_AABB: f(std::integral_constant<int, D3GS_FILTER_AABB>{}); break;
        case D3GS_FILTER_ELLIPSE: f(std::integral_constant<int, D3GS_FILTER_ELLIPSE>{}); break;
        default: f(std::integral_constant<int, D3GS_FILTER_OBB>{}); break;
    }
}

__device__ __forceinline__ int bcast_i(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ float bcast_f(float v, int src) {
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
template <int kFilter>
__device__ __forceinline__ TileWalk bcast_walk(const TileWalk& w, int src) {
    TileWalk r = {};      // (fields the filter's test does not read stay zero)
    r.lx0 = bcast_i(w.lx0, src); r.ly0 = bcast_i(w.ly0, src);
    r.lx1 = bcast_i(w.lx1, src); r.ly1 = bcast_i(w.ly1, src);
    r.bminx = bcast_i(w.bminx, src); r.bminy = bcast_i(w.bminy, src);
    r.bw = bcast_i(w.bw, src); r.bh = bcast_i(w.bh, src);
    if constexpr (kFilter != D3GS_FILTER_NONE) {
        r.uo = bcast_f(w.uo, src); r.vo = bcast_f(w.vo, src);
    }
    if constexpr (kFilter == D3GS_FILTER_AABB) {
        r.bx = bcast_f(w.bx, src); r.by = bcast_f(w.by, src);
    }
    if constexpr (kFilter == D3GS_FILTER_ELLIPSE || kFilter == D3GS_FILTER_OBB) {
        r.ow = bcast_f(w.ow, src); r.oh = bcast_f(w.oh, src);
        r.os = bcast_f(w.os, src); r.oc = bcast_f(w.oc, src);
    }
    if constexpr (kFilter == D3GS_FILTER_OBB) {
        r.or3 = bcast_f(w.or3, src); r.or4 = bcast_f(w.or4, src);
    }
    return r;
}

constexpr int kSmallWalk = 16;  // candidate tiles a lane walks alone before the wavefront takes over

// Compact record of a gaussian's kept tiles, written by the preprocess kernel so that key
// expansion does not repeat the per-tile tests: word 0 is a bit mask over the candidate rect in
// row-major order (bit ly * bw + lx), word 1 packs the rect origin and width.  Gaussians whose
// candidate rect has more than 64 tiles carry no mask (kTileMaskNone) and are walked again.
constexpr unsigned long long kTileMaskHas = 1ull << 40;
__device__ __forceinline__ unsigned long long tile_mask_meta(const TileWalk& w, bool has_mask) {
    return (unsigned long long)(uint32_t)w.bminx | ((unsigned long long)(uint32_t)w.bminy << 16) |
           ((unsigned long long)(uint32_t)w.bw << 32) | (has_mask ? kTileMaskHas : 0ull);
}

// Number of kept tiles of this lane's gaussian.  Must be called by all 64 lanes of a wavefront
// (lanes without a gaussian pass active = false).  `mask` receives the kept-tile bit mask when the
// candidate rect has at most 64 tiles (`has_mask`).
template <int kFilter>
__device__ __forceinline__ int wave_tile_count_with(bool active, const TileWalk& w, unsigned long long& mask,
                                                    bool& has_mask) {
    const int area = active ? w.bw * w.bh : 0;
    has_mask = active && area <= 64 && w.bw <= 64;
    mask = 0ull;
    if constexpr (kFilter == D3GS_FILTER_NONE) {
        if (has_mask) mask = area == 64 ? ~0ull : (1ull << area) - 1ull;
        return area;
    }
    int count = 0;
    const bool big = area > kSmallWalk;
    const float my_inv_bw = 1.0f / (float)w.bw;
    if (!big) {
        static_assert(kSmallWalk <= 32, "the kept tiles of a small walk are collected in one 32-bit word");
        uint32_t kept = 0;
        small_walk<kFilter>(w, area, [&](int t, float, float, bool k) { kept |= (k ? 1u : 0u) << t; });
        count = __popc(kept);
        mask = kept;
    }
    const int lane = threadIdx.x & 63;
    unsigned long long todo = __ballot(big);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        const TileWalk ws = bcast_walk<kFilter>(w, src);
        const int a = ws.bw * ws.bh;
        int c = 0;
        unsigned long long first = 0ull;
        // row of candidate t: exact for the rect sizes a screen can hold.  Every lane divides once for its own
        // gaussian (below the loop); dividing here would be one division per large gaussian, one after the other.
        const float inv_bw = bcast_f(my_inv_bw, src);
        for (int base = 0; base < a; base += 64) {
            const int t = base + lane;
            bool k = false;
            if (t < a) {
                const int ly = (int)(((float)t + 0.5f) * inv_bw);
                k = tile_keep<kFilter>(ws, t - ly * ws.bw, ly);
            }
            const unsigned long long b = __ballot(k);
            if (base == 0) first = b;
            c += __popcll(b);
        }
        if (lane == src) {
            count = c;
            mask = first;   // the whole rect when it has at most 64 tiles
        }
    }
    return count;
}

__device__ __forceinline__ int wave_tile_count(const int filter_algo, bool active, const TileWalk& w,
                                               unsigned long long& mask, bool& has_mask) {
    int count = 0;
    with_filter(filter_algo, [&](auto filter) {
        count = wave_tile_count_with<decltype(filter)::value>(active, w, mask, has_mask);
    });
    return count;
}

// Emits the tiles named by a kept-tile mask through `put(slot, key)`, slot counting from `off`.
template <class Put>
__device__ __forceinline__ void mask_tile_emit(unsigned long long mask, unsigned long long meta, int tiles_x,
                                               uint32_t depth_bits, long long off, long long end, Put&& put) {
    const int bminx = (int)(meta & 0xFFFFu), bminy = (int)((meta >> 16) & 0xFFFFu), bw = (int)((meta >> 32) & 0xFFu);
    const uint32_t recip = bw > 0 ? (65536u + (uint32_t)bw - 1u) / (uint32_t)bw : 0u;  // exact t / bw for t < 64
    while (mask) {
        const int t = __builtin_ctzll(mask);
        mask &= mask - 1;
        const int ly = (int)(((uint32_t)t * recip) >> 16), lx = t - ly * bw;
        if (off < end) {
            const uint64_t tile = (uint64_t)(uint32_t)((ly + bminy) * tiles_x + lx + bminx);
            put(off, (tile << 32) | depth_bits);
        }
        ++off;
    }
}

// Emits (key, value) of every kept tile of this lane's gaussian at [off, end) in row-major tile
// order.  Must be called by all 64 lanes of a wavefront.
template <typename Key>
__device__ __forceinline__ Key make_pair_key(uint64_t tile, uint32_t depth_bits) {
    if constexpr (sizeof(Key) == 8) return (Key)((tile << 32) | depth_bits);
    else return (Key)tile;
}

// Key: uint64_t for (tile << 32) | depth bits, uint32_t for the tile id alone.
template <typename Key, int kFilter>
__device__ __forceinline__ void wave_tile_emit_with(bool active, const TileWalk& w, int tiles_x,
                                               uint32_t depth_bits, int value, long long off, long long end,
                                               Key* __restrict__ keys, int32_t* __restrict__ vals) {
    const int area = active ? w.bw * w.bh : 0;
    const bool big = area > kSmallWalk;
    if (!big) {
        small_walk<kFilter>(w, area, [&](int, float px0, float py0, bool k) {
            if (k) {
                if (off < end) {
                    const int lx = (int)px0 >> 4, ly = (int)py0 >> 4;
                    const uint64_t tile = (uint64_t)(uint32_t)((ly + w.bminy) * tiles_x + lx + w.bminx);
                    keys[off] = make_pair_key<Key>(tile, depth_bits);
                    vals[off] = value;
                }
                ++off;
            }
        });
    }
    const int lane = threadIdx.x & 63;
    const unsigned long long lt_mask = (1ull << lane) - 1ull;
    const float my_inv_bw = 1.0f / (float)w.bw;
    unsigned long long todo = __ballot(big);
    while (todo) {
        const int src = __builtin_ctzll(todo);
        todo &= todo - 1;
        const TileWalk ws = bcast_walk<kFilter>(w, src);
        const uint32_t dbits = (uint32_t)bcast_i((int)depth_bits, src);
        const int val = bcast_i(value, src);
        long long o = ((long long)bcast_i((int)(off >> 32), src) << 32) | (uint32_t)bcast_i((int)off, src);
        const long long e = ((long long)bcast_i((int)(end >> 32), src) << 32) | (uint32_t)bcast_i((int)end, src);
        const int a = ws.bw * ws.bh;
        const float inv_bw = bcast_f(my_inv_bw, src);   // one division per lane, not one per large gaussian
        for (int base = 0; base < a; base += 64) {
            const int t = base + lane;
            bool k = false;
            int lx = 0, ly = 0;
            if (t < a) {
                ly = (int)(((float)t + 0.5f) * inv_bw);
                lx = t - ly * ws.bw;
                k = tile_keep<kFilter>(ws, lx, ly);
            }
            const unsigned long long b = __ballot(k);
            if (k) {
                const long long pos = o + __popcll(b & lt_mask);
                if (pos < e) {
                    const uint64_t tile = (uint64_t)(uint32_t)((ly + ws.bminy) * tiles_x + lx + ws.bminx);
                    keys[pos] = make_pair_key<Key>(tile, dbits);
                    vals[pos] = val;
                }
            }
            o += __popcll(b);
        }
    }
}

template <typename Key>
__device__ __forceinline__ void wave_tile_emit(const int filter_algo, bool active, const TileWalk& w, int tiles_x,
                                               uint32_t depth_bits, int value, long long off, long long end,
                                               Key* __restrict__ keys, int32_t* __restrict__ vals) {
    with_filter(filter_algo, [&](auto filter) {
        wave_tile_emit_with<Key, decltype(filter)::value>(active, w, tiles_x, depth_bits, value, off, end, keys, vals);
    });
}

constexpr float kShC0 = 0.28209479177387814f;
constexpr float kShC1 = 0.4886025119029199f;
__device__ constexpr float kShC2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                                       -1.0925484305920792f, 0.5462742152960396f};
__device__ constexpr float kShC3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f,
                                       0.3731763325901154f, -0.4570457994644658f, 1.445305721320277f,
                                       -0.5900435899266435f};

// Camera bundles: a call with batch_size = B > 1 works on B * n render items, item i = b * n + g.
__host__ __device__ __forceinline__ int batch_count(const d3gs_params& P) { return P.batch_size > 1 ? P.batch_size : 1; }
// render items: gaussians x cameras of a bundle, or sparse mode's compact rows of one
__host__ __device__ __forceinline__ int item_count(const d3gs_params& P) {
    return P.compact_items > 0 ? P.compact_items : P.n * batch_count(P);
}
// Camera b of the bundle into the per-camera fields (what make_params fills for a single camera); tan_fov is
// 0.5 * resolution / focal in float32, as the host computes it (render.py:358).
__device__ __forceinline__ void apply_batch_camera(d3gs_params& P, int b) {
    const float* m = P.batch_cameras + D3GS_BATCH_CAMERA_FLOATS * (size_t)b;
#pragma unroll
    for (int k = 0; k < 9; ++k) P.w2c[k] = m[k];
#pragma unroll
    for (int k = 0; k < 3; ++k) P.cam_center[k] = m[9 + k];
    P.fx = m[12];
    P.fy = m[13];
    P.cx = m[14];
    P.cy = m[15];
    P.tan_fovx = (0.5f * (float)P.width) / P.fx;
    P.tan_fovy = (0.5f * (float)P.height) / P.fy;
}

// Thread-local error string helpers live in capi.hip.
void set_error(const char* fmt, ...);
// Validates sizes / enum values of a params block (defined in preprocess.hip).
int check_params(const d3gs_params* p, const char* who);
// d3gs_tile_ranges_u32 whose last kernel also folds the error words of up to two sort workspaces into the
// pair-count words: D3GS_COUNT_SORT_GAVE_UP replaces the count when either is set (defined in binning.hip).
// publish_host: that kernel is the only one to write *total_host, count or status, by a store the host can poll for.
int tile_ranges_u32_with_status(const uint32_t* tile_keys_sorted, int64_t m, const int64_t* m_device,
                                int32_t* workload_ranges, int32_t num_tiles, int32_t* tile_order,
                                const uint32_t* sort_error_a, const uint32_t* sort_error_b, int64_t* total_dev,
                                int64_t* total_host, bool publish_host, d3gs_stream_t stream);

// value of the sorts' workspace_is_zero argument
constexpr int kSortWorkspaceIsZero = 1;
// The one-call binning on 16-bit tile ids (binning.hip, radix_sort.hip): key expansion, pair sort and tile ranges
// over uint16 keys; arguments as the 32-bit entry points'.
int make_tile_keys_u16(const d3gs_params* p, const int32_t* radii, const float* uvs, const float* conic_opacity,
                       const float* depths, const int32_t* offsets, const int32_t* gaussian_order,
                       const uint32_t* ordered_depth_keys, const uint64_t* tile_masks, uint16_t* tile_keys,
                       int32_t* gaussian_idx, int64_t m, d3gs_stream_t stream);
int sort_pairs_u16(uint16_t* keys_a, uint16_t* keys_b, int32_t* vals_a, int32_t* vals_b, void* workspace,
                   size_t workspace_bytes, int64_t m, const int64_t* m_device, int workspace_is_zero, int end_bit,
                   int* result_in_b_host, d3gs_stream_t stream);
int tile_ranges_u16_with_status(const uint16_t* tile_keys_sorted, int64_t m, const int64_t* m_device,
                                int32_t* workload_ranges, int32_t num_tiles, int32_t* tile_order,
                                const uint32_t* sort_error_a, const uint32_t* sort_error_b, int64_t* total_dev,
                                int64_t* total_host, bool publish_host, d3gs_stream_t stream);

// Depth part of the reference's sort key (render.py:767-775): the float bits (positive floats order like their
// bit patterns), or with enable_32bit_sort the depth in steps of depth_32bit_prec, truncated to 18 bits.
__device__ __forceinline__ uint32_t reference_depth_bits(const d3gs_params& P, float z) {
    if (P.enable_32bit_sort) return (uint32_t)(z / P.depth_32bit_prec) & ((1u << kDepthStepBits) - 1u);
    return __float_as_uint(z);
}

// Key of the depth sort that orders the gaussians ahead of the pair sort: the same order as the reference's
// depth bits in fewer significant bits.  Accepted depths lie in [z_near, z_far], so their float bits minus those
// of z_near fit d3gs_depth_key_bits() bits (27 for the default planes, three 9-bit digits instead of four
// 8-bit ones); rejected gaussians (depth written as 0) get key 0.
__host__ __device__ __forceinline__ uint32_t depth_key_base(const d3gs_params& P) {
    union { float f; uint32_t u; } low;
    // smallest stored value of an accepted gaussian: z_near, or with render_inv_depth 1 / z_far (division rounds
    // monotonically, so 1 / z of every z <= z_far is at least that)
    low.f = P.render_inv_depth ? (P.z_far > 0.0f ? 1.0f / P.z_far : 0.0f) : P.z_near;
    return low.f > 0.0f ? low.u : 0u;
}
// v: the value K1 stores in `depths` (z, or 1 / z with render_inv_depth; 0 for a rejected gaussian)
__device__ __forceinline__ uint32_t depth_sort_key(const d3gs_params& P, float v) {
    if (P.enable_32bit_sort) return reference_depth_bits(P, v);
    const uint32_t bits = __float_as_uint(v), base = depth_key_base(P);
    return v > 0.0f && bits >= base ? bits - base : 0u;
}

}  // namespace d3gs
