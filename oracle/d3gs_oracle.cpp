// CPU oracle for the 3DGS rasterize forward/backward path.
//
// THIS FILE IS TEST INFRASTRUCTURE. It is a from-text restatement, in plain
// C++ on float32, of the algorithm the reference implements as JIT-compiled
// CUDA strings.  Only tests/, __graft_entry__.smoke() and bench.py's
// cpu_baseline leg may load it; the product (the HIP library) never does.
//
// Reference files restated (paths relative to the reference checkout):
//   d3sim/algos/d3gs/render.py   : preprocess 421-476,569-619; tile filters
//                                  1017-1327; key expansion 745-840; tile
//                                  ranges 897-939; blend fwd/bwd 1466-2294;
//                                  preprocess backward 3217-3356
//   d3sim/csrc/gs3d.py           : SH 151-366, cov3d 368-418, EWA 420-532,
//                                  conic/det 535-588, radius 684-708,
//                                  ellipse bounds 710-791,968-989, SAT 1239-1322
//   d3sim/csrc/camera.py         : pinhole projection 307-371
//   d3sim/algos/d3gs/origin/model.py : fused activations 281-295,332-383,452-462
//   d3sim/csrc/devsort.py        : radix sort with bit range 77-129, msb 131-149
//
// Pinning status (what independent evidence checks each function; see
// tests/test_oracle_*.py):
//   orc_expf / orc_logf          : against float64 libm, <= 1.5 ulp
//   orc_expf_blend               : the same, over the range the blend evaluates it in
//   orc_preprocess_fwd           : float64 closed forms (pinhole, R S S^T R^T via
//                                  scipy Rotation, EWA J W S W^T J^T, 2x2 inverse,
//                                  eigen radius), SH against a float64 restatement
//                                  of the in-tree Inria eval_sh table
//   tile filters NONE/AABB/OBB   : from both sides: brute-force per-pixel losslessness and the
//                                  subset chain bound them from below; from above, AABB must equal
//                                  the tiles meeting the float64 box u +- sqrt(L Sigma_ii) and OBB the
//                                  tiles meeting the oriented rectangle built with numpy eigh and an
//                                  independent separating-axis test (tiles within 1e-3 of a boundary
//                                  skipped); ELLIPSE inside OBB; an isotropic conic (NaN axis) keeps
//                                  every candidate tile
//   OBB_DFVT                     : implemented as the OBB tile set (the author's
//                                  stated invariant, render.py:1051-1072); the
//                                  third-party cumm OBBCornersGridOverlap::inc_step
//                                  rounding is absent here -> "parity unpinned"
//   orc_scan/make_keys/sort/ranges : numpy cumsum + stable argsort, partition invariants; the 32-bit
//                                  key mode against numpy float32 division + stable lexsort
//   orc_blend_fwd                : float64 dense per-pixel restatement in numpy
//   orc_blend_bwd / orc_preprocess_bwd : float64 torch autograd of the forward
//                                  (straight-through alpha clamp) + finite differences
//   instance cameras             : identity poses / negative ids are no-ops, one instance equals
//                                  the plain render by the composed camera, an SH-0 render equals
//                                  the render of the gaussians moved to the world frame; the
//                                  reference composes the pose in float32 with third-party cumm
//                                  array ops whose rounding is absent here -> "parity unpinned"
//   exp used in the blend        : the reference uses CUDA __expf (approximate,
//                                  rounding unspecified); this oracle and the HIP
//                                  kernels use orc_expf's exact operation sequence so
//                                  per-pixel threshold decisions agree -> the
//                                  reference's own rounding is "parity unpinned"
//
// All float32 arithmetic below is written as explicit single operations and the
// file is compiled with -ffp-contract=off: fused multiply-adds appear only where
// fmaf() is spelled out.  The HIP kernels follow the same operation order, which
// is what makes the integer outputs (radii, tile counts, keys) bit-comparable.

#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>
#include <algorithm>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API extern "C"

enum { ORC_FILTER_NONE = 0, ORC_FILTER_AABB = 1, ORC_FILTER_ELLIPSE = 2, ORC_FILTER_OBB = 3, ORC_FILTER_OBB_DFVT = 4 };

struct orc_params {
    int32_t n;            // gaussians
    int32_t width, height;
    int32_t tiles_x, tiles_y;
    int32_t sh_degree;    // evaluated degree (cur_sh_degree), 0..3
    int32_t sh_stride;    // coefficients per gaussian stored in color_sh (K)
    int32_t has_sh_base;  // DC stored separately in color_sh_base
    int32_t filter_algo;
    int32_t training;
    float fx, fy, cx, cy;
    float tan_fovx, tan_fovy;
    float w2c[9];         // rows of the world->camera rotation (= rows 0..2 of cam2world_T)
    float cam_center[3];  // row 3 of cam2world_T
    float z_near, z_far;
    float eps;            // conic det eps (config eps)
    float radii_eigen_eps;
    float clamp_factor;
    float std_sigma;
    float lowpass;
    float alpha_eps;
    float transmittance_eps;
    float scale_global;
    float bg[3];
    int32_t fused_activation;  // 1: raw tensors, activations applied here; 0: already activated
    int32_t render_depth;          // blend the camera-space depth as one more channel (render.py:1532-1539)
    int32_t render_rgba;           // fourth colour channel = sum of blend weights (render.py:1899-1906)
    int32_t use_nchw;              // colour image stored [C,H,W] instead of [H,W,C] (render.py:702)
    int32_t enable_anti_aliasing;  // opacity scaled by sqrt(det / det_lowpass) (render.py:391-407)
    int32_t enable_32bit_sort;     // key = (tile << 18) | (uint32(depth / prec) & 0x3FFFF) (render.py:767-770, 820)
    float depth_32bit_prec;        // config_def.py:91
    int32_t render_inv_depth;      // K1 stores 1 / z where it stores z otherwise (render.py:582): the buffer is also the
                                   // sort key's depth part (render.py:773), so the lists come out in descending z
};

// ---------------------------------------------------------------------------
// Deterministic transcendental functions (Cephes-style single precision).
// ---------------------------------------------------------------------------
ORC_API float orc_expf(float x) {
    if (!(x == x)) return x;
    if (x < -86.0f) return 0.0f;
    if (x > 88.0f) return INFINITY;
    float kf = rintf(x * 1.44269504088896341f);
    float r = fmaf(kf, -0.693359375f, x);
    r = fmaf(kf, 2.12194440e-4f, r);
    float z = r * r;
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float e = fmaf(p, z, r) + 1.0f;
    return ldexpf(e, (int)kf);
}

// exp as the blend kernels evaluate it (device_math.h: det_expf_inrange): orc_expf's polynomial with a range
// reduction that costs the GPU less -- k from one fused multiply-add with 1.5 * 2^23 instead of a multiply and
// a round (the two differ only where x log2 e is within a rounding of a half-integer, and then by which of two
// equally good k is taken).  Below -80, where the kernels never evaluate it, the plain function.
ORC_API float orc_expf_blend(float x) {
    if (!(x == x) || x < -80.0f || x > 80.0f) return orc_expf(x);
    const float t = fmaf(x, 1.44269504088896341f, 12582912.0f);
    const float kf = t - 12582912.0f;
    float r = fmaf(kf, -0.693359375f, x);
    r = fmaf(kf, 2.12194440e-4f, r);
    float z = r * r;
    float p = 1.9875691500e-4f;
    p = fmaf(p, r, 1.3981999507e-3f);
    p = fmaf(p, r, 8.3334519073e-3f);
    p = fmaf(p, r, 4.1665795894e-2f);
    p = fmaf(p, r, 1.6666665459e-1f);
    p = fmaf(p, r, 5.0000001201e-1f);
    float e = fmaf(p, z, r) + 1.0f;
    return ldexpf(e, (int)kf);
}

ORC_API float orc_logf(float x) {
    if (!(x > 0.0f)) return -INFINITY;
    if (x < 1.17549435e-38f) x = 1.17549435e-38f;
    uint32_t ix;
    memcpy(&ix, &x, 4);
    int e = (int)(ix >> 23) - 126;               // x = m * 2^e, m in [0.5, 1)
    uint32_t im = (ix & 0x007fffffu) | 0x3f000000u;
    float m;
    memcpy(&m, &im, 4);
    if (m < 0.707106781186547524f) {
        e -= 1;
        m = (m + m) - 1.0f;
    } else {
        m = m - 1.0f;
    }
    float z = m * m;
    float y = 7.0376836292e-2f;
    y = fmaf(y, m, -1.1514610310e-1f);
    y = fmaf(y, m, 1.1676998740e-1f);
    y = fmaf(y, m, -1.2420140846e-1f);
    y = fmaf(y, m, 1.4249322787e-1f);
    y = fmaf(y, m, -1.6668057665e-1f);
    y = fmaf(y, m, 2.0000714765e-1f);
    y = fmaf(y, m, -2.4999993993e-1f);
    y = fmaf(y, m, 3.3333331174e-1f);
    y = (y * m) * z;
    float fe = (float)e;
    y = y + (-2.12194440e-4f * fe);
    y = y + (-0.5f * z);
    float r = m + y;
    r = r + (0.693359375f * fe);
    return r;
}

static inline float sigmoidf_det(float x) { return 1.0f / (1.0f + orc_expf(-x)); }

// (int) cast of a float that is later clamped to [0, hi]; the pre-clamp makes the
// cast defined for huge / non-finite values (render.py:472-473 uses a raw cast).
static inline int tile_coord(float v, int hi) {
    v = fminf(fmaxf(v, -1.0f), 1.0e6f);
    int t = (int)v;
    return t < 0 ? 0 : (t > hi ? hi : t);
}

static const float SH_C0 = 0.28209479177387814f;
static const float SH_C1 = 0.4886025119029199f;
static const float SH_C2[5] = {1.0925484305920792f, -1.0925484305920792f, 0.31539156525252005f,
                               -1.0925484305920792f, 0.5462742152960396f};
static const float SH_C3[7] = {-0.5900435899266435f, 2.890611442640554f, -0.4570457994644658f, 0.3731763325901154f,
                               -0.4570457994644658f, 1.445305721320277f, -0.5900435899266435f};

// quaternion (x,y,z,w), unit -> rotation matrix rows (scalar-last memory order, origin/model.py:37-38)
static inline void quat_to_rot(const float q[4], float R[9]) {
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

static inline float dot3(const float* a, const float* b) { return (a[0] * b[0] + a[1] * b[1]) + a[2] * b[2]; }

// scale+quat -> 6-vector covariance [00,01,02,11,12,22]  (gs3d.py:368-385)
static inline void cov3d_from_scale_rot(const float s[3], const float R[9], float c6[6]) {
    float M[9];
    for (int i = 0; i < 3; ++i)
        for (int j = 0; j < 3; ++j) M[i * 3 + j] = R[i * 3 + j] * s[j];
    c6[0] = dot3(M + 0, M + 0);
    c6[1] = dot3(M + 0, M + 3);
    c6[2] = dot3(M + 0, M + 6);
    c6[3] = dot3(M + 3, M + 3);
    c6[4] = dot3(M + 3, M + 6);
    c6[5] = dot3(M + 6, M + 6);
}

// Rows of T = J W (2x3) for the EWA projection (gs3d.py:436-456).
static inline void ewa_rows(const orc_params* P, const float pc[3], float t0[3], float t1[3], float* txc, float* tyc) {
    float limx = fabsf((P->tan_fovx * P->clamp_factor) * pc[2]);
    float limy = fabsf((P->tan_fovy * P->clamp_factor) * pc[2]);
    float tx = fminf(fmaxf(pc[0], -limx), limx);
    float ty = fminf(fmaxf(pc[1], -limy), limy);
    float zz = pc[2] * pc[2];
    float j00 = P->fx / pc[2];
    float j11 = P->fy / pc[2];
    float j02 = -(tx * P->fx) / zz;
    float j12 = -(ty * P->fy) / zz;
    const float* W = P->w2c;
    for (int k = 0; k < 3; ++k) {
        t0[k] = j00 * W[0 + k] + j02 * W[6 + k];
        t1[k] = j11 * W[3 + k] + j12 * W[6 + k];
    }
    *txc = tx;
    *tyc = ty;
}

static inline void sym3_mv(const float c6[6], const float v[3], float out[3]) {
    out[0] = (c6[0] * v[0] + c6[1] * v[1]) + c6[2] * v[2];
    out[1] = (c6[1] * v[0] + c6[3] * v[1]) + c6[4] * v[2];
    out[2] = (c6[2] * v[0] + c6[4] * v[1]) + c6[5] * v[2];
}

// SH basis evaluation (gs3d.py:151-201).  sh points at coefficient 1 (first non-DC).
static inline void sh_to_rgb(int degree, const float dir[3], const float* base, const float* sh, float rgb[3]) {
    float x = dir[0], y = dir[1], z = dir[2];
    for (int ch = 0; ch < 3; ++ch) {
        float r = SH_C0 * base[ch];
        if (degree > 0) {
            r = ((r - (SH_C1 * y) * sh[0 * 3 + ch]) + (SH_C1 * z) * sh[1 * 3 + ch]) - (SH_C1 * x) * sh[2 * 3 + ch];
            if (degree > 1) {
                float xx = x * x, yy = y * y, zz = z * z;
                float xy = x * y, yz = y * z, xz = x * z;
                r = r + (SH_C2[0] * xy) * sh[3 * 3 + ch];
                r = r + (SH_C2[1] * yz) * sh[4 * 3 + ch];
                r = r + (SH_C2[2] * ((2.0f * zz - xx) - yy)) * sh[5 * 3 + ch];
                r = r + (SH_C2[3] * xz) * sh[6 * 3 + ch];
                r = r + (SH_C2[4] * (xx - yy)) * sh[7 * 3 + ch];
                if (degree > 2) {
                    r = r + ((SH_C3[0] * y) * (3.0f * xx - yy)) * sh[8 * 3 + ch];
                    r = r + ((SH_C3[1] * xy) * z) * sh[9 * 3 + ch];
                    r = r + ((SH_C3[2] * y) * ((4.0f * zz - xx) - yy)) * sh[10 * 3 + ch];
                    r = r + ((SH_C3[3] * z) * ((2.0f * zz - 3.0f * xx) - 3.0f * yy)) * sh[11 * 3 + ch];
                    r = r + ((SH_C3[4] * x) * ((4.0f * zz - xx) - yy)) * sh[12 * 3 + ch];
                    r = r + ((SH_C3[5] * z) * (xx - yy)) * sh[13 * 3 + ch];
                    r = r + ((SH_C3[6] * x) * (xx - 3.0f * yy)) * sh[14 * 3 + ch];
                }
            }
        }
        rgb[ch] = r + 0.5f;
    }
}

// ---------------------------------------------------------------------------
// Tile walk shared by preprocess (count) and key expansion (emit).
// Visits the tiles a gaussian touches in row-major order (y outer, x inner) and
// calls f(x, y) for each kept tile.  (render.py:1017-1327)
// ---------------------------------------------------------------------------
struct TileWalkIn {
    float u, v;        // pixel-space centre
    float radius;      // 3-sigma radius (already ceil'ed), as float
    float conic[3];
    float opacity;
};

static inline bool obb_overlaps_box(float bx0, float by0, float bx1, float by1, const float whsc[4], float cu, float cv) {
    // separating-axis test, gs3d.py:1254-1322; NaN sin/cos make every "<=" false -> kept
    float s = whsc[2], c = whsc[3];
    float l1x = (bx1 - bx0) / 2.0f, l1y = (by1 - by0) / 2.0f;
    float l2x = whsc[0] / 2.0f, l2y = whsc[1] / 2.0f;
    float lx = (bx1 + bx0) / 2.0f - cu, ly = (by1 + by0) / 2.0f - cv;
    float r1, r2, r3, r4;
    // axis a1 = (1,0)
    r1 = l1x * 1.0f; r2 = l1y * 0.0f; r3 = l2x * fabsf(c); r4 = l2y * fabsf(-s);
    if (((r1 + r2) + r3) + r4 <= fabsf(lx)) return false;
    // axis a2 = (0,1)
    r1 = l1x * 0.0f; r2 = l1y * 1.0f; r3 = l2x * fabsf(s); r4 = l2y * fabsf(c);
    if (((r1 + r2) + r3) + r4 <= fabsf(ly)) return false;
    // axis a3 = (c,s)
    r1 = l1x * fabsf(c); r2 = l1y * fabsf(s); r3 = l2x * fabsf(c * c + s * s); r4 = l2y * fabsf((-s) * c + c * s);
    if (((r1 + r2) + r3) + r4 <= fabsf(lx * c + ly * s)) return false;
    // axis a4 = (-s,c)
    r1 = l1x * fabsf(-s); r2 = l1y * fabsf(c); r3 = l2x * fabsf(c * (-s) + s * c); r4 = l2y * fabsf((-s) * (-s) + c * c);
    if (((r1 + r2) + r3) + r4 <= fabsf(lx * (-s) + ly * c)) return false;
    return true;
}

// Where the level set {conic form = -bound} crosses a horizontal (axis = 1) or vertical (axis = 0)
// line, gs3d.py:1149-1178 / 1210-1240 ("_v2": coordinates relative to the centre).  lo = hi = -1 when
// the line misses the ellipse.
struct EllipseCut { float lo, hi; };
static inline EllipseCut ellipse_cut(int axis, float line, float cu, float cv, const float conic[3], float bound) {
    const float cx = conic[0], cy = conic[1], cz = conic[2];
    const float own = axis ? cv : cu;      // centre coordinate along the line's normal
    const float other = axis ? cu : cv;    // centre coordinate along the line
    const float lead = axis ? cx : cz;     // coefficient of the unknown squared
    const float t = line - own;
    const float val = (((-bound) * lead) - ((cx * cz) * t) * t) + ((cy * cy) * t) * t;
    if (!(val >= 0.0f)) return {-1.0f, -1.0f};
    const float sq = sqrtf(fmaxf(0.0f, val));
    return {other + ((-cy) * t - sq) / lead, other + ((-cy) * t + sq) / lead};
}

// gs3d.py:1078-1117: the ellipse touches the box when an edge line cuts it inside the edge, when it
// covers the whole box, or when its centre lies in the box.
static inline bool ellipse_overlaps_box(float bx0, float by0, float bx1, float by1, const float conic[3], float bound,
                                        float cu, float cv) {
    const EllipseCut x0 = ellipse_cut(0, bx0, cu, cv, conic, bound), x1 = ellipse_cut(0, bx1, cu, cv, conic, bound);
    const EllipseCut y0 = ellipse_cut(1, by0, cu, cv, conic, bound), y1 = ellipse_cut(1, by1, cu, cv, conic, bound);
    auto in = [](float v, float lo, float hi) { return v >= lo && v <= hi; };
    bool valid = in(x0.lo, by0, by1) || in(x0.hi, by0, by1) || in(x1.lo, by0, by1) || in(x1.hi, by0, by1) ||
                 in(y0.lo, bx0, bx1) || in(y0.hi, bx0, bx1) || in(y1.lo, bx0, bx1) || in(y1.hi, bx0, bx1);
    bool cover = x0.lo <= by0 && x0.hi >= by1 && x1.lo <= by0 && x1.hi >= by1 && y0.lo <= bx0 && y0.hi >= bx1 &&
                 y1.lo <= bx0 && y1.hi >= bx1;
    bool centre = bx0 <= cu && bx1 >= cu && by0 <= cv && by1 >= cv;
    return valid || cover || centre;
}

template <class F>
static inline int tile_walk(const orc_params* P, const TileWalkIn& g, F&& f) {
    const int TX = P->tiles_x, TY = P->tiles_y;
    int rminx = tile_coord((g.u - g.radius) / 16.0f, TX);
    int rminy = tile_coord((g.v - g.radius) / 16.0f, TY);
    int rmaxx = tile_coord((((g.u + g.radius) + 16.0f) - 1.0f) / 16.0f, TX);
    int rmaxy = tile_coord((((g.v + g.radius) + 16.0f) - 1.0f) / 16.0f, TY);
    int count = 0;
    if (P->filter_algo == ORC_FILTER_NONE) {
        for (int y = rminy; y < rmaxy; ++y)
            for (int x = rminx; x < rmaxx; ++x) { f(x, y); ++count; }
        return count;
    }
    // exact alpha >= alpha_eps ellipse: conic quadratic form <= -bound  (render.py:1019-1028)
    float bound = 2.0f * orc_logf(P->alpha_eps / g.opacity);
    float D = g.conic[0] * g.conic[2] - g.conic[1] * g.conic[1];
    float vx = ((-bound) * g.conic[2]) * D;
    float vy = ((-bound) * g.conic[0]) * D;
    float bx = sqrtf(fmaxf(0.0f, vx)) / D;
    float by = sqrtf(fmaxf(0.0f, vy)) / D;
    bx = vx > 0.0f ? bx : 0.0f;
    by = vy > 0.0f ? by : 0.0f;
    bx = fabsf(bx);
    by = fabsf(by);
    int bminx = tile_coord((g.u - bx) / 16.0f, TX);
    int bminy = tile_coord((g.v - by) / 16.0f, TY);
    int bmaxx = tile_coord(ceilf((g.u + bx) / 16.0f), TX);
    int bmaxy = tile_coord(ceilf((g.v + by) / 16.0f), TY);
    float uo = g.u - (float)bminx * 16.0f;
    float vo = g.v - (float)bminy * 16.0f;
    float whsc[4] = {0, 0, 0, 0};
    if (P->filter_algo == ORC_FILTER_OBB || P->filter_algo == ORC_FILTER_OBB_DFVT) {
        // gs3d.py:761-791, 981-987
        float eA = (-g.conic[0]) / bound, eC = (-g.conic[2]) / bound, eB = (-g.conic[1]) / bound;
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
        // the reference re-normalises (v2*major); for a unit v2 this is v2 again up to
        // sign(major) > 0, so sin/cos are v2's components
        whsc[0] = major * 2.0f;
        whsc[1] = minor * 2.0f;
        whsc[2] = v2y;
        whsc[3] = v2x;
    }
    for (int y = bminy; y < bmaxy; ++y) {
        float py0 = (float)((y - bminy) * 16);
        float py1 = py0 + 16.0f;
        for (int x = bminx; x < bmaxx; ++x) {
            float px0 = (float)((x - bminx) * 16);
            float px1 = px0 + 16.0f;
            bool keep;
            if (P->filter_algo == ORC_FILTER_AABB) {
                bool xo = (uo - bx) <= px1 && (uo + bx) >= px0;
                bool yo = (vo - by) <= py1 && (vo + by) >= py0;
                keep = xo && yo;
            } else if (P->filter_algo == ORC_FILTER_ELLIPSE) {
                keep = ellipse_overlaps_box(px0, py0, px1, py1, g.conic, bound, uo, vo);
            } else {
                keep = obb_overlaps_box(px0, py0, px1, py1, whsc, uo, vo);
            }
            keep = keep && x >= rminx && x < rmaxx && y >= rminy && y < rmaxy;
            if (keep) { f(x, y); ++count; }
        }
    }
    return count;
}

// ---------------------------------------------------------------------------
// K1 preprocess forward (render.py:421-476, 569-619)
// Outputs of invalid gaussians are zero-filled (the reference leaves them
// uninitialised).
// ---------------------------------------------------------------------------
// Instance rendering (render.py:346-356): gaussian i with instance_ids[i] = k in [0, num_instances) is seen by
// the camera expressed in the frame of instance k, instance_cameras[k] = world-to-camera rotation (9, row major) +
// camera centre (3) in that frame; the others by the view's camera.
static inline orc_params with_instance(const orc_params* P, const int32_t* instance_ids, const float* instance_cameras,
                                       int32_t num_instances, int i) {
    orc_params L = *P;
    if (instance_ids) {
        const int id = instance_ids[i];
        if (id >= 0 && id < num_instances) {
            for (int k = 0; k < 9; ++k) L.w2c[k] = instance_cameras[12 * (size_t)id + k];
            for (int k = 0; k < 3; ++k) L.cam_center[k] = instance_cameras[12 * (size_t)id + 9 + k];
        }
    }
    return L;
}

ORC_API int orc_preprocess_fwd(const orc_params* P0, const float* xyz, const float* quat, const float* scale,
                       const float* opacity, const float* sh, const float* sh_base, const uint8_t* invalid_mask,
                       float* depths, int32_t* radii,
                       float* uvs, float* conic_opacity, int32_t* tiles_touched, float* rgb_out, float* cov2d_out,
                       uint8_t* ne0_out, const int32_t* instance_ids, const float* instance_cameras,
                       int32_t num_instances) {
    const int n = P0->n;
#pragma omp parallel for schedule(dynamic, 1024)
    for (int i = 0; i < n; ++i) {
        const orc_params Pl = with_instance(P0, instance_ids, instance_cameras, num_instances, i);
        const orc_params* P = &Pl;
        depths[i] = 0.0f;
        radii[i] = 0;
        uvs[2 * i] = uvs[2 * i + 1] = 0.0f;
        for (int k = 0; k < 4; ++k) conic_opacity[4 * i + k] = 0.0f;
        tiles_touched[i] = 0;
        for (int k = 0; k < 3; ++k) rgb_out[3 * i + k] = 0.0f;
        if (cov2d_out)
            for (int k = 0; k < 3; ++k) cov2d_out[3 * i + k] = 0.0f;
        if (ne0_out) ne0_out[i] = 0;

        float d[3] = {xyz[3 * i] - P->cam_center[0], xyz[3 * i + 1] - P->cam_center[1], xyz[3 * i + 2] - P->cam_center[2]};
        float pc[3] = {dot3(P->w2c + 0, d), dot3(P->w2c + 3, d), dot3(P->w2c + 6, d)};
        float z = pc[2];
        if (!(z >= P->z_near && z <= P->z_far)) continue;
        if (invalid_mask && invalid_mask[i]) continue;  // render.py:306-308
        float u = ((pc[0] / z) * P->fx + P->cx) - 0.5f;
        float v = ((pc[1] / z) * P->fy + P->cy) - 0.5f;

        // fused activations (origin/model.py:281-295, 452-462)
        const float* qr = quat + 4 * i;
        float qn = 1.0f;
        float q[4] = {qr[0], qr[1], qr[2], qr[3]};
        float s[3] = {scale[3 * i], scale[3 * i + 1], scale[3 * i + 2]};
        if (P->fused_activation) {
            qn = sqrtf(((qr[0] * qr[0] + qr[1] * qr[1]) + qr[2] * qr[2]) + qr[3] * qr[3]);
            for (int k = 0; k < 4; ++k) q[k] = qr[k] / qn;
            for (int k = 0; k < 3; ++k) s[k] = orc_expf(s[k]);
        }
        if (!P->training) {
            s[0] = s[0] * P->scale_global;
            s[1] = s[1] * P->scale_global;
            s[2] = s[2] * P->scale_global;
        }
        float R[9], c6[6];
        quat_to_rot(q, R);
        cov3d_from_scale_rot(s, R, c6);

        float t0[3], t1[3], tx, ty;
        ewa_rows(P, pc, t0, t1, &tx, &ty);
        float v0[3], v1[3];
        sym3_mv(c6, t0, v0);
        sym3_mv(c6, t1, v1);
        float a = dot3(t0, v0) + P->lowpass;
        float b = dot3(t0, v1);
        float c = dot3(t1, v1) + P->lowpass;

        float det, con0, con1, con2;
        float op = P->fused_activation ? sigmoidf_det(opacity[i]) : opacity[i];
        if (P->enable_anti_aliasing) {
            // gs3d.py:592-617: the conic is the exact inverse of the low-passed covariance (no eps), the
            // returned determinant is the one WITHOUT the low-pass term (it feeds the radius and the
            // det > 0 test below, render.py:466-476), and the opacity is scaled by
            // sqrt(max(0.000025, det / det_lowpass)) (render.py:393, 404-407).
            const float a0 = a - P->lowpass, c0 = c - P->lowpass;
            const float det_lp = a * c - b * b;
            det = a0 * c0 - b * b;
            const float inv = 1.0f / det_lp;
            con0 = c * inv, con1 = (-b) * inv, con2 = a * inv;
            op = op * sqrtf(fmaxf(0.000025f, det / det_lp));
        } else {
            det = a * c - b * b;
            const float det_inv = 1.0f / (det + P->eps);
            con0 = c * det_inv, con1 = (-b) * det_inv, con2 = a * det_inv;
        }

        float mid = 0.5f * (a + c);
        float sq = sqrtf(fmaxf(P->radii_eigen_eps, mid * mid - det));
        float l1 = mid + sq, l2 = mid - sq;
        float radius = ceilf(P->std_sigma * sqrtf(fmaxf(l1, l2)));

        int rminx = tile_coord((u - radius) / 16.0f, P->tiles_x);
        int rminy = tile_coord((v - radius) / 16.0f, P->tiles_y);
        int rmaxx = tile_coord((((u + radius) + 16.0f) - 1.0f) / 16.0f, P->tiles_x);
        int rmaxy = tile_coord((((v + radius) + 16.0f) - 1.0f) / 16.0f, P->tiles_y);
        int area = (rmaxx - rminx) * (rmaxy - rminy);
        bool invalid = !(det > 0.0f) || area == 0 || !(op > P->alpha_eps);
        if (invalid) continue;

        TileWalkIn g{u, v, radius, {con0, con1, con2}, op};
        int cnt = tile_walk(P, g, [](int, int) {});
        radii[i] = (int)radius;
        tiles_touched[i] = cnt;
        depths[i] = P->render_inv_depth ? 1.0f / z : z;   // render.py:582
        uvs[2 * i] = u;
        uvs[2 * i + 1] = v;
        conic_opacity[4 * i + 0] = con0;
        conic_opacity[4 * i + 1] = con1;
        conic_opacity[4 * i + 2] = con2;
        conic_opacity[4 * i + 3] = op;

        float dn = sqrtf((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]);
        float dir[3] = {d[0] / dn, d[1] / dn, d[2] / dn};
        const float* shp = sh + (size_t)i * P->sh_stride * 3;
        const float* base = P->has_sh_base ? sh_base + 3 * i : shp;
        const float* rest = P->has_sh_base ? shp : shp + 3;
        float rgb[3];
        sh_to_rgb(P->sh_degree, dir, base, rest, rgb);
        uint8_t ne0 = (uint8_t)(((rgb[0] < 0.0f) << 2) | ((rgb[1] < 0.0f) << 1) | (rgb[2] < 0.0f));
        for (int k = 0; k < 3; ++k) rgb_out[3 * i + k] = fmaxf(rgb[k], 0.0f);
        if (ne0_out) ne0_out[i] = ne0;
        if (cov2d_out) {
            cov2d_out[3 * i + 0] = a;
            cov2d_out[3 * i + 1] = b;
            cov2d_out[3 * i + 2] = c;
        }
    }
    return 0;
}

// K2: inclusive scan in place, returns the total (render.py:694-695)
ORC_API int64_t orc_scan(int32_t* tiles_touched, int32_t n) {
    int64_t acc = 0;
    for (int i = 0; i < n; ++i) {
        acc += tiles_touched[i];
        tiles_touched[i] = (int32_t)acc;
    }
    return acc;
}

// K3: key expansion (render.py:745-840). offsets = inclusive scan from orc_scan.
ORC_API void orc_make_keys(const orc_params* P, const int32_t* radii, const float* uvs, const float* conic_opacity,
                   const float* depths, const int32_t* offsets, uint64_t* keys, int32_t* vals) {
    const int n = P->n;
#pragma omp parallel for schedule(dynamic, 1024)
    for (int i = 0; i < n; ++i) {
        if (radii[i] <= 0) continue;
        int64_t off = i == 0 ? 0 : offsets[i - 1];
        uint32_t dbits;
        memcpy(&dbits, depths + i, 4);
        // render.py:767-775: the float bits, or the depth in steps of depth_32bit_prec cut to 18 bits
        if (P->enable_32bit_sort) dbits = (uint32_t)(depths[i] / P->depth_32bit_prec) & 0x3FFFFu;
        const int shift = P->enable_32bit_sort ? 18 : 32;   // render.py:737
        TileWalkIn g{uvs[2 * i], uvs[2 * i + 1], (float)radii[i],
                     {conic_opacity[4 * i], conic_opacity[4 * i + 1], conic_opacity[4 * i + 2]}, conic_opacity[4 * i + 3]};
        tile_walk(P, g, [&](int x, int y) {
            uint64_t key = (uint64_t)(y * P->tiles_x + x);
            keys[off] = (key << shift) | dbits;
            vals[off] = i;
            ++off;
        });
    }
}

// devsort.py:131-149 — bit length of n
ORC_API int32_t orc_higher_msb(uint32_t n) {
    int32_t b = 0;
    while (n) { ++b; n >>= 1; }
    return b;
}

// K4: stable LSD radix sort of (u64 key, i32 value) on bits [begin_bit, end_bit)  (devsort.py:77-129)
ORC_API void orc_sort_pairs(const uint64_t* keys_in, const int32_t* vals_in, uint64_t* keys_out, int32_t* vals_out, int64_t m,
                    int32_t begin_bit, int32_t end_bit) {
    std::vector<uint64_t> ka(keys_in, keys_in + m), kb(m);
    std::vector<int32_t> va(vals_in, vals_in + m), vb(m);
    for (int bit = begin_bit; bit < end_bit; bit += 8) {
        int nb = std::min(8, end_bit - bit);
        uint64_t mask = (1ull << nb) - 1;
        std::vector<int64_t> cnt(257, 0);
        for (int64_t i = 0; i < m; ++i) cnt[((ka[i] >> bit) & mask) + 1]++;
        for (int d = 0; d < 256; ++d) cnt[d + 1] += cnt[d];
        for (int64_t i = 0; i < m; ++i) {
            int64_t dst = cnt[(ka[i] >> bit) & mask]++;
            kb[dst] = ka[i];
            vb[dst] = va[i];
        }
        ka.swap(kb);
        va.swap(vb);
    }
    std::copy(ka.begin(), ka.end(), keys_out);
    std::copy(va.begin(), va.end(), vals_out);
}

// K5: per-tile [start,end) in the sorted list (render.py:897-939). ranges must be zero-filled.
ORC_API void orc_tile_ranges(const uint64_t* keys_sorted, int64_t m, int32_t* ranges, int32_t num_tiles, int32_t shift) {
    (void)num_tiles;
    for (int64_t i = 0; i < m; ++i) {
        uint32_t t = (uint32_t)(keys_sorted[i] >> shift);
        if (i == 0) {
            ranges[2 * t] = 0;
        } else {
            uint32_t tp = (uint32_t)(keys_sorted[i - 1] >> shift);
            if (t != tp) {
                ranges[2 * tp + 1] = (int32_t)i;
                ranges[2 * t] = (int32_t)i;
            }
        }
        if (i == m - 1) ranges[2 * t + 1] = (int32_t)m;
    }
}

// power = -1/2 (a dx^2 + c dy^2) - b dx dy  (render.py:1765-1767), evaluated as two fused
// multiply-adds over the pre-scaled conic (-a/2, -b, -c/2); the scaling is exact.  The reference's
// CUDA build contracts these products into FMAs at the compiler's discretion; here the sequence is
// fixed so that CPU and GPU agree bit for bit.
static inline float blend_power(const float* co, float dx, float dy) {
    const float ha = -0.5f * co[0], nb = -co[1], hc = -0.5f * co[2];
    return fmaf(nb * dx, dy, fmaf(hc * dy, dy, (ha * dx) * dx));
}

// ---------------------------------------------------------------------------
// K6 blend forward (render.py:1541-1570, 1677-1923, 2222-2271)
// color[H,W,C] (or [C,H,W] with use_nchw), C = 3 + render_rgba; final_T[H,W], n_contrib[H,W],
// final_depth[H,W] when render_depth.
// ---------------------------------------------------------------------------
static inline size_t color_index(const orc_params* P, size_t pid, int ch) {
    const int C = 3 + (P->render_rgba ? 1 : 0);
    return P->use_nchw ? (size_t)ch * P->width * P->height + pid : pid * C + ch;
}

ORC_API void orc_blend_fwd(const orc_params* P, const int32_t* ranges, const int32_t* idx_sorted, const float* uvs,
                   const float* conic_opacity, const float* rgb_g, const float* depths, float* color, float* final_T,
                   int32_t* n_contrib, float* final_depth) {
    const int W = P->width, H = P->height;
    const int ntiles = P->tiles_x * P->tiles_y;
    const int C = 3 + (P->render_rgba ? 1 : 0);
#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < ntiles; ++t) {
        int tx = t % P->tiles_x, ty = t / P->tiles_x;
        int r0 = ranges[2 * t], r1 = ranges[2 * t + 1];
        for (int ly = 0; ly < 16; ++ly)
            for (int lx = 0; lx < 16; ++lx) {
                int px = tx * 16 + lx, py = ty * 16 + ly;
                if (px >= W || py >= H) continue;
                float pxf = (float)px, pyf = (float)py;
                float T = 1.0f;
                float acc[4] = {0, 0, 0, 0};
                float depth_accum = 0.0f;
                int contributor = 0;
                for (int k = r0; k < r1; ++k) {
                    int g = idx_sorted[k];
                    float dx = uvs[2 * g] - pxf, dy = uvs[2 * g + 1] - pyf;
                    const float* co = conic_opacity + 4 * g;
                    float power = blend_power(co, dx, dy);
                    float G = orc_expf_blend(power);
                    float alpha = fminf(0.99f, co[3] * G);
                    if (alpha < P->alpha_eps) continue;
                    float nextT = T * (1.0f - alpha);
                    bool should_done = nextT < P->transmittance_eps;
                    if (power > 0.0f || should_done) {
                        if (should_done) break;
                        continue;
                    }
                    float w = alpha * T;
                    T = nextT;
                    contributor = k - r0;
                    acc[0] = fmaf(w, rgb_g[3 * g + 0], acc[0]);
                    acc[1] = fmaf(w, rgb_g[3 * g + 1], acc[1]);
                    acc[2] = fmaf(w, rgb_g[3 * g + 2], acc[2]);
                    if (P->render_rgba) acc[3] = acc[3] + w;                               // render.py:1899-1906
                    if (P->render_depth) depth_accum = fmaf(w, depths[g], depth_accum);   // render.py:1915-1919
                }
                size_t pid = (size_t)py * W + px;
                final_T[pid] = T;
                n_contrib[pid] = contributor;
                if (P->render_depth)  // render.py:2244-2254
                    final_depth[pid] = P->training ? depth_accum : depth_accum / ((1e-10f + 1.0f) - T);
                if (P->training) {
                    for (int ch = 0; ch < C; ++ch) color[color_index(P, pid, ch)] = acc[ch];
                } else {
                    for (int ch = 0; ch < C; ++ch) {
                        float vv = acc[ch] + T * (ch < 3 ? P->bg[ch] : 0.0f);   // alpha has no background (render.py:2227-2229)
                        color[color_index(P, pid, ch)] = fminf(fmaxf(vv, 0.0f), 1.0f);
                    }
                }
            }
    }
}

// ---------------------------------------------------------------------------
// K7 blend backward (render.py:1589-1676, 1774-1792, 1868-2019).  The complete
// gradient (reference semantics with backward_reduction_balanced_factor = 0;
// the default balanced branch drops dcolor for sparse warps, render.py:2125-2148).
// Per-pixel terms in float32, accumulation over pixels in float64.
// Ten values per gaussian: duv(2), dconic(3), dopacity, dcolor(3), dz.
// ---------------------------------------------------------------------------
ORC_API void orc_blend_bwd(const orc_params* P, const int32_t* ranges, const int32_t* idx_sorted, const float* uvs,
                   const float* conic_opacity, const float* rgb_g, const float* depths, const float* final_T,
                   const int32_t* n_contrib, const float* color, const float* final_depth, const float* drgb,
                   const float* dT, const float* ddepth, double* duv, double* dconic, double* dopacity,
                   double* dcolor, double* dz /* [N], used when render_depth */,
                   double* absmass /* [N,10] sum of |terms|, may be NULL */,
                   double* statemass /* [N,6], may be NULL: how strongly duv (2), dconic (3) and dopacity depend on
                                        the rounding of a pixel's running colour state: the sum over pixels of
                                        |d term / d dl| * sum_ch |drgb_ch| * |final colour_ch|.  A backward that
                                        rebuilds "the colour still behind" from sums rounded at the magnitude of the
                                        final colour (the per-gaussian algorithm's snapshots, render.py:2601)
                                        differs from this sequence by a few ulp of that magnitude per pixel. */) {
    const int W = P->width, H = P->height;
    const int ntiles = P->tiles_x * P->tiles_y;
    const int NV = 10;
#pragma omp parallel for schedule(dynamic, 1)
    for (int t = 0; t < ntiles; ++t) {
        int tx = t % P->tiles_x, ty = t / P->tiles_x;
        int r0 = ranges[2 * t], r1 = ranges[2 * t + 1];
        int len = r1 - r0;
        if (len <= 0) continue;
        std::vector<double> acc((size_t)len * NV, 0.0);
        std::vector<double> mass((size_t)len * NV, 0.0);
        std::vector<double> smass(statemass ? (size_t)len * 6 : 0, 0.0);
        for (int ly = 0; ly < 16; ++ly)
            for (int lx = 0; lx < 16; ++lx) {
                int px = tx * 16 + lx, py = ty * 16 + ly;
                if (px >= W || py >= H) continue;
                size_t pid = (size_t)py * W + px;
                float pxf = (float)px, pyf = (float)py;
                int contributor = n_contrib[pid] + 1;
                float render_T = final_T[pid];
                float dT_val = dT[pid];
                float rr[4] = {0, 0, 0, 0}, dr[4] = {0, 0, 0, 0};
                for (int ch = 0; ch < 3 + (P->render_rgba ? 1 : 0); ++ch) {
                    rr[ch] = color[color_index(P, pid, ch)];
                    dr[ch] = drgb[color_index(P, pid, ch)];
                }
                float rdep = P->render_depth ? final_depth[pid] : 0.0f;
                float ddep = P->render_depth ? ddepth[pid] : 0.0f;
                float T = 1.0f;
                int lim = std::min(contributor, len);
                for (int j = 0; j < lim; ++j) {
                    int g = idx_sorted[r0 + j];
                    float dx = uvs[2 * g] - pxf, dy = uvs[2 * g + 1] - pyf;
                    const float* co = conic_opacity + 4 * g;
                    float power = blend_power(co, dx, dy);
                    float G = orc_expf_blend(power);
                    float alpha = fminf(0.99f, co[3] * G);
                    bool valid = power <= 0.0f && alpha >= P->alpha_eps;
                    if (!valid) continue;
                    // fixed operation sequence shared with the HIP kernel: which pixels a gaussian touches,
                    // T and the colour still behind agree bit for bit; the kernel forms dl / (1 - alpha) with
                    // the hardware reciprocal (within 2 ulp of this division), and the order of the sums differs
                    const float one_m = 1.0f - alpha;
                    float w = alpha * T;
                    T = T * one_m;
                    const float* cg = rgb_g + 3 * g;
                    rr[0] = fmaf(-w, cg[0], rr[0]);
                    rr[1] = fmaf(-w, cg[1], rr[1]);
                    rr[2] = fmaf(-w, cg[2], rr[2]);
                    float dl = (-dT_val) * render_T;
                    if (P->render_depth) {   // render.py:1887-1890, 1948-1950
                        const float dg = depths[g];
                        rdep = fmaf(-w, dg, rdep);
                        dl = fmaf(ddep, fmaf(T, dg, -rdep), dl);
                    }
                    if (P->render_rgba) {    // render.py:1871-1874, 1926-1931: the alpha channel blends the constant 1
                        rr[3] = rr[3] - w;
                        dl = fmaf(dr[3], T - rr[3], dl);
                    }
                    dl = fmaf(dr[2], fmaf(T, cg[2], -rr[2]), dl);
                    dl = fmaf(dr[1], fmaf(T, cg[1], -rr[1]), dl);
                    dl = fmaf(dr[0], fmaf(T, cg[0], -rr[0]), dl);
                    float dL_dalpha = dl / one_m;
                    // With q = dL/dG * G, the screen-space gradients are linear in five moments of q
                    // (render.py:1996-2017 per pixel):  dL/du = -(a S1 + b S2), dL/dv = -(c S2 + b S1),
                    // dL/dconic = (-S3 / 2, -S4, -S5 / 2) with S1 = sum q dx, S2 = sum q dy, S3 = sum q dx^2,
                    // S4 = sum q dx dy, S5 = sum q dy^2.  The moments are accumulated per pixel and the
                    // per-gaussian linear map is applied once per (tile, gaussian), as the kernel does.
                    const float gop = dL_dalpha * G;       // dL/dopacity term
                    const float q = co[3] * gop;
                    const float qx = q * dx, qy = q * dy;
                    double* a9 = acc.data() + (size_t)j * NV;
                    double* m9 = mass.data() + (size_t)j * NV;
                    const float term[NV] = {qx, qy, qx * dx, qx * dy, qy * dy, gop, w * dr[0], w * dr[1], w * dr[2],
                                            w * ddep /* render.py:1964-1967 */};
                    for (int k = 0; k < NV; ++k) {
                        a9[k] += (double)term[k];
                        m9[k] += fabs((double)term[k]);
                    }
                    if (statemass) {
                        double state = 0.0;
                        for (int ch = 0; ch < 3 + (P->render_rgba ? 1 : 0); ++ch)
                            state += fabs((double)dr[ch]) * fabs((double)color[color_index(P, pid, ch)]);
                        if (P->render_depth) state += fabs((double)ddep) * fabs((double)final_depth[pid]);
                        const double per_dl = fabs((double)G / (double)one_m) * state;     // d gop / d dl, times state
                        const double geom[6] = {fabs((double)co[3] * dx), fabs((double)co[3] * dy),
                                                fabs((double)co[3] * dx * dx), fabs((double)co[3] * dx * dy),
                                                fabs((double)co[3] * dy * dy), 1.0};
                        double* s6 = smass.data() + (size_t)j * 6;
                        for (int k = 0; k < 6; ++k) s6[k] += per_dl * geom[k];
                    }
                }
            }
        // moments -> (duv, dconic) per (tile, gaussian); the magnitudes follow the same map with absolute values
        for (int j = 0; j < len; ++j) {
            const float* co = conic_opacity + 4 * idx_sorted[r0 + j];
            const double a = co[0], b = co[1], c = co[2];
            double* S = acc.data() + (size_t)j * NV;
            double* Ms = mass.data() + (size_t)j * NV;
            const double S1 = S[0], S2 = S[1], M1 = Ms[0], M2 = Ms[1];
            S[0] = -(a * S1 + b * S2);
            S[1] = -(c * S2 + b * S1);
            S[2] = -0.5 * S[2];
            S[3] = -S[3];
            S[4] = -0.5 * S[4];
            Ms[0] = fabs(a) * M1 + fabs(b) * M2;
            Ms[1] = fabs(c) * M2 + fabs(b) * M1;
            Ms[2] = 0.5 * Ms[2];
            Ms[4] = 0.5 * Ms[4];
            if (statemass) {
                double* Q = smass.data() + (size_t)j * 6;
                const double Q1 = Q[0], Q2 = Q[1];
                Q[0] = fabs(a) * Q1 + fabs(b) * Q2;
                Q[1] = fabs(c) * Q2 + fabs(b) * Q1;
                Q[2] = 0.5 * Q[2];
                Q[4] = 0.5 * Q[4];
            }
        }
        for (int j = 0; j < len; ++j) {
            int g = idx_sorted[r0 + j];
            const double* a9 = acc.data() + (size_t)j * NV;
            bool any = false;
            for (int k = 0; k < NV; ++k) any = any || a9[k] != 0.0;
            if (!any) continue;
            double* dst[NV] = {duv + 2 * g, duv + 2 * g + 1, dconic + 3 * g, dconic + 3 * g + 1, dconic + 3 * g + 2,
                               dopacity + g, dcolor + 3 * g, dcolor + 3 * g + 1, dcolor + 3 * g + 2,
                               P->render_depth ? dz + g : nullptr};
            for (int k = 0; k < NV; ++k) {
                if (!dst[k]) continue;
#pragma omp atomic
                *dst[k] += a9[k];
                if (absmass) {
#pragma omp atomic
                    absmass[NV * (size_t)g + k] += mass[(size_t)j * NV + k];
                }
                if (statemass && k < 6) {
#pragma omp atomic
                    statemass[6 * (size_t)g + k] += smass[(size_t)j * 6 + k];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// K9 preprocess backward (render.py:3217-3356; gs3d.py:237-366, 387-418,
// 472-532, 559-588; camera.py:335-371; origin/model.py:332-383).
// sh_mask_compat != 0 reproduces the reference's reversed clamp-mask bit order
// (render.py:608 vs 3344-3350); 0 uses the consistent mapping.
// Gradients of gaussians with radii == 0 are zero.
// ---------------------------------------------------------------------------
ORC_API void orc_preprocess_bwd(const orc_params* P0, const float* xyz, const float* quat, const float* scale,
                        const float* opacity, const float* sh, const int32_t* radii, const float* cov2d,
                        const uint8_t* ne0, const float* duv, const float* dconic, const float* dopacity_in,
                        const float* dcolor, const float* dz, int32_t sh_mask_compat, float* dxyz, float* dquat,
                        float* dscale, float* dopacity_out, float* dsh, float* dsh_base, const int32_t* instance_ids,
                        const float* instance_cameras, int32_t num_instances) {
    const int n = P0->n;
    const int K = P0->sh_stride;
#pragma omp parallel for schedule(dynamic, 1024)
    for (int i = 0; i < n; ++i) {
        const orc_params Pl = with_instance(P0, instance_ids, instance_cameras, num_instances, i);
        const orc_params* P = &Pl;
        for (int k = 0; k < 3; ++k) dxyz[3 * i + k] = 0.0f;
        for (int k = 0; k < 4; ++k) dquat[4 * i + k] = 0.0f;
        for (int k = 0; k < 3; ++k) dscale[3 * i + k] = 0.0f;
        dopacity_out[i] = 0.0f;
        for (int k = 0; k < K * 3; ++k) dsh[(size_t)i * K * 3 + k] = 0.0f;
        if (dsh_base)
            for (int k = 0; k < 3; ++k) dsh_base[3 * i + k] = 0.0f;
        if (radii[i] == 0) continue;

        const float* W = P->w2c;
        float d[3] = {xyz[3 * i] - P->cam_center[0], xyz[3 * i + 1] - P->cam_center[1], xyz[3 * i + 2] - P->cam_center[2]};
        float pc[3] = {dot3(W + 0, d), dot3(W + 3, d), dot3(W + 6, d)};
        float z = pc[2];
        // pinhole backward (camera.py:357-369)
        float gu = duv[2 * i] * P->fx, gv = duv[2 * i + 1] * P->fy;
        float zi = 1.0f / z, zi2 = 1.0f / (z * z);
        float dzin = dz ? dz[i] : 0.0f;
        if (P->render_inv_depth) dzin = (-dzin) / (pc[2] * pc[2]);   // dz is dL/d(1/z) then (render.py:1965, 3051, 3283)
        float dpc[3] = {gu * zi, gv * zi, (dzin + ((-gu) * pc[0]) * zi2) + ((-gv) * pc[1]) * zi2};

        // conic -> cov2d backward (gs3d.py:571-586)
        float a = cov2d[3 * i], b = cov2d[3 * i + 1], c = cov2d[3 * i + 2];
        float g0 = dconic[3 * i], g1 = dconic[3 * i + 1], g2 = dconic[3 * i + 2];
        float det = a * c - b * b;
        float k2 = 1.0f / (det * det + 1e-8f);
        float da = k2 * ((((-c) * c) * g0 + (b * c) * g1) + (det - a * c) * g2);
        float db = (k2 * 2.0f) * (((b * c) * g0 - (det / 2.0f + b * b) * g1) + (a * b) * g2);
        float dc = k2 * ((((-a) * a) * g2 + (a * b) * g1) + (det - a * c) * g0);
        float dop_in = dopacity_in[i];
        if (P->enable_anti_aliasing) {
            // render.py:3293-3306; gs3d.py:671-679.  dop_in is the gradient of opacity * comp with
            // comp = sqrt(max(0.000025, ratio)), ratio = det_without_lowpass / det.
            const float lf = P->lowpass;
            const float a0 = a - lf, c0 = c - lf;
            const float ratio = (a0 * c0 - b * b) / det;
            const float comp = sqrtf(fmaxf(0.000025f, ratio));
            const float op_act = P->fused_activation ? sigmoidf_det(opacity[i]) : opacity[i];
            const float dcomp = dop_in * op_act;
            const float dratio = ratio <= 0.000025f ? 0.0f : (dcomp * 0.5f) / comp;
            const float gm = dratio * k2;
            da += (lf * ((c * c + b * b) - c * lf)) * gm;
            db += ((-2.0f * b) * lf) * ((a + c) - lf) * gm;
            dc += (lf * ((a * a + b * b) - a * lf)) * gm;
            dop_in = dop_in * comp;
        }

        // recompute activations and cov3d
        const float* qr = quat + 4 * i;
        float qn = 1.0f;
        float q[4] = {qr[0], qr[1], qr[2], qr[3]};
        float s[3] = {scale[3 * i], scale[3 * i + 1], scale[3 * i + 2]};
        if (P->fused_activation) {
            qn = sqrtf(((qr[0] * qr[0] + qr[1] * qr[1]) + qr[2] * qr[2]) + qr[3] * qr[3]);
            for (int k = 0; k < 4; ++k) q[k] = qr[k] / qn;
            for (int k = 0; k < 3; ++k) s[k] = orc_expf(s[k]);
        }
        float R[9], c6[6];
        quat_to_rot(q, R);
        cov3d_from_scale_rot(s, R, c6);

        // EWA backward (gs3d.py:490-530): cov2d = T S T^T, T = J W
        float t0[3], t1[3], tx, ty;
        ewa_rows(P, pc, t0, t1, &tx, &ty);
        float limx = fabsf((P->tan_fovx * P->clamp_factor) * z), limy = fabsf((P->tan_fovy * P->clamp_factor) * z);
        float mx = (pc[0] < -limx || pc[0] > limx) ? 0.0f : 1.0f;
        float my = (pc[1] < -limy || pc[1] > limy) ? 0.0f : 1.0f;
        float G00 = da, G01 = 0.5f * db, G11 = dc;
        // dSigma3 = T^T G T (symmetric 3x3)
        float u0[3], u1[3];  // rows of G T
        for (int k = 0; k < 3; ++k) {
            u0[k] = G00 * t0[k] + G01 * t1[k];
            u1[k] = G01 * t0[k] + G11 * t1[k];
        }
        float dS[9];
        for (int r = 0; r < 3; ++r)
            for (int k = 0; k < 3; ++k) dS[r * 3 + k] = t0[r] * u0[k] + t1[r] * u1[k];
        // dT = 2 G T Sigma3
        float dT0[3], dT1[3];
        sym3_mv(c6, u0, dT0);
        sym3_mv(c6, u1, dT1);
        for (int k = 0; k < 3; ++k) { dT0[k] = 2.0f * dT0[k]; dT1[k] = 2.0f * dT1[k]; }
        // dJ = dT W^T
        float dJ00 = dot3(dT0, W + 0), dJ02 = dot3(dT0, W + 6);
        float dJ11 = dot3(dT1, W + 3), dJ12 = dot3(dT1, W + 6);
        float zz = z * z;
        float zzi = 1.0f / zz;
        float z3 = (z * z) * z;
        float txf = tx * P->fx, tyf = ty * P->fy;
        float dmean[3];
        dmean[0] = ((mx * (-dJ02)) * P->fx) * zzi;
        dmean[1] = ((my * (-dJ12)) * P->fy) * zzi;
        dmean[2] = (-(P->fx * dJ00 + P->fy * dJ11)) * zzi + (2.0f * (dJ02 * txf + dJ12 * tyf)) / z3;
        float tot[3] = {dpc[0] + dmean[0], dpc[1] + dmean[1], dpc[2] + dmean[2]};
        float gx[3];
        for (int k = 0; k < 3; ++k) gx[k] = (W[0 + k] * tot[0] + W[3 + k] * tot[1]) + W[6 + k] * tot[2];

        // cov3d backward (gs3d.py:400-416): Sigma3 = M M^T, M = R diag(s); dM = 2 dS M
        float M[9];
        for (int r = 0; r < 3; ++r)
            for (int k = 0; k < 3; ++k) M[r * 3 + k] = R[r * 3 + k] * s[k];
        float dM[9];
        for (int r = 0; r < 3; ++r)
            for (int k = 0; k < 3; ++k)
                dM[r * 3 + k] = 2.0f * ((dS[r * 3 + 0] * M[0 + k] + dS[r * 3 + 1] * M[3 + k]) + dS[r * 3 + 2] * M[6 + k]);
        float ds[3], dR[9];
        for (int k = 0; k < 3; ++k) ds[k] = (dM[0 + k] * R[0 + k] + dM[3 + k] * R[3 + k]) + dM[6 + k] * R[6 + k];
        for (int r = 0; r < 3; ++r)
            for (int k = 0; k < 3; ++k) dR[r * 3 + k] = dM[r * 3 + k] * s[k];
        float qx = q[0], qy = q[1], qz = q[2], qw = q[3];
        float dq[4];
        dq[0] = 2.0f * (((qy * (dR[1] + dR[3]) + qz * (dR[2] + dR[6])) - (2.0f * qx) * (dR[4] + dR[8])) + qw * (dR[7] - dR[5]));
        dq[1] = 2.0f * (((qx * (dR[1] + dR[3]) - (2.0f * qy) * (dR[0] + dR[8])) + qz * (dR[5] + dR[7])) + qw * (dR[2] - dR[6]));
        dq[2] = 2.0f * (((qx * (dR[2] + dR[6]) + qy * (dR[5] + dR[7])) - (2.0f * qz) * (dR[0] + dR[4])) + qw * (dR[3] - dR[1]));
        dq[3] = 2.0f * ((qz * (dR[3] - dR[1]) + qy * (dR[2] - dR[6])) + qx * (dR[7] - dR[5]));
        // activation backward: exp, normalize, sigmoid (origin/model.py:332-383)
        if (P->fused_activation) {
            for (int k = 0; k < 3; ++k) dscale[3 * i + k] = ds[k] * s[k];
            float qd = ((q[0] * dq[0] + q[1] * dq[1]) + q[2] * dq[2]) + q[3] * dq[3];
            for (int k = 0; k < 4; ++k) dquat[4 * i + k] = (dq[k] - q[k] * qd) / qn;
            float o = sigmoidf_det(opacity[i]);
            dopacity_out[i] = dop_in * (o * (1.0f - o));
        } else {
            for (int k = 0; k < 3; ++k) dscale[3 * i + k] = ds[k];
            for (int k = 0; k < 4; ++k) dquat[4 * i + k] = dq[k];
            dopacity_out[i] = dop_in;
        }

        // SH backward (gs3d.py:262-364)
        float dn = sqrtf((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]);
        float dir[3] = {d[0] / dn, d[1] / dn, d[2] / dn};
        uint8_t m = ne0[i];
        float cg[3];
        if (sh_mask_compat) {
            cg[0] = dcolor[3 * i + 0] * ((m & 1) ? 0.0f : 1.0f);
            cg[1] = dcolor[3 * i + 1] * ((m & 2) ? 0.0f : 1.0f);
            cg[2] = dcolor[3 * i + 2] * ((m & 4) ? 0.0f : 1.0f);
        } else {
            cg[0] = dcolor[3 * i + 0] * ((m & 4) ? 0.0f : 1.0f);
            cg[1] = dcolor[3 * i + 1] * ((m & 2) ? 0.0f : 1.0f);
            cg[2] = dcolor[3 * i + 2] * ((m & 1) ? 0.0f : 1.0f);
        }
        const float* shp = sh + (size_t)i * K * 3;
        float* dshp = dsh + (size_t)i * K * 3;
        const float* rest = P->has_sh_base ? shp : shp + 3;
        float* drest = P->has_sh_base ? dshp : dshp + 3;
        float* dbase = P->has_sh_base ? dsh_base + 3 * i : dshp;
        float x = dir[0], y = dir[1], zd = dir[2];
        float ddir[3] = {0, 0, 0};
        for (int ch = 0; ch < 3; ++ch) {
            float gch = cg[ch];
            dbase[ch] = SH_C0 * gch;
            float dx_ = 0, dy_ = 0, dz_ = 0;
            if (P->sh_degree > 0) {
                drest[0 * 3 + ch] = (-SH_C1 * y) * gch;
                drest[1 * 3 + ch] = (SH_C1 * zd) * gch;
                drest[2 * 3 + ch] = (-SH_C1 * x) * gch;
                dx_ = -SH_C1 * rest[2 * 3 + ch];
                dy_ = -SH_C1 * rest[0 * 3 + ch];
                dz_ = SH_C1 * rest[1 * 3 + ch];
                if (P->sh_degree > 1) {
                    float xx = x * x, yy = y * y, zz2 = zd * zd, xy = x * y, yz = y * zd, xz = x * zd;
                    drest[3 * 3 + ch] = (SH_C2[0] * xy) * gch;
                    drest[4 * 3 + ch] = (SH_C2[1] * yz) * gch;
                    drest[5 * 3 + ch] = (SH_C2[2] * ((2.0f * zz2 - xx) - yy)) * gch;
                    drest[6 * 3 + ch] = (SH_C2[3] * xz) * gch;
                    drest[7 * 3 + ch] = (SH_C2[4] * (xx - yy)) * gch;
                    float s3 = rest[3 * 3 + ch], s4 = rest[4 * 3 + ch], s5 = rest[5 * 3 + ch], s6 = rest[6 * 3 + ch], s7 = rest[7 * 3 + ch];
                    dx_ += SH_C2[0] * y * s3 + SH_C2[2] * 2.0f * (-x) * s5 + SH_C2[3] * zd * s6 + SH_C2[4] * 2.0f * x * s7;
                    dy_ += SH_C2[0] * x * s3 + SH_C2[1] * zd * s4 + SH_C2[2] * 2.0f * (-y) * s5 + SH_C2[4] * 2.0f * (-y) * s7;
                    dz_ += SH_C2[1] * y * s4 + SH_C2[2] * 2.0f * 2.0f * zd * s5 + SH_C2[3] * x * s6;
                    if (P->sh_degree > 2) {
                        drest[8 * 3 + ch] = ((SH_C3[0] * y) * (3.0f * xx - yy)) * gch;
                        drest[9 * 3 + ch] = ((SH_C3[1] * xy) * zd) * gch;
                        drest[10 * 3 + ch] = ((SH_C3[2] * y) * ((4.0f * zz2 - xx) - yy)) * gch;
                        drest[11 * 3 + ch] = ((SH_C3[3] * zd) * ((2.0f * zz2 - 3.0f * xx) - 3.0f * yy)) * gch;
                        drest[12 * 3 + ch] = ((SH_C3[4] * x) * ((4.0f * zz2 - xx) - yy)) * gch;
                        drest[13 * 3 + ch] = ((SH_C3[5] * zd) * (xx - yy)) * gch;
                        drest[14 * 3 + ch] = ((SH_C3[6] * x) * (xx - 3.0f * yy)) * gch;
                        float s8 = rest[8 * 3 + ch], s9 = rest[9 * 3 + ch], s10 = rest[10 * 3 + ch], s11 = rest[11 * 3 + ch],
                              s12 = rest[12 * 3 + ch], s13 = rest[13 * 3 + ch], s14 = rest[14 * 3 + ch];
                        dx_ += SH_C3[0] * s8 * 3.0f * 2.0f * xy + SH_C3[1] * s9 * yz + SH_C3[2] * s10 * (-2.0f) * xy +
                               SH_C3[3] * s11 * (-3.0f) * 2.0f * xz + SH_C3[4] * s12 * ((-3.0f) * xx + 4.0f * zz2 - yy) +
                               SH_C3[5] * s13 * 2.0f * xz + SH_C3[6] * s14 * 3.0f * (xx - yy);
                        dy_ += SH_C3[0] * s8 * 3.0f * (xx - yy) + SH_C3[1] * s9 * xz + SH_C3[2] * s10 * ((-3.0f) * yy + 4.0f * zz2 - xx) +
                               SH_C3[3] * s11 * (-3.0f) * 2.0f * yz + SH_C3[4] * s12 * (-2.0f) * xy + SH_C3[5] * s13 * (-2.0f) * yz +
                               SH_C3[6] * s14 * (-3.0f) * 2.0f * xy;
                        dz_ += SH_C3[1] * s9 * xy + SH_C3[2] * s10 * 4.0f * 2.0f * yz + SH_C3[3] * s11 * 3.0f * ((2.0f * zz2 - xx) - yy) +
                               SH_C3[4] * s12 * 4.0f * 2.0f * xz + SH_C3[5] * s13 * (xx - yy);
                    }
                }
            }
            ddir[0] += dx_ * gch;
            ddir[1] += dy_ * gch;
            ddir[2] += dz_ * gch;
        }
        // normalize backward: d(point) += (ddir - dir (dir . ddir)) / |point|
        float dd = (dir[0] * ddir[0] + dir[1] * ddir[1]) + dir[2] * ddir[2];
        for (int k = 0; k < 3; ++k) dxyz[3 * i + k] = gx[k] + (ddir[k] - dir[k] * dd) / dn;
    }
}

ORC_API int32_t orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

ORC_API void orc_set_num_threads(int32_t n) {
#ifdef _OPENMP
    omp_set_num_threads(n);
#else
    (void)n;
#endif
}

