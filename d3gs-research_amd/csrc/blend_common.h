// What the blend kernels share: the staged gaussian record and its cull, the per-patch visit masks, lane-mask
// selects, the transposing wave reduction of the backward passes, tile placement.
#pragma once
#include "device_math.h"

namespace d3gs {

constexpr int kBucket = D3GS_BUCKET_SIZE;   // list entries per bucket of the per-gaussian backward: one per lane of a wavefront

// One staged gaussian: everything a visit reads sits in one 48-byte LDS record, so a visit forms one LDS
// address (the reads differ in their immediate offsets only).  The ten values every visit needs come first: two
// 16-byte reads and an 8-byte one; the LDS pipe serves the CU's four SIMDs, and a visit that reads 40 bytes
// instead of 48 is measurably shorter.
struct __attribute__((aligned(16))) StagedGaussian {
    float x, y, thr, o;         // pixel-space centre, cull threshold, opacity
    float ha, nb, hc, r;        // pre-scaled conic (-a/2, -b, -c/2); colour
    float g, b, depth, pad;     // colour; camera-space depth (depth channel only)
};

// Staged gaussian j of a wave-uniform index: the record's byte offset is formed once, in a vector register that
// every read of the visit then shares (written out because the compiler re-forms a scalar-to-vector move for
// each read instead of keeping it).
__device__ __forceinline__ const StagedGaussian& staged_at(const StagedGaussian* base, int j) {
    uint32_t off;
    asm("v_mov_b32 %0, %1" : "=v"(off) : "s"(j * (int)sizeof(StagedGaussian)));
    return *reinterpret_cast<const StagedGaussian*>(reinterpret_cast<const char*>(base) + off);
}

// Timing-only builds (csrc/Makefile, target timing-variants; never what the tests or the operator load): they
// price two parts of a visit by leaving them out, at the cost of wrong results.
//   D3GS_TIMING_ONLY_HW_EXP        exp as v_mul + v_exp_f32 (the hardware's rounding, which no CPU reproduces)
//   D3GS_TIMING_ONLY_NO_REDUCTION  the backward's ten per-lane terms are formed and kept alive, the wave reduction
//                                  is left out (the LDS atomic adds one lane's value)
//   D3GS_TIMING_ONLY_NO_VISITS     backward only (it walks as far as the forward's n_contrib says, so the forward
//                                  stays exact): no gaussian is visited; what is left is the prologue, the staging
//                                  rounds with their barriers and the flush
//   D3GS_TIMING_ONLY_LDS_PAD=bytes backward only, results unchanged: extra LDS per workgroup, so that fewer
//                                  workgroups share a compute unit (7 fit as built; 8192 more leave 5, 16384 leave 4)
//   D3GS_TIMING_ONLY_NO_FLUSH      backward only: a round ends behind its visits (no moments -> gradients step, no
//                                  flush of the tile's sums to the records)
//   D3GS_TIMING_ONLY_POWER_ONLY    backward only: every visit ends behind its first test (mask walk, record read,
//                                  power, compares)
__device__ __forceinline__ float blend_expf(float power) {
#ifdef D3GS_TIMING_ONLY_HW_EXP
    return __builtin_amdgcn_exp2f(power * 1.44269504088896341f);
#else
    return det_expf_inrange(power);
#endif
}

// power = -1/2 (a dx^2 + c dy^2) - b dx dy (render.py:1765-1767) as a fixed sequence of three
// multiplies and two fused multiply-adds; a CPU evaluating the same sequence gets the same bits.
__device__ __forceinline__ float blend_power(const StagedGaussian& g, float dx, float dy) {
    return __builtin_fmaf(g.nb * dx, dy, __builtin_fmaf(g.hc * dy, dy, (g.ha * dx) * dx));
}

// Tile index for a workgroup.  Tile list lengths are heavily skewed (dense screen regions hold
// lists 20x the median), so the launch order matters more than L2 locality: with `tile_order`
// (tiles by descending list length) the long tiles start first and, because consecutive
// workgroup ids are dealt round-robin to the 8 XCDs, spread evenly over the chip.
__device__ __forceinline__ int tile_for_block(int bid, const int32_t* __restrict__ tile_order) {
    return tile_order ? tile_order[bid] : bid;
}

// ---------------------------------------------------------------------------
// Sum of ten per-lane values over the wavefront, as a transposing reduction:
// every step exchanges halves so that the number of live registers halves with
// the group size (10 -> 5 -> 3 -> 2 -> 1), ~25 VALU operations instead of ten
// independent 64-lane butterflies.  Cross-half / cross-row exchanges use the
// gfx950 v_permlane32_swap / v_permlane16_swap, the rest DPP.  On return ten
// lanes hold one total each; reduce_slot() tells each lane which value (or none)
// it holds.  The tenth value (the depth gradient) shares the exchange of the
// ninth, so it costs nothing when it is the constant zero.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float swap_add32(float a, float b) {
    // lanes 0..31 <- a[l] + a[l+32]; lanes 32..63 <- b[l-32] + b[l]
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float swap_add16(float a, float b) {
    // rows 0,2 <- a[row] + a[row+1]; rows 1,3 <- b[row-1] + b[row]   (row = 16 lanes)
    auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
template <int kCtrl>
__device__ __forceinline__ float dpp_f(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, 0xF, 0xF, false));
}

__device__ __forceinline__ int reduce_slot(int lane) {
    if (lane & 3) return -1;
    const int r = lane >> 4, h = (lane >> 3) & 1, k = (lane >> 2) & 1;
    if (r == 0) return h + 2 * k;
    if (r == 2) return 4 + h + 2 * k;
    if (r == 1 && k == 0) return 8 + h;
    return -1;
}

// kTen = false: there is no tenth value.  Its slot's lanes (bit 3 of the lane set, in the register that carries
// v8) only ever combine with each other and end in a lane whose slot nobody reads, so they need no defined
// content: the register starts unset (no move to form a zero) and the instruction that would add the tenth
// value's halves is left out.
template <bool kTen>
__device__ __forceinline__ float wave_reduce10(float v0, float v1, float v2, float v3, float v4, float v5, float v6,
                                               float v7, float v8, float v9) {
    if constexpr (!kTen) asm volatile("" : "=v"(v9));
    // 16 -> 8 and 8 -> 4 inside each row of 16 lanes, while the most registers are live, with DPP adds whose
    // bank mask writes only one half of the lanes: "b += b[partner]" on the lanes that keep b, then
    // "b = a + a[partner]" on the lanes that keep a, merges a pair of registers in two instructions and no
    // select.  row_ror:8 pairs lane i with i ^ 8 (banks 0,1 | 2,3), row_half_mirror pairs i with 7 - i inside
    // each 8 lanes (banks 0,2 | 1,3).  The block opens and closes with two wait states: a DPP read needs
    // them after a vector write of its source, and so does what follows; the compiler cannot see inside.
    if constexpr (kTen) {
        asm("s_nop 1\n\t"
            "v_add_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %2, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %3, %3, %3 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %4, %4, %4 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %0, %5, %5 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %1, %6, %6 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %2, %7, %7 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %3, %8, %8 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %4, %9, %9 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        // now %0..%4 hold (v0|v1), (v2|v3), (v4|v5), (v6|v7), (v8|v9) in lanes (bit 3 clear | set)
            "v_add_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %3, %3, %3 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %4, %4, %4 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %1, %0, %0 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %3, %2, %2 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "s_nop 1"
            : "+v"(v1), "+v"(v3), "+v"(v5), "+v"(v7), "+v"(v9)
            : "v"(v0), "v"(v2), "v"(v4), "v"(v6), "v"(v8));
    } else {
        asm("s_nop 1\n\t"
            "v_add_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %2, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %3, %3, %3 row_ror:8 row_mask:0xf bank_mask:0xc\n\t"
            "v_add_f32_dpp %0, %5, %5 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %1, %6, %6 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %2, %7, %7 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %3, %8, %8 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
            "v_add_f32_dpp %4, %9, %9 row_ror:8 row_mask:0xf bank_mask:0x3\n\t"
        // now %0..%4 hold (v0|v1), (v2|v3), (v4|v5), (v6|v7), (v8|v9) in lanes (bit 3 clear | set)
            "v_add_f32_dpp %1, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %3, %3, %3 row_half_mirror row_mask:0xf bank_mask:0xa\n\t"
            "v_add_f32_dpp %4, %4, %4 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
            "v_add_f32_dpp %1, %0, %0 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "v_add_f32_dpp %3, %2, %2 row_half_mirror row_mask:0xf bank_mask:0x5\n\t"
            "s_nop 1"
            : "+v"(v1), "+v"(v3), "+v"(v5), "+v"(v7), "+v"(v9)
            : "v"(v0), "v"(v2), "v"(v4), "v"(v6), "v"(v8));
    }
    // v3: v0 v1 | v2 v3 by (bit 3, bit 2) of the lane; v7: v4 .. v7 likewise; v9: v8 | v9 by bit 3
    // 64 -> 32: rows 0,1 keep the first register, rows 2,3 the second
    // (v9's partner only feeds rows 2 and 3 of e1, which end in row 3 of the result, where no slot lives: any
    // register does, and an unset one costs no move)
    float unset;
    asm volatile("" : "=v"(unset));
    const float e0 = swap_add32(v3, v7), e1 = swap_add32(v9, unset);
    // 32 -> 16: rows 0,2 keep e0, rows 1,3 keep e1
    float y = swap_add16(e0, e1);
    // 4 -> 1 inside each quad: two DPP adds (written out: the compiler forms a zero "old" operand for the second
    // one and splits it into a move, a DPP move and an add); a DPP read needs two wait states after the vector
    // write of its source
    float total;
    asm("s_nop 1\n\t"
        "v_add_f32_dpp %0, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_add_f32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf"
        : "=&v"(total)
        : "v"(y));
    return total;
}

__device__ __forceinline__ int wave_max_i32(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, 64));
    return v;
}

// Stages one gaussian and returns a 4-bit mask: bit q set when the gaussian may reach a pixel of
// the tile's 8x8 patch q (q & 1 = right half, q >> 1 = lower half).  Conservative by construction.
// kColour = false: no colour is read (rgb_g may be NULL); r, g, b are staged as zeros.
template <bool kColour = true>
__device__ __forceinline__ uint32_t stage_gaussian(const d3gs_params& P, int g, const float* __restrict__ uvs,
                                                   const float* __restrict__ conic_opacity,
                                                   const float* __restrict__ rgb_g, const float* __restrict__ depths,
                                                   float tile_x0, float tile_y0, StagedGaussian* dst) {
    const float2 xy = *reinterpret_cast<const float2*>(uvs + 2 * g);
    const float4 co = *reinterpret_cast<const float4*>(conic_opacity + 4 * g);
    StagedGaussian s;
    s.x = xy.x;
    s.y = xy.y;
    s.thr = __logf(P.alpha_eps / co.w) - 1.0e-3f;
    s.o = co.w;
    s.ha = -0.5f * co.x;  // exact scalings: power = (ha dx) dx + (hc dy) dy + (nb dx) dy
    s.nb = -co.y;
    s.hc = -0.5f * co.z;
    s.depth = depths ? depths[g] : 0.0f;
    if constexpr (kColour) {
        s.r = rgb_g[3 * g];
        s.g = rgb_g[3 * g + 1];
        s.b = rgb_g[3 * g + 2];
    } else {
        s.r = s.g = s.b = 0.0f;
    }
    s.pad = 0.0f;
    *dst = s;
    // Level set {power >= thr}: a dx^2 + 2 b dx dy + c dy^2 <= R with R = -2 thr.  A pixel of this tile
    // evaluates `power` with an absolute rounding error below err; widening R by 2 err keeps every pixel
    // whose computed power can reach thr inside the box.
    const float X = fabsf(xy.x - (tile_x0 + 7.5f)) + 8.0f, Y = fabsf(xy.y - (tile_y0 + 7.5f)) + 8.0f;
    const float err = 1.0e-6f * (co.x * X * X + co.z * Y * Y + 2.0f * fabsf(co.y) * X * Y);
    const float R = -2.0f * s.thr + 2.0f * err + 1.0e-3f;
    const float D = co.x * co.z - co.y * co.y;
    // ill-conditioned conic, or one that is not positive definite (a caller of the C ABI may hand over any conic;
    // the box and the per-patch minimum below assume an ellipse): no cull, every patch visits it and the exact
    // per-pixel sequence decides
    if (!(co.x > 0.0f) || !(co.z > 0.0f) || !(D > 1.0e-4f * co.x * co.z) || !(R > 0.0f)) return 0xFu;
    const float hx = 1.01f * __fsqrt_rn(R * co.z / D) + 0.01f;
    const float hy = 1.01f * __fsqrt_rn(R * co.x / D) + 0.01f;
    const bool left = xy.x - hx <= tile_x0 + 7.0f, right = xy.x + hx >= tile_x0 + 8.0f;
    const bool top = xy.y - hy <= tile_y0 + 7.0f, bottom = xy.y + hy >= tile_y0 + 8.0f;
    const bool in_x = xy.x + hx >= tile_x0 && xy.x - hx <= tile_x0 + 15.0f;
    const bool in_y = xy.y + hy >= tile_y0 && xy.y - hy <= tile_y0 + 15.0f;
    if (!(in_x && in_y)) return 0u;
    const uint32_t box = (uint32_t)(left && top) | ((uint32_t)(right && top) << 1) | ((uint32_t)(left && bottom) << 2) |
                         ((uint32_t)(right && bottom) << 3);
    // The ellipse itself against each patch: the minimum of Q = a dx^2 + 2 b dx dy + c dy^2 over the patch's
    // pixel-centre rectangle.  Q is convex with its minimum at the centre, so over a rectangle it is attained
    // on the vertical line nearest to the centre in x or on the horizontal line nearest in y, each time at the
    // clamped one-dimensional minimiser; both candidates are points of the rectangle, so the smaller of the two
    // is the minimum.  A misplaced minimiser raises Q only in second order; the evaluation error of Q is
    // covered by widening R once more by 2 err.  A patch is dropped only on "minimum > R" (a NaN keeps it).
    const float R2 = R + 2.0f * err;
    const float slope_y = -co.y / co.z, slope_x = -co.y / co.x;  // dy* = slope_y dx on a vertical line, dx* = slope_x dy
    const float lx = tile_x0 - xy.x, ly = tile_y0 - xy.y;
    auto reaches = [&](float x_lo, float y_lo) {
        const float x_hi = x_lo + 7.0f, y_hi = y_lo + 7.0f;
        const float dxn = __builtin_amdgcn_fmed3f(0.0f, x_lo, x_hi), dyn = __builtin_amdgcn_fmed3f(0.0f, y_lo, y_hi);
        const float dys = __builtin_amdgcn_fmed3f(slope_y * dxn, y_lo, y_hi);
        const float dxs = __builtin_amdgcn_fmed3f(slope_x * dyn, x_lo, x_hi);
        const float q1 = co.x * dxn * dxn + 2.0f * co.y * dxn * dys + co.z * dys * dys;
        const float q2 = co.x * dxs * dxs + 2.0f * co.y * dxs * dyn + co.z * dyn * dyn;
        return !(q1 > R2) || !(q2 > R2);
    };
    return box & ((uint32_t)reaches(lx, ly) | ((uint32_t)reaches(lx + 8.0f, ly) << 1) |
                  ((uint32_t)reaches(lx, ly + 8.0f) << 2) | ((uint32_t)reaches(lx + 8.0f, ly + 8.0f) << 3));
}

// Publishes the four per-patch ballots of this staging wavefront's 64 gaussians.
__device__ __forceinline__ void publish_masks(uint32_t bits, int wave, int lane, unsigned long long (*s_mask)[4]) {
    const unsigned long long m0 = __ballot(bits & 1u), m1 = __ballot(bits & 2u), m2 = __ballot(bits & 4u),
                             m3 = __ballot(bits & 8u);
    if (lane == 0) {
        s_mask[0][wave] = m0;
        s_mask[1][wave] = m1;
        s_mask[2][wave] = m2;
        s_mask[3][wave] = m3;
    }
}

__device__ __forceinline__ unsigned long long uniform_u64(unsigned long long v) {
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return ((unsigned long long)hi << 32) | lo;
}

// Predicate codes of __builtin_amdgcn_fcmpf / __builtin_amdgcn_sicmp (LLVM's CmpInst::Predicate).
constexpr int kFcmpOgt = 2, kFcmpOge = 3, kFcmpOlt = 4, kFcmpOle = 5, kIcmpSlt = 40;

// a = mask ? a0 : 0 and b = mask ? b0 : 0 for a lane mask held in a scalar register pair.  The compiler has no
// cheap way from a 64-bit integer back to a per-lane predicate, hence the instruction is written out; the
// two wait states in front cover a vector instruction that has just written the mask registers.
__device__ __forceinline__ void select2_or_zero(unsigned long long mask, float a0, float b0, float& a, float& b) {
    asm("s_nop 1\n\t"
        "v_cndmask_b32_e64 %0, 0, %2, %4\n\t"
        "v_cndmask_b32_e64 %1, 0, %3, %4"
        : "=&v"(a), "=&v"(b)
        : "v"(a0), "v"(b0), "s"(mask));
}

// r = mask ? if_set : if_clear, and r = mask ? if_set : 0, for a lane mask held in a scalar register pair (the same
// reason as above: conditions that are combined as 64-bit masks with scalar instructions come back as selects)
__device__ __forceinline__ float select_by_mask(unsigned long long mask, float if_set, float if_clear) {
    float r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(if_clear), "v"(if_set), "s"(mask));
    return r;
}
__device__ __forceinline__ int select_by_mask(unsigned long long mask, int if_set, int if_clear) {
    int r;
    asm("v_cndmask_b32_e64 %0, %1, %2, %3" : "=v"(r) : "v"(if_clear), "v"(if_set), "s"(mask));
    return r;
}
__device__ __forceinline__ float select_or_zero(unsigned long long mask, float if_set) {
    float r;
    asm("v_cndmask_b32_e64 %0, 0, %1, %2" : "=v"(r) : "v"(if_set), "s"(mask));
    return r;
}

// measure_atomic_add_count: the wavefront's flush instruction issues one line-wide request per group of sixteen
// lanes that holds a non-zero value (nz: ballot of the lanes with one)
__device__ __forceinline__ void count_requests(uint32_t* counter, unsigned long long nz) {
    const uint32_t n = (uint32_t)((nz & 0xFFFFull) != 0) + (uint32_t)(((nz >> 16) & 0xFFFFull) != 0) +
                       (uint32_t)(((nz >> 32) & 0xFFFFull) != 0) + (uint32_t)((nz >> 48) != 0);
    if (n) atomicAdd(counter, n);
}

// Index of channel ch of pixel pid (= y * W + x) of image `batch` in the colour images: [B,H,W,C] or, with
// use_nchw, [B,C,H,W].
__device__ __forceinline__ size_t color_index(const d3gs_params& P, int batch, size_t pid, int ch, int channels) {
    const size_t plane = (size_t)P.width * P.height;
    return P.use_nchw ? ((size_t)batch * channels + ch) * plane + pid : ((size_t)batch * plane + pid) * channels + ch;
}

// Which camera of a bundle and which of its tiles a tile id b * tiles + y * tiles_x + x names (render.py:1515-1522,
// 1561); a single camera has batch 0.
struct TilePlace { int batch, tx, ty; };
__device__ __forceinline__ TilePlace place_tile(const d3gs_params& P, int tile) {
    const int per_view = P.tiles_x * P.tiles_y;
    TilePlace t;
    t.batch = P.batch_size > 1 ? tile / per_view : 0;
    const int local = tile - t.batch * per_view;
    t.ty = local / P.tiles_x;
    t.tx = local - t.ty * P.tiles_x;
    return t;
}

// kDepth: blend the camera-space depth as one more channel (render.py:1532-1539, 1915-1919).
// kRgba: fourth colour channel, the sum of the blend weights (render.py:1899-1906).
// kSnap: besides the image, store every pixel's running state (T and the colour accumulated so far) at the start
// of each bucket of kBucket list entries, for the per-gaussian backward (render.py:1744-1759).

}  // namespace d3gs
