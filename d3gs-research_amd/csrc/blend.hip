// Per-tile alpha blending, forward and backward.
//
// One 256-thread workgroup (4 wave64) per 16x16 tile; wave w owns the 8x8 pixel
// patch (w & 1, w >> 1) of the tile so that a wavefront covers a compact square
// and whole-wave culling of a gaussian is likely.  The tile's depth-sorted
// gaussians are staged 256 at a time into LDS by the whole workgroup and read
// back with wave-uniform (broadcast) addresses.
//
// Culling that keeps results exact: a gaussian contributes to a pixel only if
// alpha = min(0.99, o * exp(power)) >= alpha_eps.  Each staged gaussian carries
// thr = ln(alpha_eps / o) - 1e-3; power < thr implies alpha < alpha_eps with a
// margin four orders of magnitude above the rounding error of exp and log, so a
// pixel whose power is below thr never needs exp.  Two levels use it:
//   1. when a gaussian is staged, the bounding box of its {power >= thr} ellipse
//      (inflated by a bound on the rounding error of `power` inside this tile) is
//      tested against each wavefront's 8x8 patch; the four 64-bit ballots become
//      per-patch bit masks in LDS and a wavefront only visits gaussians whose
//      bit is set (scalar bit scan, no per-pixel work for the rest);
//   2. per pixel, `power < thr` skips the exact sequence.
// Every pixel that passes goes through the exact operation sequence, so the
// culling never changes a result.
//
// Reference: d3sim/algos/d3gs/render.py:1466-1570 (prologue), 1677-1923 (loop),
// 1924-2019 (gradients), 2020-2210 (reduction + atomics), 2222-2294 (epilogue).
#include "device_math.h"
#include "blend_common.h"

namespace d3gs {

template <bool kDepth, bool kRgba, bool kSnap>
__global__ __launch_bounds__(kBlock) void blend_fwd_kernel(const d3gs_params P, const int32_t* __restrict__ ranges,
                                                            const int32_t* __restrict__ idx_sorted,
                                                            const float* __restrict__ uvs,
                                                            const float* __restrict__ conic_opacity,
                                                            const float* __restrict__ rgb_g,
                                                            const float* __restrict__ depths,
                                                            const int32_t* __restrict__ tile_order,
                                                            float* __restrict__ color, float* __restrict__ final_T,
                                                            int32_t* __restrict__ n_contrib,
                                                            float* __restrict__ final_depth,
                                                            uint4* __restrict__ clear_vec, size_t clear_count,
                                                            const int32_t* __restrict__ bucket_offsets,
                                                            float4* __restrict__ snap) {
    // Optional service to the backward pass: this kernel hardly uses the memory pipes, so it clears the
    // caller's accumulator arrays (16-byte units, spread over all workgroups) on the side.
    if (clear_vec) {
        const size_t step = (size_t)gridDim.x * kBlock;
        for (size_t q = (size_t)blockIdx.x * kBlock + threadIdx.x; q < clear_count; q += step)
            clear_vec[q] = make_uint4(0u, 0u, 0u, 0u);
    }
    __shared__ StagedGaussian s_g[kBlock];
    __shared__ unsigned long long s_mask[4][4];   // [patch][64-gaussian chunk]
    constexpr int kChannels = kRgba ? 4 : 3;

    const int ntiles = P.tiles_x * P.tiles_y * batch_count(P);
    const int items = item_count(P);
    const int tile = tile_for_block(blockIdx.x, tile_order);
    if (tile < 0 || tile >= ntiles) return;
    const TilePlace place = place_tile(P, tile);
    const int tx = place.tx, ty = place.ty;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int px = tx * kTile + (wave & 1) * 8 + (lane & 7);
    const int py = ty * kTile + (wave >> 1) * 8 + (lane >> 3);
    const bool inside = px < P.width && py < P.height;
    const float pyf = (float)py;
    const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);

    const int r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int len = r1 - r0;
    const int rounds = (len + kBlock - 1) / kBlock;

    // "This pixel is finished" is kept in the pixel's x coordinate: a finished pixel's becomes NaN, which makes
    // its power NaN and fails the one ordered compare `power >= thr` that every visited gaussian pays for
    // anyway, so no separate test of a flag is needed.  (A loop-carried bool would live as a lane mask in
    // scalar registers and be merged with scalar instructions on every iteration.)
    float pxf = inside ? (float)px : __builtin_nanf("");
    float T = 1.0f;
    float acc0 = 0.0f, acc1 = 0.0f, acc2 = 0.0f, acc3 = 0.0f, depth_accum = 0.0f;
    int contributor = 0;

    for (int round = 0; round < rounds; ++round) {
        if (__syncthreads_count(pxf != pxf) == kBlock) break;
        const int src = r0 + round * kBlock + tid;
        uint32_t bits = 0;
        if (src < r1) {
            const int g = idx_sorted[src];
            if ((unsigned)g < (unsigned)items) {  // a corrupt index list must not become a wild read
                bits = stage_gaussian(P, g, uvs, conic_opacity, rgb_g, kDepth ? depths : nullptr, tile_x0, tile_y0,
                                      &s_g[tid]);
            }
        }
        publish_masks(bits, wave, lane, s_mask);
        __syncthreads();
        if (__all(pxf != pxf)) continue;
        for (int chunk = 0; chunk < 4; ++chunk) {
            if constexpr (kSnap) {
                // state of this wavefront's pixels in front of list entry round * 256 + chunk * 64 (a wavefront
                // whose pixels have all finished skips this: no gaussian from here on contributes to them)
                if (round * kBlock + chunk * kBucket < len) {
                    // one quad per pixel and bucket, two with an alpha or a depth channel (their running sums)
                    constexpr int kQuads = (kDepth || kRgba) ? 2 : 1;
                    float4* dst = snap + (((size_t)bucket_offsets[tile] + round * (kBlock / kBucket) + chunk) * kBlock + tid) * kQuads;
                    dst[0] = make_float4(T, acc0, acc1, acc2);
                    if constexpr (kQuads == 2) dst[1] = make_float4(acc3, depth_accum, 0.0f, 0.0f);
                }
            }
            unsigned long long m = uniform_u64(s_mask[wave][chunk]);
            while (m) {
                const int j = chunk * 64 + __builtin_ctzll(m);
                m &= m - 1;
                const StagedGaussian& sg = staged_at(s_g, j);
                const float dx = sg.x - pxf, dy = sg.y - pyf;
                const float power = blend_power(sg, dx, dy);
                // Per-lane conditions as 64-bit lane masks: one compare each, combined with scalar instructions
                // and applied with selects that take the mask from a scalar pair (as booleans the compiler formed
                // "any lane stops?" by a select into a vector register and a second compare, and both senses of
                // the transmittance test).  Ordered compares: a NaN fails them as it fails the C operators.
                const unsigned long long live_m = __builtin_amdgcn_fcmpf(power, sg.thr, kFcmpOge);   // a finished pixel: NaN
                if (live_m == 0ull) continue;
                // From here on every lane runs the same instructions and the outcome is applied with
                // selects (w = 0 leaves the accumulators untouched): far fewer scalar mask operations
                // than nested per-lane branches.  exp of a lane that is not live may be garbage; it is
                // never selected.
                // no overflow guard: beyond exp's range the product o * G is inf, huge or NaN, and
                // fminf(0.99, .) gives 0.99 in every case, as it does for the guarded exp's inf
                const float G = blend_expf(power);
                const float alpha = fminf(0.99f, sg.o * G);
                const unsigned long long hit_m = live_m & __builtin_amdgcn_fcmpf(alpha, P.alpha_eps, kFcmpOge);
                const float nextT = T * (1.0f - alpha);
                const unsigned long long done_m = __builtin_amdgcn_fcmpf(nextT, P.transmittance_eps, kFcmpOlt);
                const unsigned long long stop_m = hit_m & done_m;                      // render.py:1781-1792
                const unsigned long long use_m = hit_m & ~done_m & ~__builtin_amdgcn_fcmpf(power, 0.0f, kFcmpOgt);
                const float w = select_or_zero(use_m, alpha * T);
                T = select_by_mask(use_m, nextT, T);
                contributor = select_by_mask(use_m, round * kBlock + j, contributor);
                acc0 = __builtin_fmaf(w, sg.r, acc0);
                acc1 = __builtin_fmaf(w, sg.g, acc1);
                acc2 = __builtin_fmaf(w, sg.b, acc2);
                if constexpr (kRgba) acc3 = acc3 + w;
                if constexpr (kDepth) depth_accum = __builtin_fmaf(w, sg.depth, depth_accum);
                pxf = select_by_mask(stop_m, __builtin_nanf(""), pxf);
                // every pixel of the patch finished: both loops end at their next test (one way out of the
                // loops keeps the scalar control flow short; the scalar unit is shared by the CU's four SIMDs
                // and this kernel issues two scalar instructions for every three vector ones)
                if (stop_m != 0ull && __all(pxf != pxf)) {
                    m = 0ull;
                    chunk = 4;
                }
            }
        }
    }

    if (inside) {
        const size_t pid = (size_t)py * P.width + px;
        const size_t gpid = (size_t)place.batch * P.width * P.height + pid;     // pixel of the [B,H,W] images
        final_T[gpid] = T;
        n_contrib[gpid] = contributor;
        if constexpr (kDepth)  // inference normalises by the opacity (render.py:2244-2254)
            final_depth[gpid] = P.training ? depth_accum : depth_accum / ((1e-10f + 1.0f) - T);
        const float acc[4] = {acc0, acc1, acc2, acc3};
#pragma unroll
        for (int ch = 0; ch < kChannels; ++ch) {
            float v = acc[ch];
            // the alpha channel has no background (render.py:2227-2229)
            if (!P.training) v = fminf(fmaxf(v + T * (ch < 3 ? P.bg[ch] : 0.0f), 0.0f), 1.0f);
            color[color_index(P, place.batch, pid, ch, kChannels)] = v;
        }
    }
}

// ---------------------------------------------------------------------------
// Backward: front-to-back recompute; per gaussian the partial derivatives
// (nine, ten with depth) are summed over the wavefront, then over the tile's
// four wavefronts in LDS, and only then added to global memory: one atomic per
// value per (tile, gaussian).
// ---------------------------------------------------------------------------
// Gaussians staged per round: 224 instead of the workgroup's 256 keeps the kernel's LDS (staged records + ids +
// nine rows of sums) under 20 KiB, so that eight workgroups share a compute unit instead of seven (the plain colour
// instantiation is told to fit the 64 vector registers that takes; it does, without spilling).  The kernel is bound by
// how many wavefronts are there to hide each other's dependent chains: seven instead of five workgroups is worth 9-12 %.
constexpr int kBwdStage = 224;

template <bool kDepth, bool kRgba>
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu((kDepth || kRgba) ? 6 : 8, 8))) void blend_bwd_kernel(
    const d3gs_params P, const int32_t* __restrict__ ranges, const int32_t* __restrict__ idx_sorted,
    const float* __restrict__ uvs, const float* __restrict__ conic_opacity, const float* __restrict__ rgb_g,
    const float* __restrict__ depths, const int32_t* __restrict__ tile_order, const float* __restrict__ final_T,
    const int32_t* __restrict__ n_contrib, const float* __restrict__ color, const float* __restrict__ final_depth,
    const float* __restrict__ drgb, const float* __restrict__ dT, const float* __restrict__ ddepth,
    float* __restrict__ grad_records, uint8_t* __restrict__ touched) {
    constexpr int kValues = kDepth ? 10 : 9;
    constexpr int kChannels = kRgba ? 4 : 3;
    __shared__ StagedGaussian s_g[kBwdStage];
    __shared__ int s_id[kBwdStage];
    // one row per value; the odd row stride puts the (up to ten) lanes of one LDS atomic instruction,
    // which address the same gaussian in consecutive rows, into different banks
    __shared__ float s_grad[kValues][kBwdStage + 1];
    __shared__ int s_wmax[4];
    __shared__ unsigned long long s_mask[4][4];   // [patch][64-gaussian chunk]
#ifdef D3GS_TIMING_ONLY_LDS_PAD
    // fewer workgroups fit a compute unit: how the duration follows the number of resident wavefronts
    __shared__ int s_pad[D3GS_TIMING_ONLY_LDS_PAD / 4];
    if (P.n < 0) s_pad[threadIdx.x] = blockIdx.x;
#endif

    const int ntiles = P.tiles_x * P.tiles_y * batch_count(P);
    const int items = item_count(P);
    const int tile = tile_for_block(blockIdx.x, tile_order);
    if (tile < 0 || tile >= ntiles) return;
    const TilePlace place = place_tile(P, tile);
    const int tx = place.tx, ty = place.ty;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int px = tx * kTile + (wave & 1) * 8 + (lane & 7);
    const int py = ty * kTile + (wave >> 1) * 8 + (lane >> 3);
    const bool inside = px < P.width && py < P.height;
    const float pxf = (float)px, pyf = (float)py;
    const float tile_x0 = (float)(tx * kTile), tile_y0 = (float)(ty * kTile);
    const size_t pid = (size_t)py * P.width + px;
    const size_t gpid = (size_t)place.batch * P.width * P.height + pid;     // pixel of the [B,H,W] images

    const int r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int len = r1 - r0;
    if (len <= 0) return;

    int contributor = 0;
    float render_T = 0.0f, dT_val = 0.0f;
    float rr0 = 0.0f, rr1 = 0.0f, rr2 = 0.0f, rr3 = 0.0f, dr0 = 0.0f, dr1 = 0.0f, dr2 = 0.0f, dr3 = 0.0f;
    float rdep = 0.0f, ddep = 0.0f;
    if (inside) {
        contributor = min(n_contrib[gpid] + 1, len);
        render_T = final_T[gpid];
        dT_val = dT[gpid];
        rr0 = color[color_index(P, place.batch, pid, 0, kChannels)];
        rr1 = color[color_index(P, place.batch, pid, 1, kChannels)];
        rr2 = color[color_index(P, place.batch, pid, 2, kChannels)];
        dr0 = drgb[color_index(P, place.batch, pid, 0, kChannels)];
        dr1 = drgb[color_index(P, place.batch, pid, 1, kChannels)];
        dr2 = drgb[color_index(P, place.batch, pid, 2, kChannels)];
        if constexpr (kRgba) {
            rr3 = color[color_index(P, place.batch, pid, 3, kChannels)];
            dr3 = drgb[color_index(P, place.batch, pid, 3, kChannels)];
        }
        if constexpr (kDepth) {
            rdep = final_depth[gpid];
            ddep = ddepth[gpid];
        }
    }
    const float dT_term = (-dT_val) * render_T;
    int slot = reduce_slot(lane);
    if (slot >= kValues) slot = -1;
    // wave-uniform by construction; readfirstlane tells the compiler, which keeps the gaussian
    // bit masks and loop bounds below in scalar registers
    const int wave_todo = __builtin_amdgcn_readfirstlane(wave_max_i32(contributor));
    if (lane == 0) s_wmax[wave] = wave_todo;
    __syncthreads();
    const int block_todo = max(max(s_wmax[0], s_wmax[1]), max(s_wmax[2], s_wmax[3]));
    const int rounds = (block_todo + kBwdStage - 1) / kBwdStage;

    float T = 1.0f;
    for (int round = 0; round < rounds; ++round) {
        __syncthreads();  // previous round's flush has read s_grad / s_id
        const int src = r0 + round * kBwdStage + tid;
        uint32_t bits = 0;
        // entries behind the tile's last contributor are not staged
        if (tid < kBwdStage && src < r1 && round * kBwdStage + tid < block_todo) {
            const int g = idx_sorted[src];
            if ((unsigned)g < (unsigned)items) {
                s_id[tid] = g;
                bits = stage_gaussian(P, g, uvs, conic_opacity, rgb_g, kDepth ? depths : nullptr, tile_x0, tile_y0,
                                      &s_g[tid]);
            } else {
                // a corrupt index list must not become a wild read or write: the slot is staged as a gaussian
                // nobody visits (bits = 0) with finite parameters, and id -1 keeps the flush away from it
                s_id[tid] = -1;
                s_g[tid] = StagedGaussian{0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
        publish_masks(bits, wave, lane, s_mask);
        if (tid < kBwdStage) {
#pragma unroll
            for (int k = 0; k < kValues; ++k) s_grad[k][tid] = 0.0f;
        }
        __syncthreads();
        const int cnt = min(kBwdStage, wave_todo - round * kBwdStage);
        for (int chunk = 0; chunk < 4 && chunk * 64 < cnt; ++chunk) {
          unsigned long long m = uniform_u64(s_mask[wave][chunk]);
          if (cnt - chunk * 64 < 64) m &= (1ull << (cnt - chunk * 64)) - 1ull;
#ifdef D3GS_TIMING_ONLY_NO_VISITS
          m = 0ull;
#endif
          if (!m) continue;
          while (m) {
            const int j = chunk * 64 + __builtin_ctzll(m);
            m &= m - 1;
            const StagedGaussian& sg = staged_at(s_g, j);
            const float dx = sg.x - pxf, dy = sg.y - pyf;
            const float power = blend_power(sg, dx, dy);
            // Per-lane conditions as 64-bit lane masks (one compare instruction each, combined with scalar
            // instructions; ordered compares, a NaN fails them as it fails the C operators they stand for).
#ifdef D3GS_TIMING_ONLY_POWER_ONLY
            const unsigned long long cand_m = __builtin_amdgcn_sicmp(round * kBwdStage + j, contributor, kIcmpSlt) &
                                              __builtin_amdgcn_fcmpf(power, 1.0e30f, kFcmpOge) &
                                              __builtin_amdgcn_fcmpf(power, 0.0f, kFcmpOle);
#else
            const unsigned long long cand_m = __builtin_amdgcn_sicmp(round * kBwdStage + j, contributor, kIcmpSlt) &
                                              __builtin_amdgcn_fcmpf(power, sg.thr, kFcmpOge) &
                                              __builtin_amdgcn_fcmpf(power, 0.0f, kFcmpOle);
#endif
            if (cand_m == 0) continue;
            // power, exp and alpha repeat the forward's exact sequence: they decide which pixels the
            // gaussian contributed to.  From here on every lane runs the same instructions: a lane the
            // gaussian did not contribute to carries G = alpha = 0, which leaves its running state
            // (T, colour behind) untouched and makes all of its terms exact zeros, so no lane masking
            // or zero-filling is needed.  (exp of a non-candidate lane's power may be garbage; it is
            // discarded by the select.)
            const float G0 = blend_expf(power);   // candidates have power in [thr, 0]
            const float alpha0 = fminf(0.99f, sg.o * G0);
            const unsigned long long valid_m = cand_m & __builtin_amdgcn_fcmpf(alpha0, P.alpha_eps, kFcmpOge);
            if (valid_m == 0) continue;
            float G, alpha;     // G = valid ? G0 : 0, alpha = valid ? alpha0 : 0
            select2_or_zero(valid_m, G0, alpha0, G, alpha);
            // The per-pixel terms follow one fixed sequence of fused multiply-adds (the colour still
            // behind, T c - rr, cancels heavily, so a different rounding would already move a term by
            // ~1e-4): only the order of the sums over pixels differs from a sequential evaluation.
            const float one_m = 1.0f - alpha;
            const float w = alpha * T;
            T = T * one_m;
            rr0 = __builtin_fmaf(-w, sg.r, rr0);
            rr1 = __builtin_fmaf(-w, sg.g, rr1);
            rr2 = __builtin_fmaf(-w, sg.b, rr2);
            float dl = dT_term;
            float g9 = 0.0f;
            if constexpr (kDepth) {  // render.py:1887-1890, 1948-1950
                rdep = __builtin_fmaf(-w, sg.depth, rdep);
                dl = __builtin_fmaf(ddep, __builtin_fmaf(T, sg.depth, -rdep), dl);
                g9 = w * ddep;       // render.py:1964-1967
            }
            if constexpr (kRgba) {   // the alpha channel blends the constant 1 (render.py:1871-1874, 1926-1931)
                rr3 = rr3 - w;
                dl = __builtin_fmaf(dr3, T - rr3, dl);
            }
            dl = __builtin_fmaf(dr2, __builtin_fmaf(T, sg.b, -rr2), dl);
            dl = __builtin_fmaf(dr1, __builtin_fmaf(T, sg.g, -rr1), dl);
            dl = __builtin_fmaf(dr0, __builtin_fmaf(T, sg.r, -rr0), dl);
            // 1 - alpha lies in [0.01, 1): the hardware reciprocal (1 ulp) replaces the 11-instruction IEEE
            // division; the quotient scales every term of this pixel alike, by at most 2 ulp
            const float dL_dalpha = dl * __builtin_amdgcn_rcpf(one_m);
            // With q = dL/dG * G the screen-space gradients are linear in five moments of q:
            // dL/du = -(a S1 + b S2), dL/dv = -(c S2 + b S1), dL/dconic = (-S3/2, -S4, -S5/2), where
            // S1 = sum q dx, S2 = sum q dy, S3 = sum q dx^2, S4 = sum q dx dy, S5 = sum q dy^2
            // (render.py:1996-2017 evaluates the products per pixel).  The lanes only form the
            // moments; the per-gaussian map is applied once per (tile, gaussian) before the flush.
            const float g5 = dL_dalpha * G;
            const float q = sg.o * g5;
            const float g0 = q * dx;
            const float g1 = q * dy;
            const float g2 = g0 * dx;
            const float g3 = g0 * dy;
            const float g4 = g1 * dy;
            const float g6 = w * dr0;
            const float g7 = w * dr1;
            const float g8 = w * dr2;
            // the wave totals land in different lanes: one LDS atomic instruction adds them all
#ifdef D3GS_TIMING_ONLY_NO_REDUCTION
            asm volatile("" : : "v"(g0), "v"(g1), "v"(g2), "v"(g3), "v"(g4), "v"(g5), "v"(g6), "v"(g7), "v"(g8), "v"(g9));
            const float total = g5;
#else
            const float total = wave_reduce10<kDepth>(g0, g1, g2, g3, g4, g5, g6, g7, g8, g9);
#endif
            if (slot >= 0) atomicAdd(&s_grad[slot][j], total);
          }
        }
        __syncthreads();
#ifdef D3GS_TIMING_ONLY_NO_FLUSH
        continue;
#endif
        const int flush_cnt = min(kBwdStage, block_todo - round * kBwdStage);
        if (tid < flush_cnt) {  // moments -> (duv, dconic) of gaussian tid, with a = -2 ha, b = -nb, c = -2 hc
            const StagedGaussian sg = s_g[tid];
            const float S1 = s_grad[0][tid], S2 = s_grad[1][tid];
            s_grad[0][tid] = __builtin_fmaf(sg.nb, S2, (2.0f * sg.ha) * S1);
            s_grad[1][tid] = __builtin_fmaf(sg.nb, S1, (2.0f * sg.hc) * S2);
            s_grad[2][tid] = -0.5f * s_grad[2][tid];
            s_grad[3][tid] = -s_grad[3][tid];
            s_grad[4][tid] = -0.5f * s_grad[4][tid];
        }
        __syncthreads();
        // Flush: sixteen lanes add one gaussian's record (one 64-byte line) at a time, so the memory
        // side sees one line-wide atomic request per (tile, gaussian) instead of one per value.
        const int slot_k = tid & 15;
        for (int gl = tid >> 4; gl < flush_cnt; gl += kBlock / 16) {
            const int gid = s_id[gl];
            const float v = (slot_k < kValues && gid >= 0) ? s_grad[slot_k][gl] : 0.0f;
            if (v != 0.0f) unsafeAtomicAdd(grad_records + (size_t)D3GS_GRAD_RECORD_FLOATS * gid + slot_k, v);
            // one byte per gaussian that received anything: the preprocess backward finds its work in this
            // dense array instead of reading every record
            if (touched || P.atomic_add_count) {
                const unsigned long long nz = __ballot(v != 0.0f);
                if (touched && slot_k == 0 && ((nz >> (tid & 48)) & 0xFFFFull)) touched[gid] = 1;
                if (P.atomic_add_count && lane == 0) count_requests(P.atomic_add_count, nz);
            }
        }
    }
}


// ---------------------------------------------------------------------------
// Per-gaussian backward (render.py:2319-2776; config rasterize_backward_algo = PER_GAUSSIAN): the second
// algorithm for the same gradient.  Lanes are gaussians, not pixels: a wavefront takes one bucket of kBucket
// consecutive entries of a tile's list, every lane keeps its gaussian's nine sums in registers, and the pixels
// of the tile pass through the lanes one after the other, lane l handing a pixel's running state (T and the
// colour still behind) to lane l + 1 with a one-lane wave shift -- the order of the list -- so that no sum ever
// crosses lanes and each (tile, gaussian) ends in one line-wide atomic.  The state a pixel has in front of the
// bucket comes from the snapshots the forward pass stored (blend_fwd_kernel<.., kSnap>).  Only pixels that are
// still open at the bucket's start (their last contributor lies in or behind it) are passed through.
// The reference runs one 32-lane warp per bucket of 32; here a bucket is the 64 lanes of a wavefront and a
// workgroup (one per tile, longest lists first) deals its buckets to its four wavefronts.
// ---------------------------------------------------------------------------
template <int kCtrl>
__device__ __forceinline__ float dpp_shift_in(float fresh, float v) {
    // lanes 1..63 take v of the lane below; lane 0, which has no lane below, keeps `fresh`
    return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(fresh), __float_as_int(v), kCtrl, 0xF, 0xF, false));
}
constexpr int kDppWaveShr1 = 0x138;

// kDepth / kRgba: a depth and an alpha channel ride along as in the default kernel (render.py:2364-2398, 2412-2415,
// 2490-2528): their running sums are part of the pixel state handed from lane to lane, the snapshots hold them in a
// second quad, and the depth gradient is the record's tenth value.
template <bool kDepth, bool kRgba>
__global__ __launch_bounds__(kBlock) void blend_bwd_per_gaussian_kernel(
    const d3gs_params P, const int32_t* __restrict__ ranges, const int32_t* __restrict__ idx_sorted,
    const float* __restrict__ uvs, const float* __restrict__ conic_opacity, const float* __restrict__ rgb_g,
    const float* __restrict__ depths, const int32_t* __restrict__ tile_order, const float* __restrict__ final_T,
    const int32_t* __restrict__ n_contrib, const float* __restrict__ color, const float* __restrict__ final_depth,
    const float* __restrict__ drgb, const float* __restrict__ dT, const float* __restrict__ ddepth,
    const int32_t* __restrict__ bucket_offsets, const float4* __restrict__ snap, float* __restrict__ grad_records,
    uint8_t* __restrict__ touched) {
    constexpr int kWaves = kBlock / 64;
    constexpr bool kExtra = kDepth || kRgba;
    constexpr int kQuads = kExtra ? 2 : 1;
    constexpr int kChannels = kRgba ? 4 : 3;
    __shared__ float4 s_pix_grad[kBlock];    // per pixel: drgb (3), -dT * final_T
    __shared__ float4 s_pix_final[kBlock];   // per pixel: final colour (3), contributor (int bits)
    __shared__ float4 s_pix_extra[kExtra ? kBlock : 1];   // per pixel: d alpha, d depth, final alpha, final depth
    __shared__ float4 s_snap[kWaves][kBlock];            // the bucket's snapshots: T, colour in front of the bucket
    __shared__ float2 s_snap_extra[kExtra ? kWaves : 1][kExtra ? kBlock : 1];   // ... alpha and depth sums
    __shared__ unsigned short s_open[kWaves][kBlock];    // pixels still open at the bucket's start
    __shared__ float s_out[kWaves][kBucket][D3GS_GRAD_RECORD_FLOATS + 1];
    __shared__ int s_gid[kWaves][kBucket];
    __shared__ int s_wmax[kWaves];

    const int ntiles = P.tiles_x * P.tiles_y * batch_count(P);
    const int items = item_count(P);
    const int tile = tile_for_block(blockIdx.x, tile_order);
    if (tile < 0 || tile >= ntiles) return;
    const TilePlace place = place_tile(P, tile);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float tile_x0 = (float)(place.tx * kTile), tile_y0 = (float)(place.ty * kTile);
    const int r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int len = r1 - r0;
    if (len <= 0) return;

    {   // pixel tid of the tile, in the forward kernel's thread order (the snapshots are stored in that order)
        const int px = place.tx * kTile + (wave & 1) * 8 + (lane & 7);
        const int py = place.ty * kTile + (wave >> 1) * 8 + (lane >> 3);
        const bool inside = px < P.width && py < P.height;
        int contributor = 0;
        float4 pg = make_float4(0.0f, 0.0f, 0.0f, 0.0f), pf = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        float4 pe = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (inside) {
            const size_t pid = (size_t)py * P.width + px;
            const size_t gpid = (size_t)place.batch * P.width * P.height + pid;
            contributor = min(n_contrib[gpid] + 1, len);
            pg = make_float4(drgb[color_index(P, place.batch, pid, 0, kChannels)],
                             drgb[color_index(P, place.batch, pid, 1, kChannels)],
                             drgb[color_index(P, place.batch, pid, 2, kChannels)], (-dT[gpid]) * final_T[gpid]);
            pf = make_float4(color[color_index(P, place.batch, pid, 0, kChannels)],
                             color[color_index(P, place.batch, pid, 1, kChannels)],
                             color[color_index(P, place.batch, pid, 2, kChannels)], 0.0f);
            if constexpr (kRgba) {
                pe.x = drgb[color_index(P, place.batch, pid, 3, kChannels)];
                pe.z = color[color_index(P, place.batch, pid, 3, kChannels)];
            }
            if constexpr (kDepth) {
                pe.y = ddepth[gpid];
                pe.w = final_depth[gpid];
            }
        }
        pf.w = __int_as_float(contributor);
        s_pix_grad[tid] = pg;
        s_pix_final[tid] = pf;
        if constexpr (kExtra) s_pix_extra[tid] = pe;
        const int wmax = wave_max_i32(contributor);
        if (lane == 0) s_wmax[wave] = wmax;
    }
    __syncthreads();
    const int block_todo = max(max(s_wmax[0], s_wmax[1]), max(s_wmax[2], s_wmax[3]));
    const int nbuckets = (block_todo + kBucket - 1) / kBucket;
    const unsigned long long lt_mask = (1ull << lane) - 1ull;

    for (int bucket = wave; bucket < nbuckets; bucket += kWaves) {      // wave-uniform
        const int bstart = bucket * kBucket;
        // the bucket's snapshots, and the list of pixels still open at its start
        const float4* sb = snap + ((size_t)bucket_offsets[tile] + bucket) * kBlock * kQuads;
        int cnt = 0;
#pragma unroll
        for (int q = 0; q < kBlock / 64; ++q) {
            const int p = q * 64 + lane;
            const bool open = __float_as_int(s_pix_final[p].w) > bstart;
            // a snapshot of a finished pixel may never have been written: it is not read, and not staged
            s_snap[wave][p] = open ? sb[(size_t)p * kQuads] : make_float4(1.0f, 0.0f, 0.0f, 0.0f);
            if constexpr (kExtra) {
                const float4 e = open ? sb[(size_t)p * kQuads + 1] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                s_snap_extra[wave][p] = make_float2(e.x, e.y);
            }
            const unsigned long long bal = __ballot(open);
            if (open) s_open[wave][cnt + __popcll(bal & lt_mask)] = (unsigned short)p;
            cnt += __popcll(bal);
        }
        cnt = __builtin_amdgcn_readfirstlane(cnt);
        // this lane's gaussian
        const int li = bstart + lane;
        int gid = -1;
        StagedGaussian sg = StagedGaussian{0.0f, 0.0f, __builtin_inff(), 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        float c0 = 0.0f, c1 = 0.0f, c2 = 0.0f;
        if (li < len) {
            const int g = idx_sorted[r0 + li];
            if ((unsigned)g < (unsigned)items) {   // a corrupt index list must not become a wild read or write
                gid = g;
                stage_gaussian(P, g, uvs, conic_opacity, rgb_g, kDepth ? depths : nullptr, tile_x0, tile_y0, &sg);
                c0 = sg.r;
                c1 = sg.g;
                c2 = sg.b;
            }
        }
        __builtin_amdgcn_wave_barrier();    // the wavefront's own LDS writes above are read below
        float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f, a4 = 0.0f, a5 = 0.0f, a6 = 0.0f, a7 = 0.0f, a8 = 0.0f, a9 = 0.0f;
        float T = 1.0f, rr0 = 0.0f, rr1 = 0.0f, rr2 = 0.0f, rr3 = 0.0f, rdep = 0.0f;
        const int steps = cnt > 0 ? cnt + kBucket - 1 : 0;
        for (int j = 0; j < steps; ++j) {
            // lane 0 takes up open pixel j with the state it has in front of the bucket; every other lane takes
            // over the pixel its lower neighbour has just finished with
            const int q = j < cnt ? s_open[wave][j] : 0;     // wave-uniform
            const float4 sn = s_snap[wave][q];
            const float4 fin = s_pix_final[q];
            const bool fresh = j < cnt;
            T = dpp_shift_in<kDppWaveShr1>(fresh ? sn.x : 1.0f, T);
            rr0 = dpp_shift_in<kDppWaveShr1>(fresh ? fin.x - sn.y : 0.0f, rr0);
            rr1 = dpp_shift_in<kDppWaveShr1>(fresh ? fin.y - sn.z : 0.0f, rr1);
            rr2 = dpp_shift_in<kDppWaveShr1>(fresh ? fin.z - sn.w : 0.0f, rr2);
            if constexpr (kExtra) {
                const float2 se = s_snap_extra[wave][q];
                const float4 fe = s_pix_extra[q];
                if constexpr (kRgba) rr3 = dpp_shift_in<kDppWaveShr1>(fresh ? fe.z - se.x : 0.0f, rr3);
                if constexpr (kDepth) rdep = dpp_shift_in<kDppWaveShr1>(fresh ? fe.w - se.y : 0.0f, rdep);
            }
            const int k = j - lane;                        // which open pixel this lane holds now
            const bool holding = k >= 0 && k < cnt;
            const int p = holding ? s_open[wave][k] : 0;
            const float4 pg = s_pix_grad[p];
            const int contributor = __float_as_int(s_pix_final[p].w);
            const float pxf = tile_x0 + (float)(((p >> 6) & 1) * 8 + (p & 7));
            const float pyf = tile_y0 + (float)((p >> 7) * 8 + ((p >> 3) & 7));
            const float dx = sg.x - pxf, dy = sg.y - pyf;
            const float power = blend_power(sg, dx, dy);
            // the forward's exact sequence decides which pixels the gaussian contributed to
            const bool cand = holding && li < contributor && power >= sg.thr && power <= 0.0f;
            const float G0 = det_expf_inrange(cand ? power : 0.0f);
            const float alpha0 = fminf(0.99f, sg.o * G0);
            const bool valid = cand && alpha0 >= P.alpha_eps;
            const float G = valid ? G0 : 0.0f, alpha = valid ? alpha0 : 0.0f;
            const float one_m = 1.0f - alpha;
            const float w = alpha * T;
            T = T * one_m;
            rr0 = __builtin_fmaf(-w, c0, rr0);
            rr1 = __builtin_fmaf(-w, c1, rr1);
            rr2 = __builtin_fmaf(-w, c2, rr2);
            float dl = pg.w;
            if constexpr (kDepth) {      // the default kernel's order of terms: depth, alpha, then blue, green, red
                const float ddep = s_pix_extra[p].y;
                rdep = __builtin_fmaf(-w, sg.depth, rdep);
                dl = __builtin_fmaf(ddep, __builtin_fmaf(T, sg.depth, -rdep), dl);
                a9 += w * ddep;
            }
            if constexpr (kRgba) {
                rr3 = rr3 - w;
                dl = __builtin_fmaf(s_pix_extra[p].x, T - rr3, dl);
            }
            dl = __builtin_fmaf(pg.z, __builtin_fmaf(T, c2, -rr2), dl);
            dl = __builtin_fmaf(pg.y, __builtin_fmaf(T, c1, -rr1), dl);
            dl = __builtin_fmaf(pg.x, __builtin_fmaf(T, c0, -rr0), dl);
            const float dL_dalpha = dl * __builtin_amdgcn_rcpf(one_m);
            const float g5 = dL_dalpha * G;
            const float qv = sg.o * g5;
            const float g0 = qv * dx, g1 = qv * dy;
            a0 += g0;
            a1 += g1;
            a2 += g0 * dx;
            a3 += g0 * dy;
            a4 += g1 * dy;
            a5 += g5;
            a6 += w * pg.x;
            a7 += w * pg.y;
            a8 += w * pg.z;
        }
        // moments -> (duv, dconic) with a = -2 ha, b = -nb, c = -2 hc, as the default kernel's flush does
        float* row = s_out[wave][lane];
        row[0] = __builtin_fmaf(sg.nb, a1, (2.0f * sg.ha) * a0);
        row[1] = __builtin_fmaf(sg.nb, a0, (2.0f * sg.hc) * a1);
        row[2] = -0.5f * a2;
        row[3] = -a3;
        row[4] = -0.5f * a4;
        row[5] = a5;
        row[6] = a6;
        row[7] = a7;
        row[8] = a8;
        row[9] = a9;
#pragma unroll
        for (int c = 10; c < D3GS_GRAD_RECORD_FLOATS; ++c) row[c] = 0.0f;
        s_gid[wave][lane] = gid;
        __builtin_amdgcn_wave_barrier();
        // sixteen lanes add one gaussian's record: one line-wide atomic per (tile, gaussian)
        const int slot_k = lane & 15;
#pragma unroll
        for (int r = 0; r < kBucket / 4; ++r) {
            const int gl = r * 4 + (lane >> 4);
            const int id = s_gid[wave][gl];
            const float v = id >= 0 ? s_out[wave][gl][slot_k] : 0.0f;
            if (v != 0.0f) unsafeAtomicAdd(grad_records + (size_t)D3GS_GRAD_RECORD_FLOATS * id + slot_k, v);
            if (touched || P.atomic_add_count) {
                const unsigned long long nz = __ballot(v != 0.0f);
                if (touched && slot_k == 0 && ((nz >> (lane & 48)) & 0xFFFFull)) touched[id] = 1;
                if (P.atomic_add_count && lane == 0) count_requests(P.atomic_add_count, nz);
            }
        }
        __builtin_amdgcn_wave_barrier();    // the next bucket overwrites this wavefront's tables
    }
}

// Exclusive prefix sum of the tiles' bucket counts ceil(list length / kBucket) (render.py:940-950): where each
// tile's snapshots start.  One workgroup; out[num_tiles] is the total.
__global__ __launch_bounds__(1024) void bucket_offsets_kernel(const int32_t* __restrict__ ranges, int num_tiles,
                                                              int32_t* __restrict__ out) {
    __shared__ int s_wave[16];
    __shared__ int s_carry;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) s_carry = 0;
    __syncthreads();
    for (int base = 0; base < num_tiles; base += 1024) {
        const int t = base + tid;
        int c = 0;
        if (t < num_tiles) c = (max(ranges[2 * t + 1] - ranges[2 * t], 0) + kBucket - 1) / kBucket;
        int incl = c;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, 64);
            if (lane >= off) incl += v;
        }
        if (lane == 63) s_wave[wave] = incl;
        __syncthreads();
        int before = s_carry, total = 0;
#pragma unroll
        for (int w = 0; w < 16; ++w) {
            const int v = s_wave[w];
            if (w < wave) before += v;
            total += v;
        }
        if (t < num_tiles) out[t] = before + incl - c;
        __syncthreads();
        if (tid == 0) s_carry += total;
        __syncthreads();
    }
    if (tid == 0) out[num_tiles] = s_carry;
}

}  // namespace d3gs

using namespace d3gs;

static int blend_grid(const d3gs_params* p) { return p->tiles_x * p->tiles_y * batch_count(*p); }

static int finish_launch(const char* who) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", who, hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

static int launch_blend_fwd(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                            const float* uvs, const float* conic_opacity, const float* rgb_gaussian, const float* depths,
                            const int32_t* tile_order, float* color, float* final_T, int32_t* n_contrib,
                            float* final_depth, void* clear_ptr, size_t clear_bytes, const int32_t* bucket_offsets,
                            float4* snap, d3gs_stream_t stream) {
#define D3GS_LAUNCH_FWD(D, A, S)                                                                                    \
    hipLaunchKernelGGL((blend_fwd_kernel<D, A, S>), dim3(blend_grid(p)), dim3(kBlock), 0, (hipStream_t)stream, *p,  \
                       workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, rgb_gaussian, depths, tile_order,  \
                       color, final_T, n_contrib, final_depth, (uint4*)clear_ptr, clear_bytes / 16, bucket_offsets, snap)
    if (snap) {
        if (p->render_depth) { if (p->render_rgba) D3GS_LAUNCH_FWD(true, true, true); else D3GS_LAUNCH_FWD(true, false, true); }
        else                 { if (p->render_rgba) D3GS_LAUNCH_FWD(false, true, true); else D3GS_LAUNCH_FWD(false, false, true); }
    }
    else if (p->render_depth) { if (p->render_rgba) D3GS_LAUNCH_FWD(true, true, false); else D3GS_LAUNCH_FWD(true, false, false); }
    else                      { if (p->render_rgba) D3GS_LAUNCH_FWD(false, true, false); else D3GS_LAUNCH_FWD(false, false, false); }
#undef D3GS_LAUNCH_FWD
    return finish_launch("d3gs_blend_fwd");
}

extern "C" int d3gs_blend_fwd(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                              const float* uvs, const float* conic_opacity, const float* rgb_gaussian,
                              const float* depths, const int32_t* tile_order, float* color, float* final_T,
                              int32_t* n_contrib, float* final_depth, void* clear_ptr, size_t clear_bytes,
                              d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_blend_fwd");
    if (rc) return rc;
    if (clear_ptr && ((((uintptr_t)clear_ptr) | clear_bytes) & 15u)) {
        set_error("d3gs_blend_fwd: clear_ptr / clear_bytes must be multiples of 16");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (!workload_ranges || !uvs || !conic_opacity || !rgb_gaussian || !color || !final_T || !n_contrib ||
        (p->render_depth && (!depths || !final_depth))) {
        set_error("d3gs_blend_fwd: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    return launch_blend_fwd(p, workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, rgb_gaussian, depths, tile_order,
                            color, final_T, n_contrib, final_depth, clear_ptr, clear_bytes, nullptr, nullptr, stream);
}

extern "C" int d3gs_snapshot_floats(const d3gs_params* p) {
    return (p && (p->render_depth || p->render_rgba)) ? 8 : 4;
}

extern "C" int d3gs_blend_fwd_snapshots(const d3gs_params* p, const int32_t* workload_ranges,
                                        const int32_t* gaussian_idx_sorted, const float* uvs, const float* conic_opacity,
                                        const float* rgb_gaussian, const float* depths, const int32_t* tile_order,
                                        float* color, float* final_T, int32_t* n_contrib, float* final_depth,
                                        void* clear_ptr, size_t clear_bytes, const int32_t* bucket_offsets,
                                        float* snapshots, d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_blend_fwd_snapshots");
    if (rc) return rc;
    if (clear_ptr && ((((uintptr_t)clear_ptr) | clear_bytes) & 15u)) {
        set_error("d3gs_blend_fwd_snapshots: clear_ptr / clear_bytes must be multiples of 16");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (!workload_ranges || !uvs || !conic_opacity || !rgb_gaussian || !color || !final_T || !n_contrib ||
        !bucket_offsets || !snapshots || (((uintptr_t)snapshots) & 15u) || (p->render_depth && (!depths || !final_depth))) {
        set_error("d3gs_blend_fwd_snapshots: NULL buffer (snapshots must be 16-byte aligned)");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    return launch_blend_fwd(p, workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, rgb_gaussian, depths, tile_order,
                            color, final_T, n_contrib, final_depth, clear_ptr, clear_bytes, bucket_offsets,
                            (float4*)snapshots, stream);
}

extern "C" int d3gs_blend_bwd(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                              const float* uvs, const float* conic_opacity, const float* rgb_gaussian,
                              const float* depths, const int32_t* tile_order, const float* final_T,
                              const int32_t* n_contrib, const float* color, const float* final_depth,
                              const float* drgb, const float* dT, const float* ddepth, float* grad_records,
                              uint8_t* touched, d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_blend_bwd");
    if (rc) return rc;
    if (!workload_ranges || !uvs || !conic_opacity || !rgb_gaussian || !final_T || !n_contrib || !color || !drgb ||
        !dT || !grad_records || (p->render_depth && (!depths || !final_depth || !ddepth))) {
        set_error("d3gs_blend_bwd: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
#define D3GS_LAUNCH_BWD(D, A)                                                                                       \
    hipLaunchKernelGGL((blend_bwd_kernel<D, A>), dim3(blend_grid(p)), dim3(kBlock), 0, (hipStream_t)stream, *p,     \
                       workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, rgb_gaussian, depths, tile_order,  \
                       final_T, n_contrib, color, final_depth, drgb, dT, ddepth, grad_records, touched)
    if (p->render_depth) { if (p->render_rgba) D3GS_LAUNCH_BWD(true, true); else D3GS_LAUNCH_BWD(true, false); }
    else                 { if (p->render_rgba) D3GS_LAUNCH_BWD(false, true); else D3GS_LAUNCH_BWD(false, false); }
#undef D3GS_LAUNCH_BWD
    return finish_launch("d3gs_blend_bwd");
}

extern "C" int d3gs_bucket_offsets(const int32_t* workload_ranges, int32_t num_tiles, int32_t* bucket_offsets,
                                   d3gs_stream_t stream) {
    if (num_tiles < 0 || !bucket_offsets || (num_tiles > 0 && !workload_ranges)) {
        set_error("d3gs_bucket_offsets: bad argument");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    hipLaunchKernelGGL(bucket_offsets_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, workload_ranges, (int)num_tiles,
                       bucket_offsets);
    return finish_launch("d3gs_bucket_offsets");
}

extern "C" int d3gs_blend_bwd_per_gaussian(const d3gs_params* p, const int32_t* workload_ranges,
                                           const int32_t* gaussian_idx_sorted, const float* uvs, const float* conic_opacity,
                                           const float* rgb_gaussian, const float* depths, const int32_t* tile_order,
                                           const float* final_T, const int32_t* n_contrib, const float* color,
                                           const float* final_depth, const float* drgb, const float* dT,
                                           const float* ddepth, const int32_t* bucket_offsets, const float* snapshots,
                                           float* grad_records, uint8_t* touched, d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_blend_bwd_per_gaussian");
    if (rc) return rc;
    if (!workload_ranges || !uvs || !conic_opacity || !rgb_gaussian || !final_T || !n_contrib || !color || !drgb || !dT ||
        !bucket_offsets || !snapshots || !grad_records || (((uintptr_t)snapshots) & 15u) ||
        (p->render_depth && (!depths || !final_depth || !ddepth))) {
        set_error("d3gs_blend_bwd_per_gaussian: NULL buffer (snapshots must be 16-byte aligned)");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
#define D3GS_LAUNCH_PG(D, A)                                                                                          \
    hipLaunchKernelGGL((blend_bwd_per_gaussian_kernel<D, A>), dim3(blend_grid(p)), dim3(kBlock), 0, (hipStream_t)stream, \
                       *p, workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, rgb_gaussian, depths, tile_order,  \
                       final_T, n_contrib, color, final_depth, drgb, dT, ddepth, bucket_offsets,                       \
                       (const float4*)snapshots, grad_records, touched)
    if (p->render_depth) { if (p->render_rgba) D3GS_LAUNCH_PG(true, true); else D3GS_LAUNCH_PG(true, false); }
    else                 { if (p->render_rgba) D3GS_LAUNCH_PG(false, true); else D3GS_LAUNCH_PG(false, false); }
#undef D3GS_LAUNCH_PG
    return finish_launch("d3gs_blend_bwd_per_gaussian");
}
