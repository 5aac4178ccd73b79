// Custom feature channels through the blend (render.py:241-246, 1536-1538, 1571-1573, 1718-1721, 1854-1866,
// 1892-1895, 1920-1923, 1952-1955, 1969-1972, 2043-2045, 2113-2117, 2268-2270): every gaussian carries F extra
// values that are blended like a colour, C_f = sum_i T_i alpha_i f_i.  The reference compiles the channel count
// into its one rasterize kernel; here the colour kernels stay as they are and the features get kernels of their
// own that carry up to 16 channels per pass (forward) or 14 (backward) beside one evaluation of alpha:
//
//   forward   the colour forward's walk (same staging, cull, masks and per-pixel sequence, so the same pixels take
//             the same weights), with the channels' accumulators in registers and the features of the staged
//             gaussians in LDS beside their records;
//   backward  the colour backward's walk; per visit the channels' share of dL/dalpha is summed before the one
//             division by 1 - alpha, the five moments and the opacity term are formed from it, and the
//             per-gaussian sums (6 + channels values) go through the transposing wave reduction ten at a time.
//             The geometry sums are added to the gradient records of the colour pass (columns 0..5), the
//             channels' to dfeatures.
#include "blend_common.h"

namespace d3gs {

template <int kC>
__global__ __launch_bounds__(kBlock) void blend_features_fwd_kernel(
    const d3gs_params P, const int32_t* __restrict__ ranges, const int32_t* __restrict__ idx_sorted,
    const float* __restrict__ uvs, const float* __restrict__ conic_opacity, const float* __restrict__ features,
    const int F, const int c0, const int width, const int32_t* __restrict__ tile_order, float* __restrict__ out) {
    __shared__ StagedGaussian s_g[kBlock];
    __shared__ __attribute__((aligned(16))) float s_f[kBlock * kC];
    __shared__ unsigned long long s_mask[4][4];   // [patch][64-gaussian chunk]

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

    // a finished pixel's x coordinate becomes NaN, as in the colour forward
    float pxf = inside ? (float)px : __builtin_nanf("");
    float T = 1.0f;
    float acc[kC];
#pragma unroll
    for (int c = 0; c < kC; ++c) acc[c] = 0.0f;

    for (int round = 0; round < rounds; ++round) {
        if (__syncthreads_count(pxf != pxf) == kBlock) break;
        const int src = r0 + round * kBlock + tid;
        uint32_t bits = 0;
        if (src < r1) {
            const int g = idx_sorted[src];
            if ((unsigned)g < (unsigned)items) {  // a corrupt index list must not become a wild read
                bits = stage_gaussian<false>(P, g, uvs, conic_opacity, nullptr, nullptr, tile_x0, tile_y0, &s_g[tid]);
                const float* row = features + (size_t)g * F + c0;
#pragma unroll
                for (int c = 0; c < kC; ++c) s_f[tid * kC + c] = c < width ? row[c] : 0.0f;
            }
        }
        publish_masks(bits, wave, lane, s_mask);
        __syncthreads();
        if (__all(pxf != pxf)) continue;
        for (int chunk = 0; chunk < 4; ++chunk) {
            unsigned long long m = uniform_u64(s_mask[wave][chunk]);
            while (m) {
                const int j = chunk * 64 + __builtin_ctzll(m);
                m &= m - 1;
                const StagedGaussian& sg = staged_at(s_g, j);
                const float dx = sg.x - pxf, dy = sg.y - pyf;
                const float power = blend_power(sg, dx, dy);
                const unsigned long long live_m = __builtin_amdgcn_fcmpf(power, sg.thr, kFcmpOge);   // a finished pixel: NaN
                if (live_m == 0ull) continue;
                // the colour forward's sequence (render.py:1765-1792): the same pixels take the same weights
                const float G = blend_expf(power);
                const float alpha = fminf(0.99f, sg.o * G);
                const unsigned long long hit_m = live_m & __builtin_amdgcn_fcmpf(alpha, P.alpha_eps, kFcmpOge);
                const float nextT = T * (1.0f - alpha);
                const unsigned long long done_m = __builtin_amdgcn_fcmpf(nextT, P.transmittance_eps, kFcmpOlt);
                const unsigned long long stop_m = hit_m & done_m;
                const unsigned long long use_m = hit_m & ~done_m & ~__builtin_amdgcn_fcmpf(power, 0.0f, kFcmpOgt);
                const float w = select_or_zero(use_m, alpha * T);
                T = select_by_mask(use_m, nextT, T);
                const float* f = s_f + j * kC;      // wave-uniform: broadcast reads
#pragma unroll
                for (int c = 0; c < kC; ++c) acc[c] = __builtin_fmaf(w, f[c], acc[c]);      // render.py:1920-1923
                pxf = select_by_mask(stop_m, __builtin_nanf(""), pxf);
                if (stop_m != 0ull && __all(pxf != pxf)) {
                    m = 0ull;
                    chunk = 4;
                }
            }
        }
    }
    if (inside) {
        const size_t gpid = (size_t)place.batch * P.width * P.height + (size_t)py * P.width + px;
        float* dst = out + gpid * F + c0;
#pragma unroll
        for (int c = 0; c < kC; ++c)
            if (c < width) dst[c] = acc[c];
    }
}

// Backward: kC = 4 (ten sums per gaussian, one reduction) or 14 (twenty, two reductions).
template <int kC>
__global__ __launch_bounds__(kBlock) void blend_features_bwd_kernel(
    const d3gs_params P, const int32_t* __restrict__ ranges, const int32_t* __restrict__ idx_sorted,
    const float* __restrict__ uvs, const float* __restrict__ conic_opacity, const float* __restrict__ features,
    const int F, const int c0, const int width, const int32_t* __restrict__ tile_order,
    const int32_t* __restrict__ n_contrib, const float* __restrict__ feature_image,
    const float* __restrict__ dfeature_image, float* __restrict__ grad_records, float* __restrict__ dfeatures,
    uint8_t* __restrict__ touched) {
    static_assert(kC == 4 || kC == 14, "6 + kC sums per gaussian, reduced ten at a time");
    constexpr int kValues = 6 + kC;
    constexpr int kFlushLanes = kValues > 16 ? 32 : 16;
    // gaussians staged per round: half a workgroup's worth keeps the twenty rows of sums, the features and the
    // records of the wide instantiation at 24 KB, so that the registers (five wavefronts per SIMD), not the LDS
    // (three with 256 staged), decide how many wavefronts hide each other's dependent chains
    constexpr int kStage = 128;
    __shared__ StagedGaussian s_g[kStage];
    __shared__ int s_id[kStage];
    __shared__ __attribute__((aligned(16))) float s_f[kStage * kC];
    __shared__ float s_grad[kValues][kStage + 1];     // odd row stride: the lanes of one LDS atomic hit different banks
    __shared__ int s_wmax[4];
    __shared__ unsigned long long s_mask[4][4];

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
    const size_t gpid = (size_t)place.batch * P.width * P.height + (size_t)py * P.width + px;

    const int r0 = ranges[2 * tile], r1 = ranges[2 * tile + 1];
    const int len = r1 - r0;
    if (len <= 0) return;

    int contributor = 0;
    float behind[kC], dF[kC];      // the channels' blend still behind the walk; dL/d(feature image)
#pragma unroll
    for (int c = 0; c < kC; ++c) behind[c] = dF[c] = 0.0f;
    if (inside) {
        contributor = min(n_contrib[gpid] + 1, len);
        const float* img = feature_image + gpid * F + c0;
        const float* dimg = dfeature_image + gpid * F + c0;
#pragma unroll
        for (int c = 0; c < kC; ++c) {
            if (c < width) {
                behind[c] = img[c];
                dF[c] = dimg[c];
            }
        }
    }
    int slot = reduce_slot(lane);
    const int wave_todo = __builtin_amdgcn_readfirstlane(wave_max_i32(contributor));
    if (lane == 0) s_wmax[wave] = wave_todo;
    __syncthreads();
    const int block_todo = max(max(s_wmax[0], s_wmax[1]), max(s_wmax[2], s_wmax[3]));
    const int rounds = (block_todo + kStage - 1) / kStage;

    float T = 1.0f;
    for (int round = 0; round < rounds; ++round) {
        __syncthreads();  // previous round's flush has read s_grad / s_id
        const int src = r0 + round * kStage + tid;
        uint32_t bits = 0;
        if (tid < kStage) s_id[tid] = -1;
        if (tid < kStage && src < r1 && round * kStage + tid < block_todo) {
            const int g = idx_sorted[src];
            if ((unsigned)g < (unsigned)items) {
                s_id[tid] = g;
                bits = stage_gaussian<false>(P, g, uvs, conic_opacity, nullptr, nullptr, tile_x0, tile_y0, &s_g[tid]);
                const float* row = features + (size_t)g * F + c0;
#pragma unroll
                for (int c = 0; c < kC; ++c) s_f[tid * kC + c] = c < width ? row[c] : 0.0f;
            }
        }
        publish_masks(bits, wave, lane, s_mask);
        if (tid < kStage) {
#pragma unroll
            for (int k = 0; k < kValues; ++k) s_grad[k][tid] = 0.0f;
        }
        __syncthreads();
        const int cnt = min(kStage, wave_todo - round * kStage);
        for (int chunk = 0; chunk < kStage / 64 && chunk * 64 < cnt; ++chunk) {
            unsigned long long m = uniform_u64(s_mask[wave][chunk]);
            if (cnt - chunk * 64 < 64) m &= (1ull << (cnt - chunk * 64)) - 1ull;
            while (m) {
                const int j = chunk * 64 + __builtin_ctzll(m);
                m &= m - 1;
                const StagedGaussian& sg = staged_at(s_g, j);
                const float dx = sg.x - pxf, dy = sg.y - pyf;
                const float power = blend_power(sg, dx, dy);
                const unsigned long long cand_m = __builtin_amdgcn_sicmp(round * kStage + j, contributor, kIcmpSlt) &
                                                  __builtin_amdgcn_fcmpf(power, sg.thr, kFcmpOge) &
                                                  __builtin_amdgcn_fcmpf(power, 0.0f, kFcmpOle);
                if (cand_m == 0) continue;
                // power, exp and alpha repeat the forward's sequence; a lane the gaussian did not contribute to
                // carries G = alpha = 0, which makes all of its terms exact zeros
                const float G0 = blend_expf(power);
                const float alpha0 = fminf(0.99f, sg.o * G0);
                const unsigned long long valid_m = cand_m & __builtin_amdgcn_fcmpf(alpha0, P.alpha_eps, kFcmpOge);
                if (valid_m == 0) continue;
                float G, alpha;
                select2_or_zero(valid_m, G0, alpha0, G, alpha);
                const float one_m = 1.0f - alpha;
                const float w = alpha * T;
                T = T * one_m;
                const float* f = s_f + j * kC;      // wave-uniform: broadcast reads
                float dl = 0.0f, gf[kC];
#pragma unroll
                for (int c = kC - 1; c >= 0; --c) {
                    behind[c] = __builtin_fmaf(-w, f[c], behind[c]);                              // render.py:1892-1895
                    dl = __builtin_fmaf(dF[c], __builtin_fmaf(T, f[c], -behind[c]), dl);          // render.py:1952-1955
                    gf[c] = w * dF[c];                                                            // render.py:1969-1972
                }
                const float dL_dalpha = dl * __builtin_amdgcn_rcpf(one_m);
                const float g5 = dL_dalpha * G;
                const float q = sg.o * g5;
                const float g0 = q * dx;
                const float g1 = q * dy;
                const float g2 = g0 * dx;
                const float g3 = g0 * dy;
                const float g4 = g1 * dy;
                const float first = wave_reduce10<true>(g0, g1, g2, g3, g4, g5, gf[0], gf[1], gf[2], gf[3]);
                if (slot >= 0) atomicAdd(&s_grad[slot][j], first);
                if constexpr (kC == 14) {
                    const float second = wave_reduce10<true>(gf[4], gf[5], gf[6], gf[7], gf[8], gf[9], gf[10], gf[11],
                                                             gf[12], gf[13]);
                    if (slot >= 0) atomicAdd(&s_grad[10 + slot][j], second);
                }
            }
        }
        __syncthreads();
        const int flush_cnt = min(kStage, block_todo - round * kStage);
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
        // Flush: a group of lanes adds one gaussian's sums at a time: the first six to its gradient record (one
        // 64-byte line), the channels' to its row of dfeatures.
        const int slot_k = tid & (kFlushLanes - 1);
        for (int gl = tid / kFlushLanes; gl < flush_cnt; gl += kBlock / kFlushLanes) {
            const int gid = s_id[gl];
            const bool mine = slot_k < 6 || slot_k - 6 < width;
            const float v = (slot_k < kValues && mine && gid >= 0) ? s_grad[slot_k][gl] : 0.0f;
            if (v != 0.0f) {
                float* dst = slot_k < 6 ? grad_records + (size_t)D3GS_GRAD_RECORD_FLOATS * gid + slot_k
                                        : dfeatures + (size_t)gid * F + c0 + (slot_k - 6);
                unsafeAtomicAdd(dst, v);
            }
            if (touched) {      // the preprocess backward finds its work through this array
                const unsigned long long nz = __ballot(v != 0.0f && slot_k < 6);
                const unsigned long long group = (nz >> (lane & ~(kFlushLanes - 1))) & ((1ull << kFlushLanes) - 1ull);
                if (slot_k == 0 && group) touched[gid] = 1;
            }
        }
    }
}

static int check_feature_args(const char* who, const d3gs_params* p, int32_t num_features, const void* a, const void* b,
                              const void* c, const void* d, const void* e, const void* f) {
    int rc = check_params(p, who);
    if (rc) return rc;
    if (num_features < 0) { set_error("%s: num_features < 0", who); return D3GS_ERR_INVALID_ARGUMENT; }
    if (num_features > 0 && (!a || !b || !c || !d || !e || !f)) {
        set_error("%s: NULL buffer", who);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    return D3GS_OK;
}

}  // namespace d3gs

using namespace d3gs;

extern "C" int d3gs_blend_features_fwd(const d3gs_params* p, const int32_t* workload_ranges,
                                       const int32_t* gaussian_idx_sorted, const float* uvs, const float* conic_opacity,
                                       const float* features, int32_t num_features, const int32_t* tile_order,
                                       float* feature_image, d3gs_stream_t stream) {
    int rc = check_feature_args("d3gs_blend_features_fwd", p, num_features, workload_ranges, gaussian_idx_sorted, uvs,
                                conic_opacity, features, feature_image);
    if (rc) return rc;
    const int grid = p->tiles_x * p->tiles_y * batch_count(*p);
    if (grid == 0 || num_features == 0) return D3GS_OK;
    for (int c0 = 0; c0 < num_features;) {
        const int left = num_features - c0;
        if (left > 4) {
            const int w = left < 16 ? left : 16;
            hipLaunchKernelGGL(blend_features_fwd_kernel<16>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p,
                               workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, features, (int)num_features, c0, w,
                               tile_order, feature_image);
            c0 += w;
        } else {
            hipLaunchKernelGGL(blend_features_fwd_kernel<4>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p,
                               workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, features, (int)num_features, c0,
                               left, tile_order, feature_image);
            c0 += left;
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_blend_features_fwd: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_blend_features_bwd(const d3gs_params* p, const int32_t* workload_ranges,
                                       const int32_t* gaussian_idx_sorted, const float* uvs, const float* conic_opacity,
                                       const float* features, int32_t num_features, const int32_t* tile_order,
                                       const int32_t* n_contrib, const float* feature_image,
                                       const float* dfeature_image, float* grad_records, float* dfeatures,
                                       uint8_t* touched, d3gs_stream_t stream) {
    int rc = check_feature_args("d3gs_blend_features_bwd", p, num_features, workload_ranges, gaussian_idx_sorted, uvs,
                                conic_opacity, features, feature_image);
    if (rc) return rc;
    const int grid = p->tiles_x * p->tiles_y * batch_count(*p);
    if (grid == 0 || num_features == 0) return D3GS_OK;
    if (!n_contrib || !dfeature_image || !grad_records || !dfeatures) {
        set_error("d3gs_blend_features_bwd: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    for (int c0 = 0; c0 < num_features;) {
        const int left = num_features - c0;
        if (left > 4) {
            const int w = left < 14 ? left : 14;
            hipLaunchKernelGGL(blend_features_bwd_kernel<14>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p,
                               workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, features, (int)num_features, c0, w,
                               tile_order, n_contrib, feature_image, dfeature_image, grad_records, dfeatures, touched);
            c0 += w;
        } else {
            hipLaunchKernelGGL(blend_features_bwd_kernel<4>, dim3(grid), dim3(kBlock), 0, (hipStream_t)stream, *p,
                               workload_ranges, gaussian_idx_sorted, uvs, conic_opacity, features, (int)num_features, c0,
                               left, tile_order, n_contrib, feature_image, dfeature_image, grad_records, dfeatures, touched);
            c0 += left;
        }
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_blend_features_bwd: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}
