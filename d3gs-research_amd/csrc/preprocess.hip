// Per-gaussian kernels: preprocess forward (projection, EWA covariance, conic,
// radius, tile count), the SH colours, and preprocess backward (chain rule back to the
// raw model tensors).  One thread per gaussian; the SH rows (and, in the backward, the SH
// gradient rows of the gaussians that carry gradient) pass through LDS so that global
// traffic is coalesced.  All are single streaming passes over the model arrays.
//
// Reference: d3sim/algos/d3gs/render.py:421-476, 569-619 (forward) and
// 3217-3356 (backward); math in d3sim/csrc/gs3d.py and d3sim/csrc/camera.py.
#include "device_math.h"

namespace d3gs {

// SH -> RGB for one channel (gs3d.py:151-201); `rest` points at coefficient 1.
__device__ __forceinline__ float sh_channel(int degree, float x, float y, float z, float base, const float* rest, int ch) {
    float r = kShC0 * base;
    if (degree > 0) {
        r = ((r - (kShC1 * y) * rest[0 * 3 + ch]) + (kShC1 * z) * rest[1 * 3 + ch]) - (kShC1 * x) * rest[2 * 3 + ch];
        if (degree > 1) {
            float xx = x * x, yy = y * y, zz = z * z;
            float xy = x * y, yz = y * z, xz = x * z;
            r = r + (kShC2[0] * xy) * rest[3 * 3 + ch];
            r = r + (kShC2[1] * yz) * rest[4 * 3 + ch];
            r = r + (kShC2[2] * ((2.0f * zz - xx) - yy)) * rest[5 * 3 + ch];
            r = r + (kShC2[3] * xz) * rest[6 * 3 + ch];
            r = r + (kShC2[4] * (xx - yy)) * rest[7 * 3 + ch];
            if (degree > 2) {
                r = r + ((kShC3[0] * y) * (3.0f * xx - yy)) * rest[8 * 3 + ch];
                r = r + ((kShC3[1] * xy) * z) * rest[9 * 3 + ch];
                r = r + ((kShC3[2] * y) * ((4.0f * zz - xx) - yy)) * rest[10 * 3 + ch];
                r = r + ((kShC3[3] * z) * ((2.0f * zz - 3.0f * xx) - 3.0f * yy)) * rest[11 * 3 + ch];
                r = r + ((kShC3[4] * x) * ((4.0f * zz - xx) - yy)) * rest[12 * 3 + ch];
                r = r + ((kShC3[5] * z) * (xx - yy)) * rest[13 * 3 + ch];
                r = r + ((kShC3[6] * x) * (xx - 3.0f * yy)) * rest[14 * 3 + ch];
            }
        }
    }
    return r + 0.5f;
}

constexpr int kPrepBlock = 128;   // gaussians (= threads) per workgroup of the per-gaussian kernels
constexpr int kShColorBlocks = 384;   // fewest workgroups of the SH colour kernel: three on every two CUs

// Rows of `rowlen` floats per gaussian move from global memory into LDS with consecutive threads on
// consecutive addresses (the per-gaussian rows are 180-192 B apart, so per-thread access would touch a
// different cache line in every lane).  LDS rows are padded to an odd stride: conflict-free per-thread access.
// kAhead 16-byte loads of a thread are requested before the first is stored: one at a time, each waits for its own
// trip to memory, and a kernel that runs one wavefront per SIMD has nothing else to do meanwhile.
template <int kAhead>
__device__ __forceinline__ void rows_global_to_lds(const float* __restrict__ src, float* lds, int nrows, int rowlen,
                                                   int stride) {
    const int total = nrows * rowlen;
    const float inv = 1.0f / (float)rowlen;
    auto place = [&](int e, float v) {
        const int g = (int)(((float)e + 0.5f) * inv);
        lds[g * stride + (e - g * rowlen)] = v;
    };
    if ((((uintptr_t)src & 15u) == 0) && (total & 3) == 0) {
        for (int e0 = threadIdx.x * 4; e0 < total; e0 += kPrepBlock * 4 * kAhead) {
            float4 t[kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {      // (elements past the end read element 0 and store nothing)
                const int e4 = e0 + u * kPrepBlock * 4;
                t[u] = *reinterpret_cast<const float4*>(src + (e4 < total ? e4 : 0));
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int e4 = e0 + u * kPrepBlock * 4;
                if (e4 < total) {
                    place(e4, t[u].x); place(e4 + 1, t[u].y); place(e4 + 2, t[u].z); place(e4 + 3, t[u].w);
                }
            }
        }
    } else {
        for (int e = threadIdx.x; e < total; e += kPrepBlock) place(e, src[e]);
    }
}

// Per-gaussian camera for instance rendering (render.py:346-356): a gaussian with instance id k >= 0 lives in
// the frame of instance k and is seen by the camera expressed in that frame, cameras[k] = 9 floats of the
// world-to-camera rotation (row major) followed by the camera centre; the others keep the view's camera.
struct InstanceView {
    const int32_t* ids;     // [N], may be NULL
    const float* cameras;   // [count][12]; for a bundle of B cameras B such tables, camera by camera
    int count;
};

__device__ __forceinline__ void apply_instance(d3gs_params& P, const InstanceView& inst, int i, int batch = 0) {
    if (!inst.ids) return;
    const int id = inst.ids[i];
    if (id >= 0 && id < inst.count) {
        const float* m = inst.cameras + 12 * ((size_t)batch * inst.count + id);
#pragma unroll
        for (int k = 0; k < 9; ++k) P.w2c[k] = m[k];
#pragma unroll
        for (int k = 0; k < 3; ++k) P.cam_center[k] = m[9 + k];
    }
}

// Sparse mode (config sparse_mode; render.py:234-238, 478-500, 622-640): everything downstream of K1 works on the
// accepted render items only, stored compactly.  The reference counts them in a first launch of K1 and lets a
// second launch take slots from an atomic counter, in whatever order the hardware reaches it; here the first
// launch (valid_out) writes one flag per item, a scan of the flags gives every accepted item its slot in ascending
// item order (slot_scan, inclusive), and the second launch writes its outputs there, which keeps the render
// identical to the dense one bit for bit (ties in the sort go by slot, slots ascend with the item index).
struct SparseView {
    int32_t* valid_out;          // first launch: [items] 1 = accepted; nothing else is written
    const int32_t* slot_scan;    // second launch: [items] inclusive scan of the flags
    int32_t* gaussian_ids;       // second launch: [accepted] gaussian of each slot (sparse_gaussian_id)
    int32_t* batch_ids;          // second launch: [accepted] camera of each slot (sparse_batch_id)
};

// kWithSh = false leaves the SH colour to sh_colors_kernel: no LDS, twice the resident wavefronts.
template <bool kWithSh, bool kInstances, bool kSparse = false>
__global__ __launch_bounds__(kPrepBlock) void preprocess_fwd_kernel(
    const d3gs_params P0, const InstanceView inst, const SparseView sparse, const float* __restrict__ xyz,
    const float* __restrict__ quat,
    const float* __restrict__ scale, const float* __restrict__ opacity, const float* __restrict__ sh,
    const float* __restrict__ sh_base, const uint8_t* __restrict__ invalid_mask, float* __restrict__ depths,
    int32_t* __restrict__ radii, float* __restrict__ uvs, float* __restrict__ conic_opacity,
    int32_t* __restrict__ tiles_touched, float* __restrict__ rgb_out, float* __restrict__ cov2d_out,
    uint8_t* __restrict__ ne0_out, unsigned long long* __restrict__ tile_masks,
    uint32_t* __restrict__ depth_sort_keys) {
    // SH rows of this workgroup's gaussians: coalesced global read into LDS, then per-thread rows
    extern __shared__ float s_rows[];
    const int rowlen = P0.sh_stride * 3, stride = rowlen | 1;
    if constexpr (kWithSh) {
        const int first = blockIdx.x * kPrepBlock;
        rows_global_to_lds<4>(sh + (size_t)first * rowlen, s_rows, min(kPrepBlock, P0.n - first), rowlen, stride);
        __syncthreads();
    }
    // no early return: every lane of the wavefront takes part in the cooperative tile count
    const int i_raw = blockIdx.x * kPrepBlock + threadIdx.x;
    const int items = item_count(P0);
    const bool in_range = i_raw < items;
    const int i = in_range ? i_raw : items - 1;     // render item: outputs and the reject mask are indexed by it
    d3gs_params P = P0;     // with instances or a camera bundle: this lane's camera
    int g = i, batch = 0;   // gaussian (row of the model arrays) and camera of the item
    if constexpr (kInstances) {
        if (P0.batch_size > 1) {
            batch = i / P0.n;
            g = i - batch * P0.n;
            apply_batch_camera(P, batch);
        }
        if (inst.ids) apply_instance(P, inst, g, batch);
    }

    bool valid = true;
    float z = 0.0f, u = 0.0f, v = 0.0f, con0 = 0.0f, con1 = 0.0f, con2 = 0.0f, op = 0.0f;
    float a = 0.0f, b = 0.0f, c = 0.0f, radius = 0.0f;
    int count = 0;
    unsigned long long kept_mask = 0ull, kept_meta = 0ull;
    float rgb[3] = {0.0f, 0.0f, 0.0f};
    uint32_t ne0 = 0;

    float d[3] = {xyz[3 * g] - P.cam_center[0], xyz[3 * g + 1] - P.cam_center[1], xyz[3 * g + 2] - P.cam_center[2]};
    float pc[3] = {dot3(P.w2c + 0, d), dot3(P.w2c + 3, d), dot3(P.w2c + 6, d)};
    z = pc[2];
    valid = in_range && (z >= P.z_near && z <= P.z_far) && !(invalid_mask && invalid_mask[i]);
    if (valid) {
        u = ((pc[0] / z) * P.fx + P.cx) - 0.5f;
        v = ((pc[1] / z) * P.fy + P.cy) - 0.5f;

        const float4 qr = *reinterpret_cast<const float4*>(quat + 4 * g);
        float q[4] = {qr.x, qr.y, qr.z, qr.w};
        float s[3] = {scale[3 * g], scale[3 * g + 1], scale[3 * g + 2]};
        if (P.fused_activation) {
            float qn = sqrtf(((qr.x * qr.x + qr.y * qr.y) + qr.z * qr.z) + qr.w * qr.w);
            q[0] = qr.x / qn; q[1] = qr.y / qn; q[2] = qr.z / qn; q[3] = qr.w / qn;
            s[0] = det_expf(s[0]); s[1] = det_expf(s[1]); s[2] = det_expf(s[2]);
        }
        if (!P.training) {
            s[0] = s[0] * P.scale_global;
            s[1] = s[1] * P.scale_global;
            s[2] = s[2] * P.scale_global;
        }
        float R[9], c6[6];
        quat_to_rot(q, R);
        cov3d_from_scale_rot(s, R, c6);

        float t0[3], t1[3], tx, ty;
        ewa_rows(P, pc, t0, t1, tx, ty);
        float v0[3], v1[3];
        sym3_mv(c6, t0, v0);
        sym3_mv(c6, t1, v1);
        a = dot3(t0, v0) + P.lowpass;
        b = dot3(t0, v1);
        c = dot3(t1, v1) + P.lowpass;

        float det;
        op = P.fused_activation ? det_sigmoid(opacity[g]) : opacity[g];
        if (P.enable_anti_aliasing) {
            // gs3d.py:592-617: exact inverse of the low-passed covariance; the determinant handed on to
            // the radius and the det > 0 test is the one without the low-pass term (render.py:466-476);
            // opacity scaled by sqrt(max(0.000025, det / det_lowpass)) (render.py:393, 404-407)
            const float a0 = a - P.lowpass, c0 = c - P.lowpass;
            const float det_lp = a * c - b * b;
            det = a0 * c0 - b * b;
            const float inv = 1.0f / det_lp;
            con0 = c * inv;
            con1 = (-b) * inv;
            con2 = a * inv;
            op = op * sqrtf(fmaxf(0.000025f, det / det_lp));
        } else {
            det = a * c - b * b;
            const float det_inv = 1.0f / (det + P.eps);
            con0 = c * det_inv;
            con1 = (-b) * det_inv;
            con2 = a * det_inv;
        }

        float mid = 0.5f * (a + c);
        float sq = sqrtf(fmaxf(P.radii_eigen_eps, mid * mid - det));
        float l1 = mid + sq, l2 = mid - sq;
        radius = ceilf(P.std_sigma * sqrtf(fmaxf(l1, l2)));

        int rminx = tile_coord((u - radius) / 16.0f, P.tiles_x);
        int rminy = tile_coord((v - radius) / 16.0f, P.tiles_y);
        int rmaxx = tile_coord((((u + radius) + 16.0f) - 1.0f) / 16.0f, P.tiles_x);
        int rmaxy = tile_coord((((v + radius) + 16.0f) - 1.0f) / 16.0f, P.tiles_y);
        int area = (rmaxx - rminx) * (rmaxy - rminy);
        valid = (det > 0.0f) && area != 0 && (op > P.alpha_eps);
    }
    if constexpr (kSparse) {
        if (sparse.valid_out) {      // first launch: which items are accepted (wave-uniform branch)
            if (in_range) sparse.valid_out[i] = valid ? 1 : 0;
            return;
        }
    }
    {
        TileWalkIn g{u, v, radius, con0, con1, con2, op};
        TileWalk walk = {};
        if (valid) walk = tile_walk_setup(P, g);
        bool has_mask;
        count = wave_tile_count(P.filter_algo, valid, walk, kept_mask, has_mask);
        // the tile rows of camera b start at b * tiles_y: the record's origin carries the camera, so that key
        // expansion emits b * tiles + y * tiles_x + x (render.py:787, 809) without knowing about bundles
        walk.bminy += batch * P.tiles_y;
        kept_meta = tile_mask_meta(walk, has_mask);
    }
    if (valid && kWithSh) {
        float dn = sqrtf((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]);
        float dx = d[0] / dn, dy = d[1] / dn, dz = d[2] / dn;
        const float* shp = s_rows + threadIdx.x * stride;
        const float* base = P.has_sh_base ? sh_base + 3 * g : shp;     // (the fused colours run without a bundle: g = i)
        const float* rest = P.has_sh_base ? shp : shp + 3;
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) rgb[ch] = sh_channel(P.sh_degree, dx, dy, dz, base[ch], rest, ch);
        ne0 = ((rgb[0] < 0.0f) << 2) | ((rgb[1] < 0.0f) << 1) | (rgb[2] < 0.0f);
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) rgb[ch] = fmaxf(rgb[ch], 0.0f);
    }
    if (!valid) z = u = v = con0 = con1 = con2 = op = a = b = c = radius = 0.0f;
    if (!in_range) return;
    int out_i = i;          // row of the outputs
    if constexpr (kSparse) {
        if (!valid) return;     // rejected items have no slot
        out_i = sparse.slot_scan[i] - 1;
        sparse.gaussian_ids[out_i] = g;
        sparse.batch_ids[out_i] = batch;
    }
    {
    const int i = out_i;
    // render.py:582: the depth, or its inverse (a rejected gaussian's stays 0)
    const float stored = (P.render_inv_depth && valid) ? 1.0f / z : z;
    depths[i] = stored;
    if (depth_sort_keys) depth_sort_keys[i] = depth_sort_key(P, stored);
    radii[i] = (int)radius;
    *reinterpret_cast<float2*>(uvs + 2 * i) = make_float2(u, v);
    *reinterpret_cast<float4*>(conic_opacity + 4 * i) = make_float4(con0, con1, con2, op);
    tiles_touched[i] = count;
    if (tile_masks) {
        tile_masks[2 * (size_t)i] = kept_mask;
        tile_masks[2 * (size_t)i + 1] = kept_meta;
    }
    if (cov2d_out) {
        cov2d_out[3 * i + 0] = a;
        cov2d_out[3 * i + 1] = b;
        cov2d_out[3 * i + 2] = c;
    }
    if constexpr (kWithSh) {
        rgb_out[3 * i + 0] = rgb[0];
        rgb_out[3 * i + 1] = rgb[1];
        rgb_out[3 * i + 2] = rgb[2];
        if (ne0_out) ne0_out[i] = (uint8_t)ne0;
    }
    }
}

// SH colours of sparse mode's compact items: slot s holds gaussian ids[s] seen by camera batch_ids[s].  One
// thread per slot reads its gaussian's SH row from global memory (the rows of consecutive slots are not
// neighbours, so there is nothing to stage); same operations as sh_colors_kernel.
__global__ __launch_bounds__(kPrepBlock) void sh_colors_sparse_kernel(
    const d3gs_params P0, const int32_t* __restrict__ ids, const int32_t* __restrict__ batch_ids, const int count,
    const InstanceView inst, const float* __restrict__ xyz, const float* __restrict__ sh,
    const float* __restrict__ sh_base, const int32_t* __restrict__ radii, float* __restrict__ rgb_out,
    uint8_t* __restrict__ ne0_out) {
    const int slot = blockIdx.x * kPrepBlock + threadIdx.x;
    if (slot >= count) return;
    const int g = ids[slot];
    d3gs_params P = P0;
    if (P0.batch_size > 1) apply_batch_camera(P, batch_ids[slot]);
    if (inst.ids && (unsigned)g < (unsigned)P0.n) apply_instance(P, inst, g, P0.batch_size > 1 ? batch_ids[slot] : 0);
    float rgb[3] = {0.0f, 0.0f, 0.0f};
    uint32_t ne0 = 0;
    if (radii[slot] > 0 && (unsigned)g < (unsigned)P0.n) {
        float d[3] = {xyz[3 * g] - P.cam_center[0], xyz[3 * g + 1] - P.cam_center[1], xyz[3 * g + 2] - P.cam_center[2]};
        float dn = sqrtf((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]);
        float dx = d[0] / dn, dy = d[1] / dn, dz = d[2] / dn;
        const float* shp = sh + (size_t)g * P.sh_stride * 3;
        const float* base = P.has_sh_base ? sh_base + 3 * g : shp;
        const float* rest = P.has_sh_base ? shp : shp + 3;
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) rgb[ch] = sh_channel(P.sh_degree, dx, dy, dz, base[ch], rest, ch);
        ne0 = ((rgb[0] < 0.0f) << 2) | ((rgb[1] < 0.0f) << 1) | (rgb[2] < 0.0f);
#pragma unroll
        for (int ch = 0; ch < 3; ++ch) rgb[ch] = fmaxf(rgb[ch], 0.0f);
    }
    rgb_out[3 * slot + 0] = rgb[0];
    rgb_out[3 * slot + 1] = rgb[1];
    rgb_out[3 * slot + 2] = rgb[2];
    if (ne0_out) ne0_out[slot] = (uint8_t)ne0;
}

// SH colour of the gaussians the preprocess kernel accepted (radii > 0), the part of K1 that
// streams the 192-byte SH rows: same operations as the fused kernel, zeros for rejected gaussians.
template <bool kInstances>
__global__ __launch_bounds__(kPrepBlock) void sh_colors_kernel(
    const d3gs_params P0, const InstanceView inst, const float* __restrict__ xyz, const float* __restrict__ sh,
    const float* __restrict__ sh_base, const int32_t* __restrict__ radii, float* __restrict__ rgb_out,
    uint8_t* __restrict__ ne0_out) {
    extern __shared__ float s_rows[];
    const int rowlen = P0.sh_stride * 3, stride = rowlen | 1;
    // grid-stride over 128-gaussian chunks: a small grid leaves most of every CU to the kernels this
    // one runs beside
    // (with a camera bundle: the chunks of camera 0, then those of camera 1, ...; a chunk never spans two cameras)
    const int chunks_per_view = (P0.n + kPrepBlock - 1) / kPrepBlock;
    for (int chunk = blockIdx.x; chunk < chunks_per_view * batch_count(P0); chunk += gridDim.x) {
        const int batch = chunk / chunks_per_view;
        const int first = (chunk - batch * chunks_per_view) * kPrepBlock;      // first gaussian of the chunk
        __syncthreads();   // the previous chunk's rows have been read
        // what the thread's own gaussian needs besides its row, requested ahead of the rows (lanes past the end
        // read the chunk's first gaussian)
        const int g = first + threadIdx.x;
        const int g_safe = g < P0.n ? g : first;
        const int radius = radii[batch * P0.n + g_safe];
        const float centre[3] = {xyz[3 * g_safe], xyz[3 * g_safe + 1], xyz[3 * g_safe + 2]};
        rows_global_to_lds<12>(sh + (size_t)first * rowlen, s_rows, min(kPrepBlock, P0.n - first), rowlen, stride);
        __syncthreads();
        if (g >= P0.n) continue;
        const int i = batch * P0.n + g;     // render item
        d3gs_params P = P0;
        if constexpr (kInstances) {
            if (P0.batch_size > 1) apply_batch_camera(P, batch);
            if (inst.ids) apply_instance(P, inst, g, batch);
        }
        float rgb[3] = {0.0f, 0.0f, 0.0f};
        uint32_t ne0 = 0;
        if (radius > 0) {
            float d[3] = {centre[0] - P.cam_center[0], centre[1] - P.cam_center[1], centre[2] - P.cam_center[2]};
            float dn = sqrtf((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]);
            float dx = d[0] / dn, dy = d[1] / dn, dz = d[2] / dn;
            const float* shp = s_rows + threadIdx.x * stride;
            const float* base = P.has_sh_base ? sh_base + 3 * g : shp;
            const float* rest = P.has_sh_base ? shp : shp + 3;
#pragma unroll
            for (int ch = 0; ch < 3; ++ch) rgb[ch] = sh_channel(P.sh_degree, dx, dy, dz, base[ch], rest, ch);
            ne0 = ((rgb[0] < 0.0f) << 2) | ((rgb[1] < 0.0f) << 1) | (rgb[2] < 0.0f);
#pragma unroll
            for (int ch = 0; ch < 3; ++ch) rgb[ch] = fmaxf(rgb[ch], 0.0f);
        }
        rgb_out[3 * i + 0] = rgb[0];
        rgb_out[3 * i + 1] = rgb[1];
        rgb_out[3 * i + 2] = rgb[2];
        if (ne0_out) ne0_out[i] = (uint8_t)ne0;
    }
}

// ---------------------------------------------------------------------------
// Preprocess backward.
// ---------------------------------------------------------------------------
// What the backward of one gaussian reads besides its SH row: loaded ahead of the rows' way through LDS, so that
// these scattered reads and the row copy are in flight together.
struct BwdInputs {
    float xyz[3], s[3], cov[3], opacity;
    float4 q, ra, rb, rc;      // quaternion; the blend backward's record: duv(2) dconic(3) dopacity dcolor(3) dz
    uint32_t ne0;
};
// i: row of the per-item arrays (cov2d, ne0, records); m: row of the model arrays (the same unless sparse)
__device__ __forceinline__ BwdInputs load_bwd_inputs(const int i, const int m, const float* __restrict__ xyz,
                                                     const float* __restrict__ quat, const float* __restrict__ scale,
                                                     const float* __restrict__ opacity, const float* __restrict__ cov2d,
                                                     const uint8_t* __restrict__ ne0, const float4* __restrict__ rec4) {
    BwdInputs in;
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        in.xyz[k] = xyz[3 * m + k];
        in.s[k] = scale[3 * m + k];
        in.cov[k] = cov2d[3 * i + k];
    }
    in.opacity = opacity[m];
    in.q = *reinterpret_cast<const float4*>(quat + 4 * m);
    in.ra = rec4[4 * (size_t)i];
    in.rb = rec4[4 * (size_t)i + 1];
    in.rc = rec4[4 * (size_t)i + 2];
    in.ne0 = ne0[i];
    return in;
}

// One gaussian of the preprocess backward.  `shrow` is this gaussian's SH row staged in LDS: it holds
// the coefficients on entry and receives their gradients (each channel's coefficients are read into
// registers before that channel's gradients overwrite them).
__device__ __forceinline__ void preprocess_bwd_one(
    const d3gs_params& P, const int i, const BwdInputs& in, const int sh_mask_compat, const bool accumulate,
    float* __restrict__ dxyz, float* __restrict__ dquat, float* __restrict__ dscale, float* dopacity_out,
    float* shrow, float* __restrict__ dsh_base) {
    // accumulate: the gradient arrays already hold the sum over the cameras before this one (camera bundles)
    auto put = [accumulate](float* dst, float v) { *dst = accumulate ? *dst + v : v; };
    const float4 ra = in.ra, rb = in.rb, rc = in.rc;
    const int K = P.sh_stride;

    const float* W = P.w2c;
    float d[3] = {in.xyz[0] - P.cam_center[0], in.xyz[1] - P.cam_center[1], in.xyz[2] - P.cam_center[2]};
    float pc[3] = {dot3(W + 0, d), dot3(W + 3, d), dot3(W + 6, d)};
    float z = pc[2];
    // pinhole backward (camera.py:357-369)
    float gu = ra.x * P.fx, gv = ra.y * P.fy;
    float zi = 1.0f / z, zi2 = 1.0f / (z * z);
    float dzin = P.render_depth ? rc.y : 0.0f;
    if (P.render_inv_depth) dzin = (-dzin) / (z * z);      // the record holds dL/d(1/z) (render.py:1965, 3051, 3283)
    float dpc[3] = {gu * zi, gv * zi, (dzin + ((-gu) * pc[0]) * zi2) + ((-gv) * pc[1]) * zi2};

    // conic -> cov2d backward (gs3d.py:571-586)
    float a = in.cov[0], b = in.cov[1], c = in.cov[2];
    float g0 = ra.z, g1 = ra.w, g2 = rb.x;
    float det = a * c - b * b;
    float k2 = 1.0f / (det * det + 1e-8f);
    float da = k2 * ((((-c) * c) * g0 + (b * c) * g1) + (det - a * c) * g2);
    float db = (k2 * 2.0f) * (((b * c) * g0 - (det / 2.0f + b * b) * g1) + (a * b) * g2);
    float dc = k2 * ((((-a) * a) * g2 + (a * b) * g1) + (det - a * c) * g0);
    float dop_in = rb.y;
    if (P.enable_anti_aliasing) {
        // render.py:3293-3306; gs3d.py:671-679: dop_in is the gradient of opacity * comp with
        // comp = sqrt(max(0.000025, ratio)), ratio = det_without_lowpass / det
        const float lf = P.lowpass;
        const float a0 = a - lf, c0 = c - lf;
        const float ratio = (a0 * c0 - b * b) / det;
        const float comp = sqrtf(fmaxf(0.000025f, ratio));
        const float op_act = P.fused_activation ? det_sigmoid(in.opacity) : in.opacity;
        const float dcomp = dop_in * op_act;
        const float dratio = ratio <= 0.000025f ? 0.0f : (dcomp * 0.5f) / comp;
        const float gm = dratio * k2;
        da += (lf * ((c * c + b * b) - c * lf)) * gm;
        db += ((-2.0f * b) * lf) * ((a + c) - lf) * gm;
        dc += (lf * ((a * a + b * b) - a * lf)) * gm;
        dop_in = dop_in * comp;
    }

    const float4 qr = in.q;
    float qn = 1.0f;
    float q[4] = {qr.x, qr.y, qr.z, qr.w};
    float s[3] = {in.s[0], in.s[1], in.s[2]};
    if (P.fused_activation) {
        qn = sqrtf(((qr.x * qr.x + qr.y * qr.y) + qr.z * qr.z) + qr.w * qr.w);
        q[0] = qr.x / qn; q[1] = qr.y / qn; q[2] = qr.z / qn; q[3] = qr.w / qn;
        s[0] = det_expf(s[0]); s[1] = det_expf(s[1]); s[2] = det_expf(s[2]);
    }
    float R[9], c6[6];
    quat_to_rot(q, R);
    cov3d_from_scale_rot(s, R, c6);

    // EWA backward (gs3d.py:490-530): cov2d = T Sigma3 T^T with T = J W
    float t0[3], t1[3], tx, ty;
    ewa_rows(P, pc, t0, t1, tx, ty);
    float limx = fabsf((P.tan_fovx * P.clamp_factor) * z), limy = fabsf((P.tan_fovy * P.clamp_factor) * z);
    float mx = (pc[0] < -limx || pc[0] > limx) ? 0.0f : 1.0f;
    float my = (pc[1] < -limy || pc[1] > limy) ? 0.0f : 1.0f;
    float G00 = da, G01 = 0.5f * db, G11 = dc;
    float u0[3], u1[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        u0[k] = G00 * t0[k] + G01 * t1[k];
        u1[k] = G01 * t0[k] + G11 * t1[k];
    }
    float dS[9];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int k = 0; k < 3; ++k) dS[r * 3 + k] = t0[r] * u0[k] + t1[r] * u1[k];
    float dT0[3], dT1[3];
    sym3_mv(c6, u0, dT0);
    sym3_mv(c6, u1, dT1);
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        dT0[k] = 2.0f * dT0[k];
        dT1[k] = 2.0f * dT1[k];
    }
    float dJ00 = dot3(dT0, W + 0), dJ02 = dot3(dT0, W + 6);
    float dJ11 = dot3(dT1, W + 3), dJ12 = dot3(dT1, W + 6);
    float zz = z * z;
    float zzi = 1.0f / zz;
    float z3 = (z * z) * z;
    float txf = tx * P.fx, tyf = ty * P.fy;
    float dmean[3];
    dmean[0] = ((mx * (-dJ02)) * P.fx) * zzi;
    dmean[1] = ((my * (-dJ12)) * P.fy) * zzi;
    dmean[2] = (-(P.fx * dJ00 + P.fy * dJ11)) * zzi + (2.0f * (dJ02 * txf + dJ12 * tyf)) / z3;
    float tot[3] = {dpc[0] + dmean[0], dpc[1] + dmean[1], dpc[2] + dmean[2]};
    float gx[3];
#pragma unroll
    for (int k = 0; k < 3; ++k) gx[k] = (W[0 + k] * tot[0] + W[3 + k] * tot[1]) + W[6 + k] * tot[2];

    // cov3d backward (gs3d.py:400-416)
    float M[9];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int k = 0; k < 3; ++k) M[r * 3 + k] = R[r * 3 + k] * s[k];
    float dM[9];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int k = 0; k < 3; ++k)
            dM[r * 3 + k] = 2.0f * ((dS[r * 3 + 0] * M[0 + k] + dS[r * 3 + 1] * M[3 + k]) + dS[r * 3 + 2] * M[6 + k]);
    float ds[3], dR[9];
#pragma unroll
    for (int k = 0; k < 3; ++k) ds[k] = (dM[0 + k] * R[0 + k] + dM[3 + k] * R[3 + k]) + dM[6 + k] * R[6 + k];
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
        for (int k = 0; k < 3; ++k) dR[r * 3 + k] = dM[r * 3 + k] * s[k];
    float qx = q[0], qy = q[1], qz = q[2], qw = q[3];
    float dq[4];
    dq[0] = 2.0f * (((qy * (dR[1] + dR[3]) + qz * (dR[2] + dR[6])) - (2.0f * qx) * (dR[4] + dR[8])) + qw * (dR[7] - dR[5]));
    dq[1] = 2.0f * (((qx * (dR[1] + dR[3]) - (2.0f * qy) * (dR[0] + dR[8])) + qz * (dR[5] + dR[7])) + qw * (dR[2] - dR[6]));
    dq[2] = 2.0f * (((qx * (dR[2] + dR[6]) + qy * (dR[5] + dR[7])) - (2.0f * qz) * (dR[0] + dR[4])) + qw * (dR[3] - dR[1]));
    dq[3] = 2.0f * ((qz * (dR[3] - dR[1]) + qy * (dR[2] - dR[6])) + qx * (dR[7] - dR[5]));
    // activation backward: exp, normalize, sigmoid (origin/model.py:332-383)
    float4 gq;
    if (P.fused_activation) {
        put(dscale + 3 * i + 0, ds[0] * s[0]);
        put(dscale + 3 * i + 1, ds[1] * s[1]);
        put(dscale + 3 * i + 2, ds[2] * s[2]);
        float qd = ((q[0] * dq[0] + q[1] * dq[1]) + q[2] * dq[2]) + q[3] * dq[3];
        gq = make_float4((dq[0] - q[0] * qd) / qn, (dq[1] - q[1] * qd) / qn, (dq[2] - q[2] * qd) / qn,
                         (dq[3] - q[3] * qd) / qn);
        float o = det_sigmoid(in.opacity);
        put(dopacity_out + i, dop_in * (o * (1.0f - o)));
    } else {
        // inputs were activated by the caller: gradients w.r.t. the activated values
        put(dscale + 3 * i + 0, ds[0]);
        put(dscale + 3 * i + 1, ds[1]);
        put(dscale + 3 * i + 2, ds[2]);
        gq = make_float4(dq[0], dq[1], dq[2], dq[3]);
        put(dopacity_out + i, dop_in);
    }
    if (accumulate) {
        const float4 old = *reinterpret_cast<const float4*>(dquat + 4 * i);
        gq = make_float4(old.x + gq.x, old.y + gq.y, old.z + gq.z, old.w + gq.w);
    }
    *reinterpret_cast<float4*>(dquat + 4 * i) = gq;

    // SH backward (gs3d.py:262-364)
    float dn = sqrtf((d[0] * d[0] + d[1] * d[1]) + d[2] * d[2]);
    float x = d[0] / dn, y = d[1] / dn, zd = d[2] / dn;
    uint32_t m = in.ne0;
    float cg[3];
    if (sh_mask_compat) {
        cg[0] = rb.z * ((m & 1) ? 0.0f : 1.0f);
        cg[1] = rb.w * ((m & 2) ? 0.0f : 1.0f);
        cg[2] = rc.x * ((m & 4) ? 0.0f : 1.0f);
    } else {
        cg[0] = rb.z * ((m & 4) ? 0.0f : 1.0f);
        cg[1] = rb.w * ((m & 2) ? 0.0f : 1.0f);
        cg[2] = rc.x * ((m & 1) ? 0.0f : 1.0f);
    }
    const float* rest = P.has_sh_base ? shrow : shrow + 3;
    float* drest = P.has_sh_base ? shrow : shrow + 3;
    float* dbase = P.has_sh_base ? dsh_base + 3 * i : shrow;
    const int deg = P.sh_degree;
    // coefficients above the evaluated degree receive zero gradient
    const int used = (deg + 1) * (deg + 1) - 1;
    for (int k = used; k < K - (P.has_sh_base ? 0 : 1); ++k) {
        drest[k * 3 + 0] = 0.0f;
        drest[k * 3 + 1] = 0.0f;
        drest[k * 3 + 2] = 0.0f;
    }
    float ddir[3] = {0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ch = 0; ch < 3; ++ch) {
        float gch = cg[ch];
        float sv[15];
#pragma unroll
        for (int k = 0; k < 15; ++k) sv[k] = k < used ? rest[k * 3 + ch] : 0.0f;
        if (P.has_sh_base) put(dbase + ch, kShC0 * gch);   // global array; without a split base the row in LDS
        else dbase[ch] = kShC0 * gch;
        float dx_ = 0.0f, dy_ = 0.0f, dz_ = 0.0f;
        if (deg > 0) {
            drest[0 * 3 + ch] = (-kShC1 * y) * gch;
            drest[1 * 3 + ch] = (kShC1 * zd) * gch;
            drest[2 * 3 + ch] = (-kShC1 * x) * gch;
            dx_ = -kShC1 * sv[2];
            dy_ = -kShC1 * sv[0];
            dz_ = kShC1 * sv[1];
            if (deg > 1) {
                float xx = x * x, yy = y * y, zz2 = zd * zd, xy = x * y, yz = y * zd, xz = x * zd;
                drest[3 * 3 + ch] = (kShC2[0] * xy) * gch;
                drest[4 * 3 + ch] = (kShC2[1] * yz) * gch;
                drest[5 * 3 + ch] = (kShC2[2] * ((2.0f * zz2 - xx) - yy)) * gch;
                drest[6 * 3 + ch] = (kShC2[3] * xz) * gch;
                drest[7 * 3 + ch] = (kShC2[4] * (xx - yy)) * gch;
                float s3 = sv[3], s4 = sv[4], s5 = sv[5], s6 = sv[6],
                      s7 = sv[7];
                dx_ += kShC2[0] * y * s3 + kShC2[2] * 2.0f * (-x) * s5 + kShC2[3] * zd * s6 + kShC2[4] * 2.0f * x * s7;
                dy_ += kShC2[0] * x * s3 + kShC2[1] * zd * s4 + kShC2[2] * 2.0f * (-y) * s5 + kShC2[4] * 2.0f * (-y) * s7;
                dz_ += kShC2[1] * y * s4 + kShC2[2] * 2.0f * 2.0f * zd * s5 + kShC2[3] * x * s6;
                if (deg > 2) {
                    drest[8 * 3 + ch] = ((kShC3[0] * y) * (3.0f * xx - yy)) * gch;
                    drest[9 * 3 + ch] = ((kShC3[1] * xy) * zd) * gch;
                    drest[10 * 3 + ch] = ((kShC3[2] * y) * ((4.0f * zz2 - xx) - yy)) * gch;
                    drest[11 * 3 + ch] = ((kShC3[3] * zd) * ((2.0f * zz2 - 3.0f * xx) - 3.0f * yy)) * gch;
                    drest[12 * 3 + ch] = ((kShC3[4] * x) * ((4.0f * zz2 - xx) - yy)) * gch;
                    drest[13 * 3 + ch] = ((kShC3[5] * zd) * (xx - yy)) * gch;
                    drest[14 * 3 + ch] = ((kShC3[6] * x) * (xx - 3.0f * yy)) * gch;
                    float s8 = sv[8], s9 = sv[9], s10 = sv[10],
                          s11 = sv[11], s12 = sv[12], s13 = sv[13],
                          s14 = sv[14];
                    dx_ += kShC3[0] * s8 * 3.0f * 2.0f * xy + kShC3[1] * s9 * yz + kShC3[2] * s10 * (-2.0f) * xy +
                           kShC3[3] * s11 * (-3.0f) * 2.0f * xz + kShC3[4] * s12 * ((-3.0f) * xx + 4.0f * zz2 - yy) +
                           kShC3[5] * s13 * 2.0f * xz + kShC3[6] * s14 * 3.0f * (xx - yy);
                    dy_ += kShC3[0] * s8 * 3.0f * (xx - yy) + kShC3[1] * s9 * xz +
                           kShC3[2] * s10 * ((-3.0f) * yy + 4.0f * zz2 - xx) + kShC3[3] * s11 * (-3.0f) * 2.0f * yz +
                           kShC3[4] * s12 * (-2.0f) * xy + kShC3[5] * s13 * (-2.0f) * yz +
                           kShC3[6] * s14 * (-3.0f) * 2.0f * xy;
                    dz_ += kShC3[1] * s9 * xy + kShC3[2] * s10 * 4.0f * 2.0f * yz +
                           kShC3[3] * s11 * 3.0f * ((2.0f * zz2 - xx) - yy) + kShC3[4] * s12 * 4.0f * 2.0f * xz +
                           kShC3[5] * s13 * (xx - yy);
                }
            }
        }
        ddir[0] += dx_ * gch;
        ddir[1] += dy_ * gch;
        ddir[2] += dz_ * gch;
    }
    float dirv[3] = {x, y, zd};
    float dd = (dirv[0] * ddir[0] + dirv[1] * ddir[1]) + dirv[2] * ddir[2];
    put(dxyz + 3 * i + 0, gx[0] + (ddir[0] - dirv[0] * dd) / dn);
    put(dxyz + 3 * i + 1, gx[1] + (ddir[1] - dirv[1] * dd) / dn);
    put(dxyz + 3 * i + 2, gx[2] + (ddir[2] - dirv[2] * dd) / dn);
}

// A gaussian whose record is all zero -- culled in the forward pass, or in tile lists but never reached before
// its pixels saturated, which is most of a dense scene -- has an all-zero gradient: nothing of it is read beyond
// the record, and with outputs_are_zero (the caller cleared the gradient arrays beforehand) nothing is written.
// The others are compacted inside the workgroup (kPer gaussians per thread, so that what is left still fills
// whole wavefronts) and worked off kBwdBlock at a time: thread t takes the t-th of them, their SH rows are
// staged in LDS and leave as gradient rows.
constexpr int kBwdBlock = 256;
// Gaussians worked off per pass: as many LDS rows as leave room for four workgroups on a CU (160 KB of LDS, and the
// kernel's registers allow four as well), at most one per thread: 192 rows of 48 coefficients, 209 of 45 (split
// DC term).  A workgroup of a dense view holds about 170 gaussians with gradient; those beyond the rows of a
// pass cost a second, nearly empty one (176 -> 192 rows: -2 us; keeping the DC term out of LDS to reach 209: no
// further gain).
constexpr int kBwdLdsBudget = 160 * 1024 / 4;
constexpr int kBwdStaticLds = 3328;     // s_list, s_active, s_count, with some slack
static inline int bwd_rows_per_pass(int sh_stride) {
    const int row_bytes = ((sh_stride * 3) | 1) * (int)sizeof(float);
    const int rows = (kBwdLdsBudget - kBwdStaticLds) / row_bytes;
    return rows < kBwdBlock ? rows : kBwdBlock;
}

// element e of a block of `cnt` staged rows <-> element of the global [N][rowlen] array, for the gaussians
// first + list[0 .. cnt)
template <bool kToLds>
__device__ __forceinline__ void bwd_rows_copy(float* __restrict__ global, float* lds, const unsigned short* list, int cnt,
                                              int first, int rowlen, int stride, bool accumulate = false,
                                              const int32_t* __restrict__ origin = nullptr) {
    // origin (sparse mode, reads of the model's rows): row first + list[r] of the items is row origin[..] of `global`
    auto row_of = [&](int r) { const int i = first + list[r]; return (size_t)(origin ? origin[i] : i); };
    if ((rowlen & 3) == 0 && ((uintptr_t)global & 15u) == 0) {
        const int per_row = rowlen >> 2;
        if constexpr (kToLds) {
            // Rows in: four 16-byte loads of a thread are requested before the first is stored to LDS.  One at a
            // time, each would wait for its own trip to memory (the row's position comes out of LDS, and the
            // compiler does not move that read ahead of the stores before it).  Elements past the end read
            // element 0 and store nothing.
            constexpr int kAhead = 4;
            const int total = cnt * per_row;
            for (int q0 = threadIdx.x; q0 < total; q0 += kBwdBlock * kAhead) {
                float4 t[kAhead];
                int at[kAhead], col[kAhead];
                size_t row[kAhead];
#pragma unroll
                for (int u = 0; u < kAhead; ++u) {
                    const int q = q0 + u * kBwdBlock;
                    const int qq = q < total ? q : 0;
                    const int r = qq / per_row;
                    col[u] = (qq - r * per_row) * 4;
                    at[u] = q < total ? r * stride + col[u] : -1;
                    row[u] = (size_t)(first + list[r]);
                }
                if (origin) {
#pragma unroll
                    for (int u = 0; u < kAhead; ++u) row[u] = (size_t)origin[row[u]];
                }
#pragma unroll
                for (int u = 0; u < kAhead; ++u)
                    t[u] = *reinterpret_cast<const float4*>(global + row[u] * rowlen + col[u]);
#pragma unroll
                for (int u = 0; u < kAhead; ++u) {
                    if (at[u] >= 0) {
                        float* lp = lds + at[u];
                        lp[0] = t[u].x; lp[1] = t[u].y; lp[2] = t[u].z; lp[3] = t[u].w;
                    }
                }
            }
            return;
        }
        for (int q = threadIdx.x; q < cnt * per_row; q += kBwdBlock) {
            const int r = q / per_row, c = (q - r * per_row) * 4;
            float4* gp = reinterpret_cast<float4*>(global + row_of(r) * rowlen + c);
            float* lp = lds + r * stride + c;
            if (kToLds) {
                const float4 t = *gp;
                lp[0] = t.x; lp[1] = t.y; lp[2] = t.z; lp[3] = t.w;
            } else if (accumulate) {
                const float4 t = *gp;
                *gp = make_float4(t.x + lp[0], t.y + lp[1], t.z + lp[2], t.w + lp[3]);
            } else {
                *gp = make_float4(lp[0], lp[1], lp[2], lp[3]);
            }
        }
    } else {
        for (int e = threadIdx.x; e < cnt * rowlen; e += kBwdBlock) {
            const int r = e / rowlen, c = e - r * rowlen;
            float* gp = global + row_of(r) * rowlen + c;
            if (kToLds) lds[r * stride + c] = *gp;
            else *gp = accumulate ? *gp + lds[r * stride + c] : lds[r * stride + c];
        }
    }
}

__device__ __forceinline__ bool record_is_zero(const float4 ra, const float4 rb, const float4 rc) {
    return ra.x == 0.0f && ra.y == 0.0f && ra.z == 0.0f && ra.w == 0.0f && rb.x == 0.0f && rb.y == 0.0f &&
           rb.z == 0.0f && rb.w == 0.0f && rc.x == 0.0f && rc.y == 0.0f;
}

template <int kPer, bool kInstances, bool kMany>
__global__ __launch_bounds__(kBwdBlock) void preprocess_bwd_kernel(
    const d3gs_params P_in, const int batch_index, const int batch_last, const int accumulate_in, const InstanceView inst,
    const float* __restrict__ xyz, const float* __restrict__ quat,
    const float* __restrict__ scale, const float* __restrict__ opacity, const float* __restrict__ sh,
    const int32_t* __restrict__ radii_in, const float* __restrict__ cov2d_in, const uint8_t* __restrict__ ne0_in,
    const float* __restrict__ grad_records, const uint8_t* __restrict__ touched_in, const int sh_mask_compat,
    const int outputs_are_zero, const int rows_per_pass, const int32_t* __restrict__ origin,
    const int32_t* __restrict__ row_batch_ids, float* __restrict__ dxyz, float* __restrict__ dquat,
    float* __restrict__ dscale, float* dopacity_out, float* __restrict__ dsh, float* __restrict__ dsh_base) {
    constexpr int kSpan = kBwdBlock * kPer, kWaves = kBwdBlock / 64;
    // Cameras batch_index .. batch_last of a bundle, one after the other (render.py:2972-2989, 3180-3219 loop over
    // the batch inside the kernel too): the per-item arrays come in pointing at camera batch_index's rows, camera c's
    // follow (c - batch_index) * n rows further on, its parameters come from the table, and from the second camera
    // on the gradients are added to what the workgroup itself stored for the cameras before.  Sparse mode's compact
    // rows of a bundle name their camera row by row (row_batch_ids) instead and go through once.
    extern __shared__ float s_rows[];                    // rows_per_pass rows of `stride` floats
    __shared__ unsigned short s_list[kSpan];             // gaussians (offsets from `first`) with work
    __shared__ unsigned char s_active[kSpan];
    __shared__ int s_count[kPer * kWaves];
    const int rowlen = P_in.sh_stride * 3, stride = rowlen | 1;
    const int first = blockIdx.x * kSpan;
    const int nrows = min(kSpan, P_in.n - first);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    // (kMany = false: the one camera batch_index, straight-line code, the kernel's parameters stay where the
    // compiler keeps kernel arguments)
    auto one_camera = [&](const int cam) {
    d3gs_params P = P_in;
    if (P_in.batch_size > 1 && !row_batch_ids) apply_batch_camera(P, cam);
    const size_t item0 = (size_t)(cam - batch_index) * (size_t)P_in.n;     // this camera's rows of the per-item arrays
    const int32_t* radii = radii_in + item0;
    const uint8_t* touched = touched_in ? touched_in + item0 : nullptr;
    const float* cov2d = cov2d_in + 3 * item0;
    const uint8_t* ne0 = ne0_in + item0;
    const float4* rec4 = reinterpret_cast<const float4*>(grad_records) + 4 * item0;
    const int accumulate = accumulate_in || cam > batch_index;
    bool active[kPer];
    unsigned long long mates[kPer];
    // all radii first, then all records: two round trips to memory instead of two per gaussian.  With the blend
    // backward's `touched` bytes a gaussian it did not mark counts as culled, and its record is never read.
    // (Every load below is unconditional: one behind a per-lane condition is issued and waited for on its own, one
    // after the other.  Lanes past the end read the block's last gaussian, gaussians without a mark the block's
    // first record, and what they read is dropped.)
    int rad[kPer];
    unsigned char mark[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        rad[k] = radii[(size_t)first + min(k * kBwdBlock + tid, nrows - 1)];
        mark[k] = 1;
    }
    if (touched) {
#pragma unroll
        for (int k = 0; k < kPer; ++k) mark[k] = touched[(size_t)first + min(k * kBwdBlock + tid, nrows - 1)];
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k)
        if (k * kBwdBlock + tid >= nrows || !mark[k]) rad[k] = 0;
    float4 ra[kPer], rb[kPer], rc[kPer];
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const size_t i = rad[k] != 0 ? (size_t)first + k * kBwdBlock + tid : (size_t)first;
        ra[k] = rec4[4 * i];
        rb[k] = rec4[4 * i + 1];
        rc[k] = rec4[4 * i + 2];
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k)
        if (rad[k] == 0) ra[k] = rb[k] = rc[k] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
    for (int k = 0; k < kPer; ++k) {
        const int local = k * kBwdBlock + tid;
        active[k] = rad[k] != 0 && !record_is_zero(ra[k], rb[k], rc[k]);
        mates[k] = __ballot(active[k]);
        if (lane == 0) s_count[k * kWaves + wave] = __popcll(mates[k]);
        s_active[local] = active[k] ? 1 : 0;
    }
    __syncthreads();
    int nactive = 0;
    int before[kPer];      // entries of the list ahead of this wavefront's group k
#pragma unroll
    for (int k = 0; k < kPer; ++k) before[k] = 0;
#pragma unroll
    for (int q = 0; q < kPer * kWaves; ++q) {
        const int c = s_count[q];
#pragma unroll
        for (int k = 0; k < kPer; ++k)
            if (q < k * kWaves + wave) before[k] += c;
        nactive += c;
    }
#pragma unroll
    for (int k = 0; k < kPer; ++k)
        if (active[k])
            s_list[before[k] + __popcll(mates[k] & ((1ull << lane) - 1ull))] = (unsigned short)(k * kBwdBlock + tid);
    if (!outputs_are_zero && !accumulate) {   // the zero gradients of the gaussians without work
#pragma unroll
        for (int k = 0; k < kPer; ++k) {
            const int local = k * kBwdBlock + tid;
            const size_t i = (size_t)first + local;
            if (local < nrows && !active[k]) {
                dxyz[3 * i] = dxyz[3 * i + 1] = dxyz[3 * i + 2] = 0.0f;
                *reinterpret_cast<float4*>(dquat + 4 * i) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                dscale[3 * i] = dscale[3 * i + 1] = dscale[3 * i + 2] = 0.0f;
                dopacity_out[i] = 0.0f;
                if (dsh_base) dsh_base[3 * i] = dsh_base[3 * i + 1] = dsh_base[3 * i + 2] = 0.0f;
            }
        }
        float* block_dsh = dsh + (size_t)first * rowlen;
        const float inv = 1.0f / (float)rowlen;
        for (int e = tid; e < nrows * rowlen; e += kBwdBlock)
            if (!s_active[(int)(((float)e + 0.5f) * inv)]) block_dsh[e] = 0.0f;
    }
    __syncthreads();
    for (int base = 0; base < nactive; base += rows_per_pass) {
        const int cnt = min(rows_per_pass, nactive - base);
        const int g = first + s_list[base + min(tid, cnt - 1)];
        BwdInputs in = {};
        if (tid < cnt) in = load_bwd_inputs(g, origin ? origin[g] : g, xyz, quat, scale, opacity, cov2d, ne0, rec4);
        bwd_rows_copy<true>(const_cast<float*>(sh), s_rows, s_list + base, cnt, first, rowlen, stride, false, origin);
        __syncthreads();
        if (tid < cnt) {
            d3gs_params Pg = P;
            if constexpr (kInstances) {
                // (the instance table starts at camera batch_index's poses)
                const int b = (row_batch_ids && P_in.batch_size > 1) ? row_batch_ids[g] : cam - batch_index;
                if (row_batch_ids && P_in.batch_size > 1) apply_batch_camera(Pg, b);
                apply_instance(Pg, inst, origin ? origin[g] : g, b);      // ids are per model row
            }
            preprocess_bwd_one(Pg, g, in, sh_mask_compat, accumulate != 0, dxyz, dquat, dscale, dopacity_out,
                               s_rows + tid * stride, dsh_base);
        }
        __syncthreads();
        bwd_rows_copy<false>(dsh, s_rows, s_list + base, cnt, first, rowlen, stride, accumulate != 0);
        __syncthreads();
    }
    };
    if constexpr (kMany) {
        for (int cam = batch_index; cam <= batch_last; ++cam) {
            one_camera(cam);
            __syncthreads();      // the lists are rebuilt for the next camera
        }
    } else {
        one_camera(batch_index);
    }
}

int check_params(const d3gs_params* p, const char* who) {
    if (!p) { set_error("%s: params is NULL", who); return D3GS_ERR_INVALID_ARGUMENT; }
    if (p->n < 0 || p->width <= 0 || p->height <= 0) {
        set_error("%s: bad sizes n=%d width=%d height=%d", who, p->n, p->width, p->height);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (p->tiles_x != (p->width + kTile - 1) / kTile || p->tiles_y != (p->height + kTile - 1) / kTile) {
        set_error("%s: tiles_x/tiles_y do not match ceil(width/16), ceil(height/16)", who);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (p->sh_degree < 0 || p->sh_degree > 3) {
        set_error("%s: sh_degree %d outside [0,3]", who, p->sh_degree);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    int need = (p->sh_degree + 1) * (p->sh_degree + 1) - (p->has_sh_base ? 1 : 0);
    if (p->sh_stride < need) {
        set_error("%s: sh_stride %d holds fewer coefficients than degree %d needs (%d)", who, p->sh_stride,
                  p->sh_degree, need);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (p->filter_algo < 0 || p->filter_algo > 4) {
        set_error("%s: unknown early_filter_algo %d", who, p->filter_algo);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (p->batch_size < 0 || (p->batch_size > 1 && !p->batch_cameras)) {
        set_error("%s: batch_size %d needs batch_cameras", who, p->batch_size);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if ((long long)p->n * batch_count(*p) >= (1ll << 31) ||
        (long long)p->tiles_y * batch_count(*p) >= (1ll << 16) ||
        (long long)p->tiles_x * p->tiles_y * batch_count(*p) >= (1ll << 31)) {
        set_error("%s: bundle of %d cameras is too large (render items and tiles must fit 31 bits, tile rows 16)", who,
                  p->batch_size);
        return D3GS_ERR_UNSUPPORTED;
    }
    if (p->enable_32bit_sort && (!(p->depth_32bit_prec > 0.0f) || p->tiles_x * p->tiles_y * batch_count(*p) >= (1 << 14))) {
        // render.py:227-228: 14 bits of tile index above the 18 depth bits
        set_error("%s: enable_32bit_sort needs depth_32bit_prec > 0 and fewer than 2^14 tiles", who);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    return D3GS_OK;
}

}  // namespace d3gs

using namespace d3gs;

// host view of the optional instance table -> what the kernels take; returns false on a malformed table
static bool instance_view(const d3gs_instances* in, InstanceView* out, const char* who) {
    out->ids = nullptr;
    out->cameras = nullptr;
    out->count = 0;
    if (!in || !in->instance_ids) return true;
    if (in->num_instances < 0 || (in->num_instances > 0 && !in->instance_cameras)) {
        set_error("%s: instance table with %d entries and no cameras", who, in->num_instances);
        return false;
    }
    out->ids = in->instance_ids;
    out->cameras = in->instance_cameras;
    out->count = in->num_instances;
    return true;
}

extern "C" int d3gs_preprocess_fwd(const d3gs_params* p, const float* xyz, const float* quaternion_xyzw,
                                   const float* scale, const float* opacity, const float* color_sh,
                                   const float* color_sh_base, const uint8_t* invalid_mask, float* depths,
                                   int32_t* radii, float* uvs, float* conic_opacity, int32_t* tiles_touched,
                                   float* rgb_gaussian, float* cov2d_vecs, uint8_t* sh_to_rgb_ne_0,
                                   uint64_t* tile_masks, uint32_t* depth_sort_keys, const d3gs_instances* instances,
                                   d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_preprocess_fwd");
    if (rc) return rc;
    if (p->n == 0) return D3GS_OK;
    const bool with_sh = rgb_gaussian != nullptr;
    if (!xyz || !quaternion_xyzw || !scale || !opacity || !depths || !radii || !uvs || !conic_opacity ||
        !tiles_touched || (with_sh && ((!color_sh && p->sh_stride > 0) || (p->has_sh_base && !color_sh_base)))) {
        set_error("d3gs_preprocess_fwd: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    InstanceView inst;
    if (!instance_view(instances, &inst, "d3gs_preprocess_fwd")) return D3GS_ERR_INVALID_ARGUMENT;
    const bool bundle = p->batch_size > 1;
    if (bundle && with_sh) {
        set_error("d3gs_preprocess_fwd: a camera bundle takes its colours from d3gs_sh_colors (rgb_gaussian = NULL)");
        return D3GS_ERR_UNSUPPORTED;
    }
    dim3 grid((item_count(*p) + kPrepBlock - 1) / kPrepBlock), block(kPrepBlock);
    const size_t lds_bytes = with_sh ? (size_t)kPrepBlock * ((p->sh_stride * 3) | 1) * sizeof(float) : 0;
    const SparseView dense = {nullptr, nullptr, nullptr, nullptr};
#define D3GS_LAUNCH_K1(SH, INST)                                                                                      \
    hipLaunchKernelGGL((preprocess_fwd_kernel<SH, INST>), grid, block, lds_bytes, (hipStream_t)stream, *p, inst, dense, \
                       xyz, quaternion_xyzw, scale, opacity, color_sh, color_sh_base, invalid_mask, depths, radii, uvs, \
                       conic_opacity, tiles_touched, rgb_gaussian, cov2d_vecs, sh_to_rgb_ne_0,                         \
                       (unsigned long long*)tile_masks, depth_sort_keys)
    if (with_sh) { if (inst.ids) D3GS_LAUNCH_K1(true, true); else D3GS_LAUNCH_K1(true, false); }
    else         { if (inst.ids || bundle) D3GS_LAUNCH_K1(false, true); else D3GS_LAUNCH_K1(false, false); }
#undef D3GS_LAUNCH_K1
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_preprocess_fwd: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_preprocess_fwd_sparse(const d3gs_params* p, const float* xyz, const float* quaternion_xyzw,
                                          const float* scale, const float* opacity, const uint8_t* invalid_mask,
                                          int32_t* valid_flags, const int32_t* slot_scan, int32_t* sparse_gaussian_ids,
                                          int32_t* sparse_batch_ids, float* depths, int32_t* radii, float* uvs,
                                          float* conic_opacity, int32_t* tiles_touched, float* cov2d_vecs,
                                          uint64_t* tile_masks, uint32_t* depth_sort_keys,
                                          const d3gs_instances* instances, d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_preprocess_fwd_sparse");
    if (rc) return rc;
    if (p->n == 0) return D3GS_OK;
    if (!xyz || !quaternion_xyzw || !scale || !opacity) {
        set_error("d3gs_preprocess_fwd_sparse: NULL model buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    const bool first = valid_flags != nullptr;
    if (first == (slot_scan != nullptr) ||
        (!first && (!sparse_gaussian_ids || !sparse_batch_ids || !depths || !radii || !uvs || !conic_opacity ||
                    !tiles_touched))) {
        set_error("d3gs_preprocess_fwd_sparse: give valid_flags alone (first call), or slot_scan with the id and output "
                  "buffers (second call)");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    InstanceView inst;
    if (!instance_view(instances, &inst, "d3gs_preprocess_fwd_sparse")) return D3GS_ERR_INVALID_ARGUMENT;
    const SparseView sparse = {valid_flags, slot_scan, sparse_gaussian_ids, sparse_batch_ids};
    dim3 grid((item_count(*p) + kPrepBlock - 1) / kPrepBlock), block(kPrepBlock);
    hipLaunchKernelGGL((preprocess_fwd_kernel<false, true, true>), grid, block, 0, (hipStream_t)stream, *p, inst, sparse,
                       xyz, quaternion_xyzw, scale, opacity, (const float*)nullptr, (const float*)nullptr, invalid_mask,
                       depths, radii, uvs, conic_opacity, tiles_touched, (float*)nullptr, cov2d_vecs, (uint8_t*)nullptr,
                       (unsigned long long*)tile_masks, depth_sort_keys);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_preprocess_fwd_sparse: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_sh_colors_sparse(const d3gs_params* p, const int32_t* sparse_gaussian_ids,
                                     const int32_t* sparse_batch_ids, int32_t count, const float* xyz,
                                     const float* color_sh, const float* color_sh_base, const int32_t* radii,
                                     float* rgb_gaussian, uint8_t* sh_to_rgb_ne_0, const d3gs_instances* instances,
                                     d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_sh_colors_sparse");
    if (rc) return rc;
    if (count < 0) { set_error("d3gs_sh_colors_sparse: count < 0"); return D3GS_ERR_INVALID_ARGUMENT; }
    if (count == 0) return D3GS_OK;
    if (!sparse_gaussian_ids || !sparse_batch_ids || !xyz || (!color_sh && p->sh_stride > 0) || !radii || !rgb_gaussian ||
        (p->has_sh_base && !color_sh_base)) {
        set_error("d3gs_sh_colors_sparse: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    InstanceView inst;
    if (!instance_view(instances, &inst, "d3gs_sh_colors_sparse")) return D3GS_ERR_INVALID_ARGUMENT;
    hipLaunchKernelGGL(sh_colors_sparse_kernel, dim3((count + kPrepBlock - 1) / kPrepBlock), dim3(kPrepBlock), 0,
                       (hipStream_t)stream, *p, sparse_gaussian_ids, sparse_batch_ids, (int)count, inst, xyz, color_sh,
                       color_sh_base, radii, rgb_gaussian, sh_to_rgb_ne_0);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_sh_colors_sparse: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_sh_colors(const d3gs_params* p, const float* xyz, const float* color_sh, const float* color_sh_base,
                              const int32_t* radii, float* rgb_gaussian, uint8_t* sh_to_rgb_ne_0,
                              const d3gs_instances* instances, d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_sh_colors");
    if (rc) return rc;
    if (p->n == 0) return D3GS_OK;
    if (!xyz || (!color_sh && p->sh_stride > 0) || !radii || !rgb_gaussian || (p->has_sh_base && !color_sh_base)) {
        set_error("d3gs_sh_colors: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    InstanceView inst;
    if (!instance_view(instances, &inst, "d3gs_sh_colors")) return D3GS_ERR_INVALID_ARGUMENT;
    const int chunks = ((p->n + kPrepBlock - 1) / kPrepBlock) * batch_count(*p);
    // A small grid, so that the kernel fills idle slots beside the binning stages it runs next to instead of
    // displacing them; what it has to do is end before the forward blend starts.  Measured per view: 1M gaussians
    // 0.837 ms with 512 workgroups, 0.842 with 325 to 384, 0.846 with 768, 0.857 with 1024 (the larger grids slow
    // the depth sort by more than they gain); 3M gaussians 1.94 ms with 384, 1.96 with 512, 1.97 with 976 (the depth
    // sort of 3M keys suffers most).  Hence 512 falling to 384 between 1M and 2M gaussians, and growing with the
    // scene only where 384 could no longer end in time.
    const int falling = std::min(512, std::max(kShColorBlocks, 768 - chunks / 30));
    const int blocks = std::min(1024, std::max(falling, chunks / 60));
    dim3 grid(chunks < blocks ? chunks : blocks), block(kPrepBlock);
    const size_t lds_bytes = (size_t)kPrepBlock * ((p->sh_stride * 3) | 1) * sizeof(float);
    if (inst.ids || p->batch_size > 1)
        hipLaunchKernelGGL(sh_colors_kernel<true>, grid, block, lds_bytes, (hipStream_t)stream, *p, inst, xyz, color_sh,
                           color_sh_base, radii, rgb_gaussian, sh_to_rgb_ne_0);
    else
        hipLaunchKernelGGL(sh_colors_kernel<false>, grid, block, lds_bytes, (hipStream_t)stream, *p, inst, xyz, color_sh,
                           color_sh_base, radii, rgb_gaussian, sh_to_rgb_ne_0);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_sh_colors: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

static int preprocess_bwd_impl(const char* who, const d3gs_params* p, int32_t batch_index, int32_t batch_last,
                               int32_t accumulate,
                               const int32_t* origin, const float* xyz, const float* quaternion_xyzw,
                               const float* scale, const float* opacity, const float* color_sh, const int32_t* radii,
                               const float* cov2d_vecs, const uint8_t* sh_to_rgb_ne_0, const float* grad_records,
                               const uint8_t* touched, int32_t sh_mask_compat, int32_t outputs_are_zero, float* dxyz,
                               float* dquaternion_xyzw, float* dscale, float* dopacity_out, float* dcolor_sh,
                               float* dcolor_sh_base, const d3gs_instances* instances, const int32_t* row_batch_ids,
                               d3gs_stream_t stream);

extern "C" int d3gs_preprocess_bwd(const d3gs_params* p, const float* xyz, const float* quaternion_xyzw,
                                   const float* scale, const float* opacity, const float* color_sh,
                                   const int32_t* radii, const float* cov2d_vecs, const uint8_t* sh_to_rgb_ne_0,
                                   const float* grad_records, const uint8_t* touched, int32_t sh_mask_compat,
                                   int32_t outputs_are_zero,
                                   float* dxyz, float* dquaternion_xyzw, float* dscale, float* dopacity_out,
                                   float* dcolor_sh, float* dcolor_sh_base, const d3gs_instances* instances,
                                   d3gs_stream_t stream) {
    // a bundle: every camera in this one launch, the per-item arrays holding batch_size * n rows
    return preprocess_bwd_impl("d3gs_preprocess_bwd", p, 0, p ? batch_count(*p) - 1 : 0, 0, nullptr, xyz, quaternion_xyzw,
                               scale, opacity, color_sh, radii, cov2d_vecs, sh_to_rgb_ne_0, grad_records, touched,
                               sh_mask_compat, outputs_are_zero, dxyz, dquaternion_xyzw, dscale, dopacity_out, dcolor_sh,
                               dcolor_sh_base, instances, nullptr, stream);
}

extern "C" int d3gs_preprocess_bwd_sparse(const d3gs_params* p, const int32_t* sparse_gaussian_ids, const float* xyz,
                                          const float* quaternion_xyzw, const float* scale, const float* opacity,
                                          const float* color_sh, const int32_t* radii, const float* cov2d_vecs,
                                          const uint8_t* sh_to_rgb_ne_0, const float* grad_records, const uint8_t* touched,
                                          int32_t sh_mask_compat, int32_t outputs_are_zero, float* dxyz,
                                          float* dquaternion_xyzw, float* dscale, float* dopacity_out, float* dcolor_sh,
                                          float* dcolor_sh_base, const d3gs_instances* instances,
                                          const int32_t* sparse_batch_ids, d3gs_stream_t stream) {
    if (!sparse_gaussian_ids && p && p->n > 0) {
        set_error("d3gs_preprocess_bwd_sparse: sparse_gaussian_ids is NULL");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (p && p->batch_size > 1 && !sparse_batch_ids) {
        set_error("d3gs_preprocess_bwd_sparse: the compact rows of a bundle need sparse_batch_ids");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    return preprocess_bwd_impl("d3gs_preprocess_bwd_sparse", p, 0, 0, 0, sparse_gaussian_ids, xyz, quaternion_xyzw, scale,
                               opacity, color_sh, radii, cov2d_vecs, sh_to_rgb_ne_0, grad_records, touched, sh_mask_compat,
                               outputs_are_zero, dxyz, dquaternion_xyzw, dscale, dopacity_out, dcolor_sh, dcolor_sh_base,
                               instances, sparse_batch_ids, stream);
}

extern "C" int d3gs_preprocess_bwd_camera(const d3gs_params* p, int32_t batch_index, int32_t accumulate, const float* xyz,
                                          const float* quaternion_xyzw, const float* scale, const float* opacity,
                                          const float* color_sh, const int32_t* radii, const float* cov2d_vecs,
                                          const uint8_t* sh_to_rgb_ne_0, const float* grad_records,
                                          const uint8_t* touched, int32_t sh_mask_compat, int32_t outputs_are_zero,
                                          float* dxyz, float* dquaternion_xyzw, float* dscale, float* dopacity_out,
                                          float* dcolor_sh, float* dcolor_sh_base, const d3gs_instances* instances,
                                          d3gs_stream_t stream) {
    return preprocess_bwd_impl("d3gs_preprocess_bwd_camera", p, batch_index, batch_index, accumulate, nullptr, xyz, quaternion_xyzw, scale,
                               opacity, color_sh, radii, cov2d_vecs, sh_to_rgb_ne_0, grad_records, touched, sh_mask_compat,
                               outputs_are_zero, dxyz, dquaternion_xyzw, dscale, dopacity_out, dcolor_sh, dcolor_sh_base,
                               instances, nullptr, stream);
}

// origin (sparse mode): p->n compact items, item i being row origin[i] of the model arrays; gradients are written per
// item.
static int preprocess_bwd_impl(const char* who, const d3gs_params* p, int32_t batch_index, int32_t batch_last,
                               int32_t accumulate, const int32_t* origin, const float* xyz,
                               const float* quaternion_xyzw, const float* scale, const float* opacity,
                               const float* color_sh, const int32_t* radii, const float* cov2d_vecs,
                               const uint8_t* sh_to_rgb_ne_0, const float* grad_records, const uint8_t* touched,
                               int32_t sh_mask_compat, int32_t outputs_are_zero, float* dxyz, float* dquaternion_xyzw,
                               float* dscale, float* dopacity_out, float* dcolor_sh, float* dcolor_sh_base,
                               const d3gs_instances* instances, const int32_t* row_batch_ids, d3gs_stream_t stream) {
    int rc = check_params(p, who);
    if (rc) return rc;
    if (batch_index < 0 || batch_index >= batch_count(*p) || batch_last < batch_index || batch_last >= batch_count(*p)) {
        set_error("%s: cameras %d..%d outside the bundle of %d", who, batch_index, batch_last, batch_count(*p));
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (p->n == 0) return D3GS_OK;
    // a model whose only colour coefficient is the split-off DC term has empty color_sh arrays (sh_stride 0)
    if (!xyz || !quaternion_xyzw || !scale || !opacity || !radii || !cov2d_vecs || !sh_to_rgb_ne_0 ||
        !grad_records || !dxyz || !dquaternion_xyzw || !dscale || !dopacity_out ||
        ((!color_sh || !dcolor_sh) && p->sh_stride > 0) || (p->has_sh_base && !dcolor_sh_base)) {
        set_error("d3gs_preprocess_bwd: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    InstanceView inst;
    if (!instance_view(instances, &inst, "d3gs_preprocess_bwd")) return D3GS_ERR_INVALID_ARGUMENT;
    const int rows_per_pass = bwd_rows_per_pass(p->sh_stride);
    const size_t lds_bytes = (size_t)rows_per_pass * ((p->sh_stride * 3) | 1) * sizeof(float);
    // four gaussians per thread once there are enough workgroups to fill the chip that way
    const bool wide = p->n >= 512 * kBwdBlock * 4;
    const int per = wide ? 4 : 1;
    dim3 grid((p->n + kBwdBlock * per - 1) / (kBwdBlock * per)), block(kBwdBlock);
#define D3GS_LAUNCH_K9(PER, INST, MANY)                                                                                     \
    hipLaunchKernelGGL((preprocess_bwd_kernel<PER, INST, MANY>), grid, block, lds_bytes, (hipStream_t)stream, *p,      \
                       (int)batch_index, (int)batch_last, (int)accumulate, inst, xyz,                                                   \
                       quaternion_xyzw, scale, opacity, color_sh, radii, cov2d_vecs, sh_to_rgb_ne_0, grad_records,     \
                       touched,                                                                                        \
                       (int)sh_mask_compat, (int)outputs_are_zero, rows_per_pass, origin, row_batch_ids, dxyz,         \
                       dquaternion_xyzw,                                                                               \
                       dscale,                                                                                         \
                       dopacity_out,                                                                                   \
                       dcolor_sh, dcolor_sh_base)
    const bool per_row = inst.ids || (row_batch_ids && p->batch_size > 1);      // the instantiation that forms a camera per row
    const bool many = batch_last > batch_index;
    if (wide) {
        if (many) { if (per_row) D3GS_LAUNCH_K9(4, true, true); else D3GS_LAUNCH_K9(4, false, true); }
        else      { if (per_row) D3GS_LAUNCH_K9(4, true, false); else D3GS_LAUNCH_K9(4, false, false); }
    } else {
        if (many) { if (per_row) D3GS_LAUNCH_K9(1, true, true); else D3GS_LAUNCH_K9(1, false, true); }
        else      { if (per_row) D3GS_LAUNCH_K9(1, true, false); else D3GS_LAUNCH_K9(1, false, false); }
    }
#undef D3GS_LAUNCH_K9
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_preprocess_bwd: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}
