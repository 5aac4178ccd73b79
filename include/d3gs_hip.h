/*
 * d3gs_hip.h — C ABI of libd3gs_hip.so, the MI355X (gfx950) implementation of
 * the 3D-Gaussian-splatting rasterize forward/backward path.
 *
 * The reference reaches its GPU code through two native boundaries:
 *   (1) JIT kernel launches  `self._inliner.kernel_1d / kernel_raw(name, ..., code)`
 *       (d3sim/csrc/inliner.py:35-43; call sites listed per entry point below);
 *   (2) the pybind module    `d3sim.d3sim_thtools.device_sort.DeviceSort`
 *       (d3sim/csrc/devsort.py:20-149, stubs d3sim_thtools/device_sort.pyi:3-38).
 * Every entry point below replaces one of those call sites.
 *
 * Conventions
 *   - all pointers are DEVICE pointers unless the name ends in `_host`;
 *   - the caller owns every buffer (outputs, accumulators, workspaces); nothing
 *     here allocates or frees device memory;
 *   - every call enqueues work on `stream` (a hipStream_t passed as void*) and
 *     returns without synchronising;
 *   - return value 0 = success; negative = error (D3GS_ERR_*), with a message
 *     available from d3gs_last_error_string() (thread local);
 *   - accumulators written with atomics (duv, dconic, dopacity, dcolor) and the
 *     tile range table must be zero-filled by the caller, as in the reference
 *     (render.py:897, 1388-1411).
 */
#ifndef D3GS_HIP_H_
#define D3GS_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define D3GS_ABI_VERSION 34

#define D3GS_OK 0
#define D3GS_ERR_INVALID_ARGUMENT (-1)
#define D3GS_ERR_UNSUPPORTED (-2)
#define D3GS_ERR_WORKSPACE_TOO_SMALL (-3)
#define D3GS_ERR_LAUNCH (-4)
#define D3GS_ERR_SORT_LOOKBACK (-5) /* status word of d3gs_sort_status: a workgroup's bounded wait ran out */

/* Values a pair-count word (total_dev / total_host of d3gs_scan_gathered and d3gs_bin_pairs) takes in place of
 * the count when a kernel's bounded wait on an earlier workgroup ran out; the lists are then not valid. */
#define D3GS_COUNT_SCAN_GAVE_UP (-1)
#define D3GS_COUNT_SORT_GAVE_UP (-2)
/* not written by the library: what a caller that polls the host word of d3gs_bin_pairs puts there beforehand */
#define D3GS_COUNT_PENDING (-3)
/* Most (tile, gaussian) pairs of one call: list positions are 31-bit (int32 offsets, tile ranges and sort
 * prefixes, like the reference's, whose CUB sort takes an int count, devsort.py:96-129).  A sort of more is
 * refused with D3GS_ERR_UNSUPPORTED; the scans still return the true int64 total, so a caller sees it. */
#define D3GS_MAX_PAIRS ((1ll << 31) - 1024)

/* EarlyFilterAlgo, d3sim/algos/d3gs/config_def.py:59-70 */
#define D3GS_FILTER_NONE 0
#define D3GS_FILTER_AABB 1
#define D3GS_FILTER_ELLIPSE 2 /* exact ellipse / tile test, render.py:1277-1297; gs3d.py:1078-1240 */
#define D3GS_FILTER_OBB 3
#define D3GS_FILTER_OBB_DFVT 4 /* computed as the OBB tile set */

typedef void* d3gs_stream_t;

/* Scalars the reference bakes into the JIT source text (render.py:198-230,
 * 333-358; config_def.py:77-151). Plain data, passed by pointer from the host. */
typedef struct d3gs_params {
    int32_t n;           /* number of gaussians */
    int32_t width, height;
    int32_t tiles_x, tiles_y; /* ceil(width/16), ceil(height/16) */
    int32_t sh_degree;   /* evaluated SH degree (cur_sh_degree), 0..3 */
    int32_t sh_stride;   /* coefficients per gaussian stored in color_sh */
    int32_t has_sh_base; /* DC coefficient lives in color_sh_base */
    int32_t filter_algo; /* D3GS_FILTER_* */
    int32_t training;
    float fx, fy, cx, cy;
    float tan_fovx, tan_fovy; /* 0.5 * (W,H) / focal */
    float w2c[9];        /* rows 0..2 of cam2world_T = world->camera rotation */
    float cam_center[3]; /* row 3 of cam2world_T */
    float z_near, z_far;
    float eps;
    float radii_eigen_eps;
    float clamp_factor;
    float std_sigma;
    float lowpass;
    float alpha_eps;
    float transmittance_eps;
    float scale_global;
    float bg[3];
    int32_t fused_activation; /* 1: scale/quaternion/opacity are raw and the kernels apply exp / normalize /
                                 sigmoid (GaussianModelOriginFused, origin/model.py:435-465); 0: they are already
                                 activated (GaussianModelOrigin, origin/model.py:249-270) and gradients are
                                 returned w.r.t. the activated values */
    int32_t render_depth;         /* blend camera-space depth as one more channel (render.py:1532-1539, 1915-1919) */
    int32_t render_rgba;          /* colour has a fourth channel, the sum of the blend weights (render.py:1899-1906) */
    int32_t use_nchw;             /* colour / drgb stored [C,H,W] instead of [H,W,C] (render.py:702, 2272-2294) */
    int32_t enable_anti_aliasing; /* conic without eps and opacity *= sqrt(det / det_lowpass) (render.py:391-407) */
    int32_t enable_32bit_sort;    /* the depth part of the sort key is uint32(depth / depth_32bit_prec) & 0x3FFFF instead
                                     of the float bits (render.py:767-770, 853-854): gaussians of a tile that fall into
                                     the same depth step are blended in index order.  At most 2^14 tiles. */
    float depth_32bit_prec;       /* config_def.py:91, default 0.001 */
    int32_t render_inv_depth;     /* config_def.py:95; render.py:582, 773, 1965, 3051, 3283: K1 stores 1 / z in `depths`
                                     where it stores z otherwise.  The sort key's depth part is taken from that same
                                     buffer, as in the reference, so the lists come out in descending camera depth and
                                     the blend runs over them in that order; the depth channel blends 1 / z, the blend
                                     backward's dz is dL/d(1/z), and K9 turns it into -dz / z^2. */
    /* Camera bundle (render.py:129-150, 314-326): batch_size = B > 1 renders B cameras of one image size in one
     * pass over B * n "render items", item i = b * n + g being gaussian g seen by camera b.  The model arrays keep
     * n rows; everything K1 writes (and the reject mask it reads) has B * n rows; tile ids carry the camera,
     * b * tiles_x * tiles_y + y * tiles_x + x (render.py:787, 809), so the sort and the range table cover
     * B * tiles_x * tiles_y tiles; images are [B, H, W, C].  The cameras come from device memory: batch_cameras
     * [B][16] = rows 0-2 of cam2world_T (9 floats, the layout of w2c), its row 3 (the centre), focal x, y and
     * principal point x, y; the fields w2c, cam_center, fx, fy, cx, cy, tan_fovx, tan_fovy above are then not read
     * (render.py:316-323 loads the same from its [B,4,3] and [B,4] tensors).  batch_size 0 or 1: one camera, the
     * fields above. */
    int32_t batch_size;
    /* Sparse mode over a bundle (no counterpart field in the reference, whose kernels take the sparse ids as extra
     * arguments): when > 0, the per-item arrays of the entry points BEHIND K1 hold this many rows -- the accepted
     * (camera, gaussian) items, in ascending item order -- instead of batch_size * n; the camera of a row is named by
     * the kept-tile record (d3gs_make_keys then needs tile_masks) and by sparse_batch_ids (K9).  0: batch_size * n. */
    int32_t compact_items;
    const float* batch_cameras;
    /* measure_atomic_add_count (config_def.py:134; render.py:1451-1453, 2145-2148, 2310-2311): when not NULL, the
     * blend backward kernels add to this device counter the number of global atomic requests they issue (one
     * line-wide request per (tile, gaussian) whose sums are not all zero; the reference counts its per-value
     * atomicAdd calls).  The caller zeroes it. */
    uint32_t* atomic_add_count;
} d3gs_params;

#define D3GS_BATCH_CAMERA_FLOATS 16

int d3gs_abi_version(void);
const char* d3gs_last_error_string(void);

/* DeviceSort.get_higher_msb — devsort.py:131-149: bit length of n. */
int d3gs_higher_msb(uint32_t n);

/* Number of significant bits of the depth-sort keys that d3gs_preprocess_fwd writes to depth_sort_keys (no
 * counterpart in the reference): accepted depths lie in [z_near, z_far], so the key is the depth's float bits
 * minus those of z_near -- the same order in fewer bits (27 for the default planes 0.2 and 1e4) -- or, with
 * enable_32bit_sort, the 18-bit depth step; with render_inv_depth the stored 1 / z lies in [1 / z_far, 1 / z_near]
 * and the key is its float bits minus those of 1 / z_far.  The depth sort runs on bits [0, d3gs_depth_key_bits(p)). */
int d3gs_depth_key_bits(const d3gs_params* p);

/* Instance rendering (render.py:207-220, 346-356): a gaussian with instance_ids[i] = k >= 0 belongs to object
 * instance k, its parameters are given in that object's frame, and it is seen by the camera expressed in that
 * frame: instance_cameras[k] holds the 9 floats of the world-to-camera rotation in the instance frame (row
 * major, the layout of d3gs_params.w2c) followed by the camera centre in the instance frame, i.e.
 * cam2instance = world2instance o cam2world, which the reference derives from instance2world_T[frame][k] inside
 * its kernels and the caller derives here.  Gaussians with a negative (or out of range) id use the view's own
 * camera.  Passed by pointer to K1, the SH colours and K9; NULL, or instance_ids == NULL, means no instances. */
typedef struct d3gs_instances {
    const int32_t* instance_ids;     /* [N] device */
    const float* instance_cameras;   /* [num_instances][12] device; with d3gs_params.batch_size = B > 1 one such
                                      * table per camera, [B][num_instances][12] (d3gs_preprocess_bwd_camera takes
                                      * the table of its camera alone) */
    int32_t num_instances;
} d3gs_instances;

/* K1 — replaces kernel_raw("gs3d_preprocess_...") at render.py:629-681 (body
 * 421-476, 569-619).  One pass over the gaussians: fused activations, projection,
 * EWA covariance, conic, radius, tile rect, validity, tile count under the chosen
 * early filter, SH colour.  Outputs of rejected gaussians are written as zeros.
 * cov2d_vecs and sh_to_rgb_ne_0 may be NULL (inference). sh_base may be NULL.
 * invalid_mask (uint8[N], may be NULL): non-zero rejects the gaussian (render.py:306-308).
 * tile_masks (uint64[N][2], 16-byte aligned, may be NULL; no counterpart in the reference): a record of the tiles the
 * early filter kept for each gaussian (word 0: bit mask over its candidate rect, word 1: the rect), which
 * d3gs_make_keys expands instead of repeating the per-tile tests.
 * rgb_gaussian may be NULL: the SH colour (and sh_to_rgb_ne_0) is then left to d3gs_sh_colors, which a
 * caller can run on a second stream beside the sort, the only consumer being the blend.
 * depth_sort_keys (uint32[N], may be NULL): the keys of the depth sort, the float bits of depths relative to
 * those of z_near or, with enable_32bit_sort, the 18-bit depth steps (saves the d3gs_depth_keys pass; the depth
 * sort then runs on bits [0, d3gs_depth_key_bits(p))). */
int d3gs_preprocess_fwd(const d3gs_params* p, const float* xyz, const float* quaternion_xyzw, const float* scale,
                        const float* opacity, const float* color_sh, const float* color_sh_base,
                        const uint8_t* invalid_mask, float* depths,
                        int32_t* radii, float* uvs, float* conic_opacity, int32_t* tiles_touched, float* rgb_gaussian,
                        float* cov2d_vecs, uint8_t* sh_to_rgb_ne_0, uint64_t* tile_masks, uint32_t* depth_sort_keys,
                        const d3gs_instances* instances, d3gs_stream_t stream);

/* The SH-colour part of K1 on its own (render.py:569-613): rgb_gaussian [N,3] and, when not NULL, the
 * clamp mask sh_to_rgb_ne_0 [N] of the gaussians with radii > 0, zeros for the rest.  Same values as the
 * fused call. */
int d3gs_sh_colors(const d3gs_params* p, const float* xyz, const float* color_sh, const float* color_sh_base,
                   const int32_t* radii, float* rgb_gaussian, uint8_t* sh_to_rgb_ne_0, const d3gs_instances* instances,
                   d3gs_stream_t stream);

/* K2 — replaces `tiles_touched.cumsum_(0)` + `.item()` at render.py:694-695.
 * In-place inclusive scan; the grand total is written to *total_dev (device
 * int64).  Workspace size from d3gs_scan_workspace_bytes. */
int d3gs_scan_workspace_bytes(int32_t n, size_t* bytes_out_host);
int d3gs_scan_tiles(int32_t* tiles_touched, int32_t n, void* workspace, size_t workspace_bytes, int64_t* total_dev,
                    d3gs_stream_t stream);

/* K2 over a permutation, in one launch: out[j] = sum_{i <= j} src[index[i]] (index NULL: the identity), the same
 * `cumsum_` (render.py:694-695) taken in the order K3 emits the pairs; the grand total goes to *total_dev
 * (device int64; D3GS_COUNT_SCAN_GAVE_UP if the kernel's bounded wait on an earlier chunk ran out) and, when total_host is not NULL, to
 * that word of pinned (device-mapped) host memory as well, stored by the kernel itself: the host may read it
 * once it has waited for the stream to pass this call.  An index outside [0, src_n)
 * counts as 0.  The workspace (size from d3gs_scan_gathered_workspace_bytes) must be zero on entry:
 * workspace_is_zero != 0 says the caller has cleared it, otherwise a fill kernel runs first. */
int d3gs_scan_gathered_workspace_bytes(int32_t n, size_t* bytes_out_host);
int d3gs_scan_gathered(const int32_t* src, int32_t src_n, const int32_t* index, int32_t n, int32_t* out,
                       void* workspace, size_t workspace_bytes, int32_t workspace_is_zero, int64_t* total_dev,
                       int64_t* total_host, d3gs_stream_t stream);

/* d3gs_scan_gathered without a workspace argument, for callers that cannot allocate one.  It has no counterpart
 * in the reference (whose `cumsum_` allocates its temporary storage inside torch); it is meant for code under HIP
 * graph capture, tight serving loops and harnesses that forbid hipMalloc.  The look-back's status words live in
 * a file-scope device array of the library (32 KiB + 256 B per GPU, held until the process ends), so n is limited
 * to D3GS_SCAN_NOALLOC_MAX_N elements (a larger n returns D3GS_ERR_WORKSPACE_TOO_SMALL).  The call allocates and
 * frees nothing; it clears the part of the array it uses with a fill kernel on `stream` and then runs the same
 * kernel as d3gs_scan_gathered: same outputs bit for bit.  The array is resolved for the device that is
 * current at the first call on that device (make that first call outside a graph capture).  All calls on one
 * GPU share the array: calls that overlap on one GPU (two streams) race; calls on one stream are safe. */
#define D3GS_SCAN_NOALLOC_MAX_N (1 << 24)
int d3gs_scan_gathered_noalloc(const int32_t* src, int32_t src_n, const int32_t* index, int32_t n, int32_t* out,
                               int64_t* total_dev, int64_t* total_host, d3gs_stream_t stream);

/* K3 — replaces kernel_1d("prepare_sort_data_...") at render.py:739-840.
 * Without gaussian_order (NULL) this is the reference's call: offsets = the inclusive
 * scan of tiles_touched from d3gs_scan_tiles, m = its total, pairs are emitted in
 * gaussian-index order.  With gaussian_order (a permutation of 0..n-1), slot j emits
 * gaussian gaussian_order[j] and offsets must be the inclusive scan of the tile counts
 * taken in that order (see d3gs_depth_keys).  Two optional inputs (may be NULL) save gathers
 * without changing the pairs emitted: ordered_depth_keys[j] (uint32), the sorted keys of the depth sort
 * (= depth bits of gaussian gaussian_order[j]), read instead of depths[gaussian_order[j]];
 * tile_masks, the record d3gs_preprocess_fwd wrote with the same params.
 * Exactly one of keys / tile_keys is given.  tile_keys (uint32[m]) receives the tile id alone: with the
 * pairs emitted in depth order the pair sort only needs the tile digits, so the 32-bit variants below
 * (d3gs_sort_pairs_u32 on bits [0, d3gs_higher_msb(num_tiles)), d3gs_tile_ranges_u32) move a third less. */
int d3gs_make_keys(const d3gs_params* p, const int32_t* radii, const float* uvs, const float* conic_opacity,
                   const float* depths, const int32_t* offsets, const int32_t* gaussian_order,
                   const uint32_t* ordered_depth_keys, const uint64_t* tile_masks, uint64_t* keys,
                   uint32_t* tile_keys, int32_t* gaussian_idx, int64_t m, d3gs_stream_t stream);

/* Depth-first factorisation of the pair sort (no counterpart in the reference, which
 * radix-sorts all M pairs on the full (tile, depth) key; the result is bit-identical).
 * An LSD radix sort is a chain of stable sorts from the least significant digit up, and
 * the depth digits only depend on the gaussian, so: sort the N gaussians by depth bits
 * (d3gs_depth_keys + d3gs_sort_pairs on bits [0, 32)), emit the pairs in that order
 * (d3gs_gather_i32 of the tile counts, d3gs_scan_tiles, d3gs_make_keys with
 * gaussian_order) and run only the tile digits, bits [32, end_bit), over the M pairs.
 *   d3gs_depth_keys: keys[i] = float bits of depths[i] (zero-extended), gaussian_idx[i] = i
 *   d3gs_gather_i32: dst[j] = src[index[j]] (0 for an index outside [0, src_n)) */
int d3gs_depth_keys(const float* depths, int32_t n, uint64_t* keys, int32_t* gaussian_idx, d3gs_stream_t stream);
int d3gs_gather_i32(const int32_t* src, int32_t src_n, const int32_t* index, int32_t n, int32_t* dst,
                    d3gs_stream_t stream);

/* K4 — replaces DeviceSort.get_sort_workspace_size / do_radix_sort_with_bit_range
 * (devsort.py:38-129; call site render.py:846-887).  Stable LSD radix sort of
 * (uint64 key, int32 value) pairs on key bits [begin_bit, end_bit), ping-ponging
 * between the a and b buffers.  *result_in_b_host (host int) tells which pair of
 * buffers holds the result, like the reference's (key_swap, value_swap).  m <= D3GS_MAX_PAIRS. */
int d3gs_sort_workspace_bytes(int64_t m, int begin_bit, int end_bit, size_t* bytes_out_host);
int d3gs_sort_pairs(uint64_t* keys_a, uint64_t* keys_b, int32_t* vals_a, int32_t* vals_b, void* workspace,
                    size_t workspace_bytes, int64_t m, int begin_bit, int end_bit, int* result_in_b_host,
                    d3gs_stream_t stream);
/* The same over 32-bit keys (end_bit <= 32); the workspace size is that of d3gs_sort_workspace_bytes(m).
 * m_device (device int64, may be NULL): when given, m is the capacity of the buffers and the number of
 * pairs sorted is min(m, *m_device), read on the device - a caller that sized its buffers from an
 * earlier view can enqueue the sort without waiting for the scan total to reach the host.
 * values_are_indices != 0: the input values are taken to be 0..m-1 and vals_a is not read (it is still
 * one of the two output buffers).
 * workspace_is_zero != 0: the caller has zero-filled the workspace (say, together with its other
 * zero-initialised buffers in one fill) and the sort does not clear it again. */
int d3gs_sort_pairs_u32(uint32_t* keys_a, uint32_t* keys_b, int32_t* vals_a, int32_t* vals_b, void* workspace,
                        size_t workspace_bytes, int64_t m, const int64_t* m_device, int values_are_indices,
                        int workspace_is_zero, int begin_bit, int end_bit, int* result_in_b_host,
                        d3gs_stream_t stream);

/* Error report of a sort (the reference's sort throws through TV_THROW_RT_ERR, devsort.py:34-37).  The pass
 * kernels learn where their digits start from the workgroups before them by polling status words; the polling is
 * bounded, and a workgroup whose wait runs out raises an error word in the workspace and carries on, so the
 * grid always drains but the output is not sorted.  d3gs_sort_status enqueues, behind the sort on `stream`, a
 * one-thread kernel that writes 0 or D3GS_ERR_SORT_LOOKBACK to *status_dev (device) and *status_host (pinned,
 * device-mapped host memory; the host reads it once it has waited for the stream to pass this call); either
 * may be NULL.  workspace, m and the bit range are those of the sort call.  d3gs_sort_error_offset gives the
 * byte offset of that uint32 error word inside the workspace for callers that copy it out themselves. */
int d3gs_sort_error_offset(int64_t m, int begin_bit, int end_bit, size_t* offset_out_host);
int d3gs_sort_status(const void* workspace, size_t workspace_bytes, int64_t m, int begin_bit, int end_bit,
                     int32_t* status_dev, int32_t* status_host, d3gs_stream_t stream);

/* K5 — replaces kernel_1d("prepare_workload_range_...") at render.py:896-939.
 * ranges[num_tiles][2] must be zero-filled by the caller.  tile_order (int32[num_tiles],
 * may be NULL) receives the tile ids sorted by descending list length: a launch order
 * for the blend kernels that starts the longest tiles first (no counterpart in the
 * reference, which launches tiles in raster order; it changes scheduling, not results). */
int d3gs_tile_ranges(const uint64_t* keys_sorted, int64_t m, int32_t* workload_ranges, int32_t num_tiles,
                     int32_t* tile_order, d3gs_stream_t stream);
/* the same over 32-bit tile keys (see d3gs_make_keys); m_device as in d3gs_sort_pairs_u32 */
int d3gs_tile_ranges_u32(const uint32_t* tile_keys_sorted, int64_t m, const int64_t* m_device,
                         int32_t* workload_ranges, int32_t num_tiles, int32_t* tile_order, d3gs_stream_t stream);

/* The binning of one view from K1's outputs to the tile ranges, enqueued by one call (no counterpart in the
 * reference, whose host issues render.py:694-939 launch by launch): d3gs_sort_pairs_u32 of the N depth keys
 * (depth_keys_a = K1's depth_sort_keys; values are the gaussian indices), d3gs_scan_gathered of tiles_touched in
 * that order into offsets [N], d3gs_make_keys into tile_keys_a / idx_a [capacity], d3gs_sort_pairs_u32 on the
 * tile bits with the pair count read from *total_dev, d3gs_tile_ranges_u32 (+ tile_order, may be NULL).
 * Results: *order_in_b / *pairs_in_b say which of the a / b buffers hold the depth order and the sorted pairs;
 * *total_dev the pair count M (the kernels touch min(M, capacity) pairs: a caller that sized capacity from a
 * guess compares M with it afterwards and bins again when M is larger); total_host, when not NULL, is a pinned
 * host word that the scan kernel stores M to (see d3gs_scan_gathered).  When either sort raised its error word
 * (see d3gs_sort_status) the last kernel of the call replaces the count in *total_dev and *total_host by
 * D3GS_COUNT_SORT_GAVE_UP, so a caller that checks the count for a negative value never takes a mis-sorted list
 * for a result.  Workspace sizes as for the single calls
 * (d3gs_sort_workspace_bytes(n, 0, d3gs_depth_key_bits(p)), d3gs_scan_gathered_workspace_bytes(n),
 * d3gs_sort_workspace_bytes(capacity, 0, d3gs_higher_msb(tiles))).  flags: D3GS_BIN_WORKSPACES_ARE_ZERO says the
 * caller has cleared all three.  With D3GS_BIN_HOST_COUNT_AT_END *total_host is written once, by the last kernel
 * of the call (it needs tile_order != NULL or a workspace to run), with the count or the status in its place, as
 * a system-scope release store: a caller that sets the word to D3GS_COUNT_PENDING before the call can poll it
 * from the host while the stream runs on, where waiting on an event would put a marker into the stream ahead of
 * the kernels that follow.  With D3GS_BIN_KEYS_16BIT (at most 2^16 tiles in the call) the pair keys are 16-bit tile
 * ids: tile_keys_a / tile_keys_b are then read and written as uint16[capacity] (the front half of the buffers) and
 * the sorted keys are found there in that form; the sorted gaussian indices, the ranges and the order are the same.
 * workload_ranges must be zero on entry. */
#define D3GS_BIN_WORKSPACES_ARE_ZERO 1
#define D3GS_BIN_HOST_COUNT_AT_END 2
#define D3GS_BIN_KEYS_16BIT 4
int d3gs_bin_pairs(const d3gs_params* p, const int32_t* radii, const float* uvs, const float* conic_opacity,
                   const float* depths, const int32_t* tiles_touched, const uint64_t* tile_masks,
                   uint32_t* depth_keys_a, uint32_t* depth_keys_b, int32_t* order_a, int32_t* order_b,
                   void* depth_sort_ws, size_t depth_sort_ws_bytes, int32_t* offsets, void* scan_ws,
                   size_t scan_ws_bytes, int64_t* total_dev, int64_t* total_host, int64_t capacity,
                   uint32_t* tile_keys_a, uint32_t* tile_keys_b, int32_t* idx_a, int32_t* idx_b, void* pair_sort_ws,
                   size_t pair_sort_ws_bytes, int32_t* workload_ranges, int32_t* tile_order,
                   int32_t flags, int32_t* order_in_b, int32_t* pairs_in_b, d3gs_stream_t stream);

/* K6 — replaces kernel_raw("rasterize_False_...") at render.py:1434-1464, 2304-2309.
 * color [H,W,C] (or [C,H,W] when p->use_nchw), C = 3 + p->render_rgba; final_T [H,W], n_contrib [H,W].
 * depths [N] (K1's output) and final_depth [H,W] are read / written only when p->render_depth and may be
 * NULL otherwise.  In inference the depth is divided by the accumulated opacity, which makes it NaN (0/0)
 * for a pixel nothing reached, as in the reference (render.py:2244-2250).
 * clear_ptr (may be NULL; no counterpart in the reference): clear_bytes of device memory, both multiples of
 * 16, that the kernel sets to zero while it runs -- meant for the arrays the backward pass accumulates into
 * (grad_records, and the gradient arrays handed to d3gs_preprocess_bwd with outputs_are_zero): the blend is
 * bound by arithmetic and leaves the memory pipes idle, so the clear costs nothing here.
 * conic_opacity may hold any conic: the kernels' staging cull (bounding box and per-patch minimum of the quadratic
 * form) only acts on positive definite ones and leaves the rest to the exact per-pixel sequence.  What is asked
 * for is that power = -1/2 (a dx^2 + c dy^2) - b dx dy stays below 80 at every pixel of a tile that lists the
 * gaussian (the blend's exp has no overflow guard); every positive semi-definite conic satisfies it, K1 writes no
 * other.  The same holds for d3gs_blend_bwd. */
int d3gs_blend_fwd(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                   const float* uvs, const float* conic_opacity, const float* rgb_gaussian, const float* depths,
                   const int32_t* tile_order /* from d3gs_tile_ranges, or NULL for raster order */, float* color,
                   float* final_T, int32_t* n_contrib, float* final_depth, void* clear_ptr, size_t clear_bytes,
                   d3gs_stream_t stream);

/* Per-gaussian gradient record written by K7 and read by K9: one 64-byte line per gaussian so that
 * the sixteen lanes flushing one gaussian issue a single line-wide atomic request.  The reference keeps
 * four separate tensors (duv [N,2], dconic [N,3], dopacity [N], dcolor [N,3], render.py:1388-1411) and dz;
 * they are the strided slices below of this buffer. */
#define D3GS_GRAD_RECORD_FLOATS 16
#define D3GS_GRAD_DUV 0      /* 2 floats */
#define D3GS_GRAD_DCONIC 2   /* 3 floats */
#define D3GS_GRAD_DOPACITY 5 /* 1 float  */
#define D3GS_GRAD_DCOLOR 6   /* 3 floats */
#define D3GS_GRAD_DZ 9       /* 1 float, written with p->render_depth */

/* K7 — replaces kernel_raw("rasterize_True_...") (same generator, grad != None,
 * render.py:1341, 1589-1676, 1774-2210).  Produces the complete gradient (the
 * reference's backward_reduction_balanced_factor <= 0 branch, render.py:2024-2050,
 * 2182-2210).  grad_records [N][D3GS_GRAD_RECORD_FLOATS] is accumulated with
 * atomics: zero-fill it first.  drgb has the layout of color; final_depth /
 * ddepth [H,W] may be NULL without p->render_depth.
 * touched (uint8[N], may be NULL; no counterpart in the reference): set to 1 for every gaussian whose record
 * received a non-zero value; zero-fill it with the records.  d3gs_preprocess_bwd takes it to find the gaussians
 * with work without reading all records. */
int d3gs_blend_bwd(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                   const float* uvs, const float* conic_opacity, const float* rgb_gaussian, const float* depths,
                   const int32_t* tile_order, const float* final_T, const int32_t* n_contrib, const float* color,
                   const float* final_depth, const float* drgb, const float* dT, const float* ddepth,
                   float* grad_records, uint8_t* touched, d3gs_stream_t stream);

/* Custom feature channels (render.py:241-246, 1536-1538, 1571-1573, 1718-1721, 1892-1895, 1920-1923, 1952-1955,
 * 1969-1972, 2113-2117, 2268-2270; the reference compiles the channel count into its rasterize kernel): features
 * [items][num_features] are blended like a colour over the lists of a finished forward pass.
 *   d3gs_blend_features_fwd   feature_image [B][H][W][num_features] = sum_i T_i alpha_i f_i, the raw sums (no
 *                             background, no clamp), with the weights of d3gs_blend_fwd pixel for pixel; up to 16
 *                             channels per launch.
 *   d3gs_blend_features_bwd   given n_contrib of the forward pass, the blended feature_image and its gradient
 *                             dfeature_image: adds the channels' share of the geometry gradient to columns 0..5 of
 *                             grad_records (D3GS_GRAD_DUV, _DCONIC, _DOPACITY: the records d3gs_blend_bwd adds the
 *                             colour's share to, in either order), marks `touched` (may be NULL) like d3gs_blend_bwd,
 *                             and adds dL/dfeatures to dfeatures [items][num_features] (zero-fill it first); up to
 *                             14 channels per launch, their terms of dL/dalpha summed before the one division by
 *                             1 - alpha (render.py:1952-1955).
 * p: the fields the blend reads (sizes, tiles, alpha_eps, transmittance_eps, batch); num_features = 0 does nothing. */
int d3gs_blend_features_fwd(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                            const float* uvs, const float* conic_opacity, const float* features, int32_t num_features,
                            const int32_t* tile_order, float* feature_image, d3gs_stream_t stream);
int d3gs_blend_features_bwd(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                            const float* uvs, const float* conic_opacity, const float* features, int32_t num_features,
                            const int32_t* tile_order, const int32_t* n_contrib, const float* feature_image,
                            const float* dfeature_image, float* grad_records, float* dfeatures, uint8_t* touched,
                            d3gs_stream_t stream);

/* The per-gaussian backward, config rasterize_backward_algo = PER_GAUSSIAN (config_def.py:72-74, 149-151;
 * render.py:940-962, 1577-1583, 1744-1759, 2319-2776): a second algorithm for K7's gradient in which lanes are
 * gaussians and pixels pass through them, so that no sum crosses lanes.  Three calls:
 *   d3gs_bucket_offsets (K8, replaces kernel_1d("prepare_bucket_...") + cumsum_, render.py:941-950):
 *     bucket_offsets[t] = sum over tiles before t of ceil(list length / D3GS_BUCKET_SIZE), [num_tiles + 1] int32,
 *     the last entry the total; no host read-back is needed: ceil(M / D3GS_BUCKET_SIZE) + num_tiles bounds the total;
 *   d3gs_blend_fwd_snapshots: d3gs_blend_fwd (same arguments, same image bit for bit) that also stores every pixel's
 *     running state in front of each bucket: snapshots [total buckets][256][d3gs_snapshot_floats(p)] float32, pixel
 *     order of the kernel's threads: (T, accumulated r, g, b) and, with render_depth or render_rgba, a second quad
 *     (accumulated alpha, accumulated depth, 0, 0) -- the reference's T_snap / color_snap and their depth / alpha
 *     companions (render.py:958-959, 1744-1759, 2412-2415);
 *   d3gs_blend_bwd_per_gaussian: the backward over those snapshots; arguments as d3gs_blend_bwd (depth, RGBA and
 *     NCHW included, render.py:2364-2398, 2490-2528).  One wavefront per bucket of 64 list entries (the reference:
 *     one 32-lane warp per 32), one workgroup per tile.
 * The gradient is the complete one, as d3gs_blend_bwd's, up to the order of the float32 sums. */
#define D3GS_BUCKET_SIZE 64
int d3gs_bucket_offsets(const int32_t* workload_ranges, int32_t num_tiles, int32_t* bucket_offsets, d3gs_stream_t stream);
int d3gs_snapshot_floats(const d3gs_params* p);      /* 4, or 8 with render_depth / render_rgba */
int d3gs_blend_fwd_snapshots(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                             const float* uvs, const float* conic_opacity, const float* rgb_gaussian,
                             const float* depths, const int32_t* tile_order, float* color, float* final_T,
                             int32_t* n_contrib, float* final_depth, void* clear_ptr, size_t clear_bytes,
                             const int32_t* bucket_offsets, float* snapshots, d3gs_stream_t stream);
int d3gs_blend_bwd_per_gaussian(const d3gs_params* p, const int32_t* workload_ranges, const int32_t* gaussian_idx_sorted,
                                const float* uvs, const float* conic_opacity, const float* rgb_gaussian,
                                const float* depths, const int32_t* tile_order, const float* final_T,
                                const int32_t* n_contrib, const float* color, const float* final_depth,
                                const float* drgb, const float* dT, const float* ddepth,
                                const int32_t* bucket_offsets, const float* snapshots, float* grad_records,
                                uint8_t* touched, d3gs_stream_t stream);

/* K9 — replaces kernel_1d("gs3d_preprocess_bwd_...") at render.py:2922-3369
 * (body 3217-3356).  Chain rule from K7's records (duv, dconic, dopacity, dcolor
 * [, dz]) to the raw model tensors, including the fused activation gradients.
 * Gradients of gaussians with radii == 0, and of gaussians whose record is all
 * zero (in no tile list, or never reached before their pixels saturated), are
 * zeros; nothing but the record is read for them.  outputs_are_zero != 0 (no
 * counterpart in the reference) says the caller has cleared the six gradient
 * arrays beforehand: those zeros are then not written again.  touched (uint8[N],
 * may be NULL; no counterpart in the reference) is d3gs_blend_bwd's array of the
 * same name: gaussians it marks 0 are taken to have an all-zero record, which is
 * then not read.  The *_base pointers may be NULL.  sh_mask_compat != 0 reads the SH clamp mask with the
 * reference's reversed bit order (render.py:3344-3350).
 * A bundle (p->batch_size = B > 1) goes through in this one launch, as in the reference, whose kernel loops over
 * the batch (render.py:2972-2989, 3180-3219): the per-item arrays (radii, cov2d_vecs, sh_to_rgb_ne_0, grad_records,
 * touched) hold B * n rows, camera after camera, `instances` the B tables K1 was given, and each workgroup works
 * its gaussians off camera by camera, adding every camera's gradient to what it stored for those before. */
int d3gs_preprocess_bwd(const d3gs_params* p, const float* xyz, const float* quaternion_xyzw, const float* scale,
                        const float* opacity, const float* color_sh, const int32_t* radii, const float* cov2d_vecs,
                        const uint8_t* sh_to_rgb_ne_0, const float* grad_records, const uint8_t* touched,
                        int32_t sh_mask_compat, int32_t outputs_are_zero, float* dxyz, float* dquaternion_xyzw, float* dscale,
                        float* dopacity_out, float* dcolor_sh, float* dcolor_sh_base, const d3gs_instances* instances,
                        d3gs_stream_t stream);

/* K9 for one camera of a bundle (render.py:2972-2989, 3180-3219 loop over the batch inside the kernel): with
 * p->batch_size = B > 1 the call works on camera batch_index, taken from p->batch_cameras, and every per-item
 * array (radii, cov2d_vecs, sh_to_rgb_ne_0, grad_records, touched) points at that camera's n rows.  accumulate != 0
 * adds to the six gradient arrays instead of storing (gaussians without work are left alone): the gradient of a
 * bundle is then B calls, the first storing (or adding to cleared arrays), the others accumulating (what
 * d3gs_preprocess_bwd does for a bundle inside one launch; this entry serves callers that hold the cameras' arrays
 * apart, or that add a camera to gradients they already have).  With
 * batch_size <= 1, batch_index 0 and accumulate 0 this is d3gs_preprocess_bwd.  `instances` is the table of this
 * camera alone ([num_instances][12], the batch_index-th of the B tables K1 was given). */
int d3gs_preprocess_bwd_camera(const d3gs_params* p, int32_t batch_index, int32_t accumulate, const float* xyz,
                               const float* quaternion_xyzw, const float* scale, const float* opacity,
                               const float* color_sh, const int32_t* radii, const float* cov2d_vecs,
                               const uint8_t* sh_to_rgb_ne_0, const float* grad_records, const uint8_t* touched,
                               int32_t sh_mask_compat, int32_t outputs_are_zero, float* dxyz, float* dquaternion_xyzw,
                               float* dscale, float* dopacity_out, float* dcolor_sh, float* dcolor_sh_base,
                               const d3gs_instances* instances, d3gs_stream_t stream);

/* Sparse mode (config sparse_mode, config_def.py:119; render.py:234-238, 478-500, 622-640, 753, 2857-2866,
 * 3185-3213): everything after K1 works on the accepted render items only, stored compactly -- for scenes of which
 * a view sees a small part.  The reference counts the accepted items with a first launch of K1
 * (block_reduce + atomicAdd, render.py:480-486), reads the count back, and lets a second launch take slots from an
 * atomic counter (render.py:490-495).  Here:
 *   1. d3gs_preprocess_fwd_sparse with valid_flags [items] (slot_scan = NULL): 1 where the item is accepted;
 *   2. the caller scans the flags (d3gs_scan_gathered with index = NULL; its total is the accepted count V, which the
 *      caller needs on the host to size the compact buffers, as the reference does);
 *   3. d3gs_preprocess_fwd_sparse with slot_scan (valid_flags = NULL): outputs [V] in ascending item order,
 *      sparse_gaussian_ids [V] and sparse_batch_ids [V] say which gaussian and camera each slot holds (the
 *      reference's sparse_gaussian_id / sparse_batch_id; its slot order is whatever the atomic gives);
 *   4. d3gs_sh_colors_sparse for the colours, then the binning and blend entry points with params whose n = V
 *      (they only index per-item arrays), then
 *   5. d3gs_preprocess_bwd_sparse: K9 over the V items; gradients are written per item, [V] rows (the rows of the
 *      model arrays are found through sparse_gaussian_ids), as the reference's sparse gradient (render.py:2918).
 * The render is the dense one bit for bit: slots ascend with the item index, so ties in the sort fall the same way.
 * `instances` (may be NULL) as in the dense entry points: instance ids are per row of the model arrays.
 * A bundle of B cameras in one pass: steps 1-3 run over the B * n items (p->batch_size = B); behind them the
 * params carry n = V, batch_size = B (the tile ids and images keep the camera) and compact_items = V;
 * d3gs_preprocess_bwd_sparse then takes sparse_batch_ids (NULL for one camera) to give each row its camera. */
int d3gs_preprocess_fwd_sparse(const d3gs_params* p, const float* xyz, const float* quaternion_xyzw, const float* scale,
                               const float* opacity, const uint8_t* invalid_mask, int32_t* valid_flags,
                               const int32_t* slot_scan, int32_t* sparse_gaussian_ids, int32_t* sparse_batch_ids,
                               float* depths, int32_t* radii, float* uvs, float* conic_opacity, int32_t* tiles_touched,
                               float* cov2d_vecs, uint64_t* tile_masks, uint32_t* depth_sort_keys,
                               const d3gs_instances* instances, d3gs_stream_t stream);
int d3gs_sh_colors_sparse(const d3gs_params* p, const int32_t* sparse_gaussian_ids, const int32_t* sparse_batch_ids,
                          int32_t count, const float* xyz, const float* color_sh, const float* color_sh_base,
                          const int32_t* radii, float* rgb_gaussian, uint8_t* sh_to_rgb_ne_0,
                          const d3gs_instances* instances, d3gs_stream_t stream);
int d3gs_preprocess_bwd_sparse(const d3gs_params* p /* n = V */, const int32_t* sparse_gaussian_ids, const float* xyz,
                               const float* quaternion_xyzw, const float* scale, const float* opacity,
                               const float* color_sh, const int32_t* radii, const float* cov2d_vecs,
                               const uint8_t* sh_to_rgb_ne_0, const float* grad_records, const uint8_t* touched,
                               int32_t sh_mask_compat, int32_t outputs_are_zero, float* dxyz, float* dquaternion_xyzw,
                               float* dscale, float* dopacity_out, float* dcolor_sh, float* dcolor_sh_base,
                               const d3gs_instances* instances, const int32_t* sparse_batch_ids, d3gs_stream_t stream);

/* K10 -- replaces the hash-table deduplication of a sparse bundle's gradient rows (render.py:2864-2903: insert the
 * accepted gaussian ids of all cameras, collect the distinct ones, query each row's slot, add the rows with atomics).
 * d3gs_unique_ids: ids [count] (each in [0, id_limit)) -> the distinct ids in ascending order (unique_ids, the
 * first *unique_count_dev entries of a [count] buffer), for every input row the index of its id in that list
 * (inverse [count]), and the rows grouped by id: run_rows [count] lists the input rows sorted by id (rows of equal
 * id in input order), run_starts [count + 1] where each id's run begins in it (run_starts[unique] = count).
 * Built from the library's radix sort (value = row) and scan; the count also goes to unique_count_host (pinned
 * host word, may be NULL) as in d3gs_scan_gathered.  workspace: d3gs_unique_ids_workspace_bytes, 256-byte aligned,
 * need not be cleared.
 * d3gs_merge_rows: merged[u][c] = sum of rows[r][c] over the rows r of run u, added in run order by one thread per
 * (u, c): no atomics, so the sums do not depend on scheduling.  rows [n_rows][width], merged [n_runs][width]. */
int d3gs_unique_ids_workspace_bytes(int32_t count, int32_t id_limit, size_t* bytes_out_host);
int d3gs_unique_ids(const int32_t* ids, int32_t count, int32_t id_limit, int32_t* unique_ids, int32_t* inverse,
                    int32_t* run_rows, int32_t* run_starts, void* workspace, size_t workspace_bytes,
                    int64_t* unique_count_dev, int64_t* unique_count_host, d3gs_stream_t stream);
int d3gs_merge_rows(const float* rows, int32_t n_rows, int32_t width, const int32_t* run_rows,
                    const int32_t* run_starts, int32_t n_runs, float* merged, d3gs_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* D3GS_HIP_H_ */
