// Tile binning: prefix scan of per-gaussian tile counts, (tile, depth) key
// expansion, stable LSD radix sort of (u64 key, i32 value) pairs, and tile-range
// extraction (the radix sort itself lives in radix_sort.hip).  All stages are
// HBM-bandwidth-bound integer work.
//
// Reference: d3sim/algos/d3gs/render.py:694-695 (cumsum), 739-840 (keys),
// 845-887 + d3sim/csrc/devsort.py:38-149 (CUB radix sort), 896-939 (ranges).
#include <mutex>

#include "device_math.h"

namespace d3gs {

// ---------------------------------------------------------------------------
// Inclusive scan, int32, three phases (chunk sums -> scan of sums -> chunk scan).
// ---------------------------------------------------------------------------
constexpr int kScanItems = 8;                      // per thread
constexpr int kScanChunk = kBlock * kScanItems;    // 2048 per block

__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        int t = __shfl_up(v, off, 64);
        if (lane >= off) v += t;
    }
    return v;
}

// block-wide exclusive scan of one int per thread; returns exclusive prefix and the block total
__device__ __forceinline__ int block_excl_scan(int v, int& total, int* smem /* >= 4 ints */) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int incl = wave_incl_scan(v, lane);
    if (lane == 63) smem[wave] = incl;
    __syncthreads();
    int w0 = smem[0], w1 = smem[1], w2 = smem[2], w3 = smem[3];
    __syncthreads();
    int base = (wave > 0 ? w0 : 0) + (wave > 1 ? w1 : 0) + (wave > 2 ? w2 : 0);
    total = w0 + w1 + w2 + w3;
    return base + incl - v;
}

__global__ __launch_bounds__(kBlock) void scan_chunk_sums_kernel(const int32_t* __restrict__ in, int n,
                                                                  int32_t* __restrict__ sums) {
    __shared__ int smem[4];
    const int base = blockIdx.x * kScanChunk + threadIdx.x * kScanItems;
    int s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) s += (base + k < n) ? in[base + k] : 0;
    int total;
    block_excl_scan(s, total, smem);
    if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// single block: exclusive scan of `sums` in place (int32), grand total as int64
__global__ __launch_bounds__(kBlock) void scan_sums_kernel(int32_t* __restrict__ sums, int nchunks,
                                                            int64_t* __restrict__ total_out) {
    __shared__ int smem[4];
    long long carry = 0;
    for (int start = 0; start < nchunks; start += kBlock) {
        int idx = start + threadIdx.x;
        int v = idx < nchunks ? sums[idx] : 0;
        int total;
        int ex = block_excl_scan(v, total, smem);
        if (idx < nchunks) sums[idx] = (int)(carry + ex);
        carry += total;
    }
    if (threadIdx.x == 0 && total_out) *total_out = carry;
}

__global__ __launch_bounds__(kBlock) void scan_apply_kernel(int32_t* __restrict__ data, int n,
                                                             const int32_t* __restrict__ chunk_prefix) {
    __shared__ int smem[4];
    const int base = blockIdx.x * kScanChunk + threadIdx.x * kScanItems;
    int v[kScanItems];
    int s = 0;
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        v[k] = (base + k < n) ? data[base + k] : 0;
        s += v[k];
    }
    int total;
    int ex = block_excl_scan(s, total, smem) + chunk_prefix[blockIdx.x];
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
        ex += v[k];
        if (base + k < n) data[base + k] = ex;
    }
}

// ---------------------------------------------------------------------------
// Gather + inclusive scan in one launch: out[j] = sum_{i <= j} src[index[i]].
// Each workgroup takes the chunk of 4096 with its own id, publishes its sum (aggregate), walks back
// over its predecessors' status words until one that already knows its inclusive
// prefix, and publishes its own.  Status word: flag in bits 62-63, value below.
// Polling is bounded: past the limit the workgroup raises the error word and goes
// on, and the grand total is reported as -1.
// ---------------------------------------------------------------------------
constexpr unsigned long long kScanAggregate = 1ull << 62, kScanPrefix = 2ull << 62, kScanValueMask = (1ull << 62) - 1ull;
constexpr int kScanSpinLimit = 1 << 22;
constexpr int kScanLookRounds = 4;

// few items per thread: the gather is a dependent random read, and it is the number of wavefronts in flight
// that hides its latency.  4096-element chunks: as fast as 2048-element ones on a million gaussians (0.022 ms), a
// fifth faster on three million (0.069 against 0.086 ms), where the gathered array no longer fits an XCD's L2 and
// every wavefront's gather pulls in 64 lines; 8192 is slower on both, 1024 was slower on the first.
constexpr int kGatherScanItems = 4;
constexpr int kGatherScanBlock = 1024;
constexpr int kGatherScanWaves = kGatherScanBlock / 64;
constexpr int kGatherScanChunk = kGatherScanBlock * kGatherScanItems;

struct ScanWorkspace {
    unsigned long long* status;  // [chunks]
    uint32_t* error;             // [1]
};

__device__ __forceinline__ long long wave_sum_i64(long long v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__global__ __launch_bounds__(kGatherScanBlock) void scan_gather_lookback_kernel(const int32_t* __restrict__ src, int src_n,
                                                                       const int32_t* __restrict__ index, int n,
                                                                       int32_t* __restrict__ out, ScanWorkspace ws,
                                                                       int64_t* __restrict__ total_out,
                                                                       int64_t* __restrict__ total_host) {
    __shared__ int s_wave[kGatherScanWaves];
    __shared__ long long s_prefix;
    // Chunk = workgroup id.  Workgroups of a 1-D grid are dispatched in id order (per XCD, which gets every
    // 8th id), so every chunk this one waits on has been dispatched before it and finishes without help; an
    // atomic ticket would put one chip-wide same-address atomic per workgroup (about 15 ns each, one after the
    // other) in front of the launch.
    const int chunk = blockIdx.x;
    const int base = chunk * kGatherScanChunk + threadIdx.x * kGatherScanItems;
    // every index first, then every gather: two trips to memory, not one per item after the other (positions past
    // the end take position 0's index and count nothing)
    int v[kGatherScanItems], at[kGatherScanItems];
#pragma unroll
    for (int k = 0; k < kGatherScanItems; ++k) {
        const int j = base + k < n ? base + k : 0;
        at[k] = index ? index[j] : j;
    }
    int s = 0;
#pragma unroll
    for (int k = 0; k < kGatherScanItems; ++k) {
        // a corrupt index must not become a wild read
        const bool ok = (unsigned)at[k] < (unsigned)src_n;      // (false throughout for an empty source)
        const int x = src_n > 0 ? src[ok ? at[k] : 0] : 0;
        v[k] = (ok && base + k < n) ? x : 0;
        s += v[k];
    }
    // exclusive scan of s over the workgroup
    const int wlane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int incl = wave_incl_scan(s, wlane);
    if (wlane == 63) s_wave[wave] = incl;
    __syncthreads();
    int wave_base = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kGatherScanWaves; ++w) {
        const int c = s_wave[w];
        if (w < wave) wave_base += c;
        total += c;
    }
    int ex = wave_base + incl - s;
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        if (lane == 0)
            __hip_atomic_store(ws.status + chunk, (chunk == 0 ? kScanPrefix : kScanAggregate) | (unsigned long long)total,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        long long prefix = 0;
        if (chunk > 0) {
            // lane l polls chunks pos - l - 64 r for r = 0 .. 3 with independent loads: 256 predecessors per
            // round trip to memory, taken 64 at a time from the nearest on
            int pos = chunk - 1;
            int spins = 0;
            bool walking = true;
            while (walking) {
                unsigned long long w[kScanLookRounds];
#pragma unroll
                for (int r = 0; r < kScanLookRounds; ++r) {
                    const int t = pos - lane - 64 * r;
                    w[r] = t >= 0 ? __hip_atomic_load(ws.status + t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                  : kScanPrefix;   // before the first chunk: an empty prefix
                }
                int taken = 0;
#pragma unroll
                for (int r = 0; r < kScanLookRounds; ++r) {
                    if (!walking || taken != 64 * r) continue;    // an earlier group stopped short
                    const unsigned long long flag = w[r] & ~kScanValueMask;
                    const unsigned long long not_ready = __ballot(flag == 0ull), is_prefix = __ballot(flag == kScanPrefix);
                    const int first_nr = not_ready ? __builtin_ctzll(not_ready) : 64;
                    const int first_p = is_prefix ? __builtin_ctzll(is_prefix) : 64;
                    if (first_p < first_nr) {          // a chunk that knows its inclusive prefix: done
                        prefix += wave_sum_i64(lane <= first_p ? (long long)(w[r] & kScanValueMask) : 0ll);
                        walking = false;
                    } else {                           // a run of aggregates (possibly empty): take them
                        prefix += wave_sum_i64(lane < first_nr ? (long long)(w[r] & kScanValueMask) : 0ll);
                        taken += first_nr;
                    }
                }
                if (!walking) break;
                pos -= taken;
                if (taken > 0) {
                    spins = 0;
                } else if (++spins > kScanSpinLimit) {
                    if (lane == 0) atomicOr(ws.error, 1u);
                    __threadfence();
                    walking = false;
                } else {
                    __builtin_amdgcn_s_sleep(1);
                }
            }
        }
        if (lane == 0) {
            if (chunk > 0)
                __hip_atomic_store(ws.status + chunk, kScanPrefix | ((unsigned long long)(prefix + total) & kScanValueMask),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            s_prefix = prefix;
            if (chunk == (int)gridDim.x - 1) {
                const uint32_t err = __hip_atomic_load(ws.error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                const long long grand = err ? (long long)D3GS_COUNT_SCAN_GAVE_UP : prefix + total;
                if (total_out) *total_out = grand;
                // pinned host memory is mapped into the device's address space: the count reaches the host with
                // this store, and is visible there once the host has waited for the kernel
                if (total_host) *total_host = grand;
            }
        }
    }
    __syncthreads();
    ex += (int)s_prefix;
#pragma unroll
    for (int k = 0; k < kGatherScanItems; ++k) {
        ex += v[k];
        if (base + k < n) out[base + k] = ex;
    }
}

__global__ __launch_bounds__(kBlock) void scan_clear_kernel(uint32_t* __restrict__ words, int count) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < count) words[i] = 0u;
}

// ---------------------------------------------------------------------------
// Key expansion: one thread per gaussian, emits its (tile << 32 | depth bits)
// keys at the offset the scan assigned (render.py:745-840).
// ---------------------------------------------------------------------------
constexpr int kKeyStage = 512;   // pairs a wavefront stages in LDS before writing them out coalesced

// Key = uint64_t: the reference's (tile << 32) | depth bits.  Key = uint32_t: the tile id alone, all the
// pair sort needs once the pairs are emitted in depth order.
template <typename Key>
__global__ __launch_bounds__(kBlock) void make_keys_kernel(const d3gs_params P, const int32_t* __restrict__ radii,
                                                            const float* __restrict__ uvs,
                                                            const float* __restrict__ conic_opacity,
                                                            const float* __restrict__ depths,
                                                            const int32_t* __restrict__ offsets,
                                                            const int32_t* __restrict__ order,
                                                            const uint32_t* __restrict__ ordered_depth_keys,
                                                            const unsigned long long* __restrict__ tile_masks,
                                                            Key* __restrict__ keys, int32_t* __restrict__ vals,
                                                            long long m) {
    __shared__ Key s_key[kBlock / 64][kKeyStage];
    __shared__ int32_t s_val[kBlock / 64][kKeyStage];
    __shared__ int s_start[kBlock / 64][64], s_slot[kBlock / 64][64];
    __shared__ unsigned char s_owner[kBlock / 64][kKeyStage];
    // no early return: every lane takes part in the cooperative emission of large gaussians
    const int j_raw = blockIdx.x * kBlock + threadIdx.x;
    const int items = item_count(P);     // gaussians x cameras of a bundle
    const bool in_range = j_raw < items;
    const int j = in_range ? j_raw : items - 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // slot j of the emission order holds gaussian order[j] (identity without an order table);
    // `offsets` is the inclusive scan of the tile counts taken in that same order
    int i = order ? order[j] : j;
    const bool sane = (unsigned)i < (unsigned)items;
    i = sane ? i : 0;
    const long long end = offsets[j];
    // requested with the loads above, whether it is needed or not (the empty statement keeps the compiler from
    // moving the load behind the test of the lane, where it would wait for a round trip of its own)
    const int before = offsets[j > 0 ? j - 1 : 0];
    asm volatile("" : : "v"(before));
    long long off = !in_range ? end : (j == 0 ? 0 : before);   // lanes past the end: an empty range at the total
    // a gaussian with no tiles has an empty slot range; a caller that passed a smaller buffer than
    // the scan total must never be written past, and offsets that wrapped (a view with more than 2^31 - 1 pairs
    // has negative 32-bit prefix sums) must not be written in front of the buffer either
    const bool active = in_range && sane && off >= 0 && end > off && end <= m;
    const uint32_t dbits = ordered_depth_keys ? ordered_depth_keys[j] : reference_depth_bits(P, depths[i]);
    // the preprocess kernel's record of the kept tiles, when it was asked to write one
    unsigned long long kept = 0ull, meta = 0ull;
    // both words in one 16-byte load, and requested as soon as the gaussian is known: whether the lane has pairs to
    // emit is known a round trip earlier than it is needed here
    if (tile_masks && in_range && sane) {
        const ulonglong2 rec = *reinterpret_cast<const ulonglong2*>(tile_masks + 2 * (size_t)i);
        kept = active ? rec.x : 0ull;
        meta = active ? rec.y : 0ull;
    }
    const bool has_mask = (meta & kTileMaskHas) != 0;
    const bool walk_again = active && !has_mask;
    // The pairs of the wavefront's gaussians that come from masks are assembled in LDS, packed, and leave as
    // coalesced segments: consecutive lanes write consecutive slots, stepping over the runs of the (few, large)
    // gaussians that are walked again below.  Each packed element carries the lane it came from, which gives its
    // slot: the lane's first slot plus the element's place in the lane's run.
    // a mask names at most 64 tiles; the bound keeps the wave's packed total small whatever the offsets hold
    const int my_cnt = (active && has_mask) ? (int)min(end - off, 64ll) : 0;
    int incl = my_cnt;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int t = __shfl_up(incl, d, 64);
        if (lane >= d) incl += t;
    }
    const int start = incl - my_cnt, packed_total = __shfl(incl, 63, 64);
    const long long wave_base = __shfl(off, 0, 64);
    const bool staged = packed_total <= kKeyStage && !__any(in_range && !sane);
    if (staged) {
        s_start[wave][lane] = start;
        s_slot[wave][lane] = (int)(off - wave_base);    // a wavefront's slots span far less than 2^31
        if (has_mask)
            mask_tile_emit(kept, meta, P.tiles_x, dbits, (long long)start, (long long)(start + my_cnt),
                           [&](long long e, uint64_t key) {
                               s_key[wave][e] = sizeof(Key) == 8 ? (Key)key : (Key)(key >> 32);
                               s_val[wave][e] = i;
                               s_owner[wave][e] = (unsigned char)lane;
                           });
        __builtin_amdgcn_wave_barrier();
        for (int e = lane; e < packed_total; e += 64) {
            const int lo = s_owner[wave][e];
            const long long slot = wave_base + s_slot[wave][lo] + (e - s_start[wave][lo]);
            keys[slot] = s_key[wave][e];
            vals[slot] = s_val[wave][e];
        }
    } else if (has_mask) {
        mask_tile_emit(kept, meta, P.tiles_x, dbits, off, end, [&](long long slot, uint64_t key) {
            keys[slot] = sizeof(Key) == 8 ? (Key)key : (Key)(key >> 32);
            vals[slot] = i;
        });
    }
    if (!__any(walk_again)) return;   // wave-uniform
    TileWalk walk = {};
    if (walk_again) {
        const float2 uv = *reinterpret_cast<const float2*>(uvs + 2 * i);
        const float4 co = *reinterpret_cast<const float4*>(conic_opacity + 4 * i);
        TileWalkIn g{uv.x, uv.y, (float)radii[i], co.x, co.y, co.z, co.w};
        walk = tile_walk_setup(P, g);
        // camera b of a bundle owns the tile rows from b * tiles_y on (render.py:787, 809); the per-tile test works
        // in candidate-rect coordinates, so moving the rect's origin leaves the single camera's decisions as they are
        // (with a kept-tile record the shifted origin is in the record: sparse mode's compact rows of a bundle do
        // not say which camera they belong to otherwise)
        const int shift = P.batch_size <= 1 ? 0 : tile_masks ? (int)((meta >> 16) & 0xFFFFu) - walk.bminy
                                                             : (i / P.n) * P.tiles_y;
        walk.bminy += shift;
    }
    wave_tile_emit<Key>(P.filter_algo, walk_again, walk, P.tiles_x, dbits, i, off, end, keys, vals);
}

// Sort keys of the gaussians themselves: the float bits of the depth (positive floats order like
// their bit patterns), value = gaussian index.
__global__ __launch_bounds__(kBlock) void depth_keys_kernel(const float* __restrict__ depths, int n,
                                                             uint64_t* __restrict__ keys, int32_t* __restrict__ idx) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i >= n) return;
    keys[i] = (uint64_t)__float_as_uint(depths[i]);
    idx[i] = i;
}

__global__ __launch_bounds__(kBlock) void gather_i32_kernel(const int32_t* __restrict__ src,
                                                             const int32_t* __restrict__ index, int n, int src_n,
                                                             int32_t* __restrict__ dst) {
    const int j = blockIdx.x * kBlock + threadIdx.x;
    if (j >= n) return;
    const int i = index[j];
    dst[j] = (unsigned)i < (unsigned)src_n ? src[i] : 0;
}

// ---------------------------------------------------------------------------
// Tile ranges (render.py:897-939)
// ---------------------------------------------------------------------------
template <typename Key>
__device__ __forceinline__ uint32_t key_tile(Key k) {
    if constexpr (sizeof(Key) == 8) return (uint32_t)(k >> 32);
    else return (uint32_t)k;
}

// consecutive keys per thread: one 16-byte load (four 32-bit keys, eight 16-bit ones)
template <typename Key> constexpr int range_items() { return sizeof(Key) == 2 ? 8 : 4; }

template <typename Key>
__global__ __launch_bounds__(kBlock) void tile_ranges_kernel(const Key* __restrict__ keys, long long m,
                                                              const long long* __restrict__ m_device,
                                                              int32_t* __restrict__ ranges, int num_tiles) {
    constexpr int kRangeItems = range_items<Key>();
    if (m_device) m = min(m, max(*m_device, 0ll));   // m is then the capacity of the key buffer
    const long long i0 = ((long long)blockIdx.x * kBlock + threadIdx.x) * kRangeItems;
    if (i0 >= m) return;
    const Key before = keys[i0 > 0 ? i0 - 1 : 0];     // (requested together with the thread's own keys)
    Key k[kRangeItems];
    if (i0 + kRangeItems <= m) {
        if constexpr (sizeof(Key) == 4) {
            const uint4 v = *reinterpret_cast<const uint4*>(keys + i0);   // i0 is a multiple of 4
            k[0] = v.x; k[1] = v.y; k[2] = v.z; k[3] = v.w;
        } else if constexpr (sizeof(Key) == 2) {
            const uint4 v = *reinterpret_cast<const uint4*>(keys + i0);   // i0 is a multiple of 8
            const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                k[2 * j] = (Key)(w[j] & 0xFFFFu);
                k[2 * j + 1] = (Key)(w[j] >> 16);
            }
        } else {
#pragma unroll
            for (int j = 0; j < kRangeItems; ++j) k[j] = keys[i0 + j];
        }
    } else {
#pragma unroll
        for (int j = 0; j < kRangeItems; ++j) k[j] = i0 + j < m ? keys[i0 + j] : (Key)0;
    }
    uint32_t tp = i0 > 0 ? key_tile<Key>(before) : 0u;
#pragma unroll
    for (int j = 0; j < kRangeItems; ++j) {
        const long long i = i0 + j;
        if (i >= m) break;
        const uint32_t t = key_tile<Key>(k[j]);
        if (t < (uint32_t)num_tiles) {   // a corrupt key never writes outside the table
            if (i == 0) {
                ranges[2 * t] = 0;
            } else if (t != tp) {
                if (tp < (uint32_t)num_tiles) ranges[2 * tp + 1] = (int32_t)i;
                ranges[2 * t] = (int32_t)i;
            }
            if (i == m - 1) ranges[2 * t + 1] = (int32_t)m;
        }
        tp = t;
    }
}

// Tile ids ordered by descending list length (counting sort over 1024 length buckets, one workgroup; each
// thread keeps its tiles' lengths in registers and takes its place inside a bucket from the counting atomic's
// return value, so the lists are read once and every tile costs one LDS atomic).  Order inside a bucket is
// arbitrary: the result only steers scheduling.
constexpr int kOrderThreads = 1024, kOrderBuckets = 1024;
constexpr int kOrderPerThread = 8, kOrderPerThreadLarge = 32;    // 8 192 tiles (1080p has 8 160), 32 768 (4K has 32 400)

__device__ __forceinline__ int order_wave_max(int v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = max(v, __shfl_xor(v, off, 64));
    return v;
}

// What a caller reads back in place of the pair count when one of the sorts that built the lists gave up
// a look-back: the error words of the two sort workspaces are folded into the count words (device and
// pinned host) by the last kernel of the binning, so a mis-sorted list never passes for a result.
struct BinStatus {
    const uint32_t* sort_error[2];   // error words of the depth sort and the pair sort (either may be NULL)
    int64_t* total_dev;              // count words to poison (either may be NULL)
    int64_t* total_host;
    // the host word is written here and only here (the count, or the status in its place), by a store that the
    // host sees while the stream runs on: a caller polls the word instead of putting an event into the stream
    bool publish_host;
};

__device__ __forceinline__ void fold_sort_errors(const BinStatus& st) {
    uint32_t err = 0;
#pragma unroll
    for (int k = 0; k < 2; ++k)
        if (st.sort_error[k]) err |= __hip_atomic_load(st.sort_error[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (err && st.total_dev) *st.total_dev = D3GS_COUNT_SORT_GAVE_UP;
    if (st.publish_host) {
        const long long word = err ? (long long)D3GS_COUNT_SORT_GAVE_UP : (st.total_dev ? *st.total_dev : 0ll);
        __hip_atomic_store((long long*)st.total_host, word, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    } else if (err && st.total_host) {
        *st.total_host = D3GS_COUNT_SORT_GAVE_UP;
    }
}

__global__ void bin_status_kernel(BinStatus st) { fold_sort_errors(st); }

template <int kPerThread>
__global__ __launch_bounds__(kOrderThreads) void tile_order_kernel(const int32_t* __restrict__ work, int num_tiles,
                                                                   int32_t* __restrict__ order, BinStatus st) {
    if (threadIdx.x == 0) fold_sort_errors(st);
    __shared__ int s_bin[kOrderBuckets];
    __shared__ int s_wave[kOrderThreads / 64];
    __shared__ int s_max[kOrderThreads / 64];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int2* ranges = reinterpret_cast<const int2*>(work);
    auto amount_of = [&](int t) { const int2 r = ranges[t]; return max(r.y - r.x, 0); };
    auto bucket_of = [&](int a, float scale) { return kOrderBuckets - 1 - min(kOrderBuckets - 1, (int)((float)a * scale)); };
    const bool in_registers = num_tiles <= kOrderThreads * kPerThread;   // else the lists are read three times

    int amount[kPerThread];
    int mx = 0;
    if (in_registers) {
#pragma unroll
        for (int k = 0; k < kPerThread; ++k) {      // (tiles past the end read the last tile: loads without a
            const int t = k * kOrderThreads + tid;  // condition are issued together, conditional ones one by one)
            const int a = amount_of(min(t, num_tiles - 1));
            amount[k] = t < num_tiles ? a : 0;
            mx = max(mx, amount[k]);
        }
    } else {
        for (int t = tid; t < num_tiles; t += kOrderThreads) mx = max(mx, amount_of(t));
    }
    s_bin[tid] = 0;
    mx = order_wave_max(mx);
    if (lane == 0) s_max[wave] = mx;
    __syncthreads();
    mx = 0;
#pragma unroll
    for (int w = 0; w < kOrderThreads / 64; ++w) mx = max(mx, s_max[w]);
    const float scale = (float)kOrderBuckets / ((float)mx + 1.0f);

    int bucket[kPerThread], rank[kPerThread];
    if (in_registers) {
#pragma unroll
        for (int k = 0; k < kPerThread; ++k) {
            bucket[k] = bucket_of(amount[k], scale);
            rank[k] = (k * kOrderThreads + tid < num_tiles) ? atomicAdd(&s_bin[bucket[k]], 1) : 0;
        }
    } else {
        for (int t = tid; t < num_tiles; t += kOrderThreads) atomicAdd(&s_bin[bucket_of(amount_of(t), scale)], 1);
    }
    __syncthreads();
    // exclusive scan of the bucket counts, one bucket per thread
    const int c = s_bin[tid];
    int incl = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int v = __shfl_up(incl, off, 64);
        if (lane >= off) incl += v;
    }
    if (lane == 63) s_wave[wave] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < wave; ++w) base += s_wave[w];
    s_bin[tid] = base + incl - c;
    __syncthreads();
    if (in_registers) {
#pragma unroll
        for (int k = 0; k < kPerThread; ++k) {
            const int t = k * kOrderThreads + tid;
            if (t < num_tiles) order[s_bin[bucket[k]] + rank[k]] = t;
        }
    } else {
        for (int t = tid; t < num_tiles; t += kOrderThreads)
            order[atomicAdd(&s_bin[bucket_of(amount_of(t), scale)], 1)] = t;
    }
}

static inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
static inline int scan_chunks(long long n) { return (int)((n + kScanChunk - 1) / kScanChunk); }

// workspace for scanning `n` ints: chunk sums
static size_t scan_ws_bytes(long long n) { return align_up((size_t)std::max(1, scan_chunks(n)) * sizeof(int32_t), 256); }

static int launch_scan(int32_t* data, long long n, void* ws, int64_t* total_dev, hipStream_t s) {
    const int nchunks = scan_chunks(n);
    int32_t* sums = (int32_t*)ws;
    hipLaunchKernelGGL(scan_chunk_sums_kernel, dim3(nchunks), dim3(kBlock), 0, s, data, (int)n, sums);
    hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(kBlock), 0, s, sums, nchunks, total_dev);
    hipLaunchKernelGGL(scan_apply_kernel, dim3(nchunks), dim3(kBlock), 0, s, data, (int)n, sums);
    return hipGetLastError() == hipSuccess ? D3GS_OK : D3GS_ERR_LAUNCH;
}

}  // namespace d3gs

using namespace d3gs;

extern "C" int d3gs_scan_workspace_bytes(int32_t n, size_t* bytes_out_host) {
    if (n < 0 || !bytes_out_host) { set_error("d3gs_scan_workspace_bytes: bad argument"); return D3GS_ERR_INVALID_ARGUMENT; }
    *bytes_out_host = scan_ws_bytes(n);
    return D3GS_OK;
}

static inline int gather_scan_chunks(long long n) { return (int)((n + kGatherScanChunk - 1) / kGatherScanChunk); }
static size_t scan_gathered_ws_bytes(long long n) {
    return align_up((size_t)std::max(1, gather_scan_chunks(n)) * sizeof(unsigned long long) + 2 * sizeof(uint32_t), 256);
}

extern "C" int d3gs_scan_gathered_workspace_bytes(int32_t n, size_t* bytes_out_host) {
    if (n < 0 || !bytes_out_host) { set_error("d3gs_scan_gathered_workspace_bytes: bad argument"); return D3GS_ERR_INVALID_ARGUMENT; }
    *bytes_out_host = scan_gathered_ws_bytes(n);
    return D3GS_OK;
}

extern "C" int d3gs_scan_gathered(const int32_t* src, int32_t src_n, const int32_t* index, int32_t n, int32_t* out,
                                  void* workspace, size_t workspace_bytes, int32_t workspace_is_zero, int64_t* total_dev,
                                  int64_t* total_host, d3gs_stream_t stream) {
    if (n < 0 || src_n < 0 || !total_dev) { set_error("d3gs_scan_gathered: bad argument"); return D3GS_ERR_INVALID_ARGUMENT; }
    hipStream_t s = (hipStream_t)stream;
    if (n == 0) {   // total = 0
        hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(kBlock), 0, s, (int32_t*)nullptr, 0, total_dev);
        if (total_host) hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(kBlock), 0, s, (int32_t*)nullptr, 0, total_host);
    } else {
        if (!src || !out || !workspace) { set_error("d3gs_scan_gathered: NULL buffer"); return D3GS_ERR_INVALID_ARGUMENT; }
        if (workspace_bytes < scan_gathered_ws_bytes(n)) {
            set_error("d3gs_scan_gathered: workspace %zu < required %zu", workspace_bytes, scan_gathered_ws_bytes(n));
            return D3GS_ERR_INVALID_ARGUMENT;
        }
        const int nchunks = gather_scan_chunks(n);
        ScanWorkspace ws;
        ws.status = (unsigned long long*)workspace;
        ws.error = (uint32_t*)(ws.status + nchunks);
        if (!workspace_is_zero) {
            const int words = 2 * nchunks + 2;
            hipLaunchKernelGGL(scan_clear_kernel, dim3((words + kBlock - 1) / kBlock), dim3(kBlock), 0, s,
                               (uint32_t*)workspace, words);
        }
        hipLaunchKernelGGL(scan_gather_lookback_kernel, dim3(nchunks), dim3(kGatherScanBlock), 0, s, src, (int)src_n, index, (int)n,
                           out, ws, total_dev, total_host);
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_scan_gathered: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

// ---------------------------------------------------------------------------
// d3gs_scan_gathered for callers that cannot allocate (code under graph capture, serving loops, harnesses that
// forbid hipMalloc): the look-back's status words and error word live in a file-scope device array instead of a
// caller workspace.  Every GPU the library runs on holds its own copy of the array, at its own address, until
// the process ends; the address is resolved once per device, with that device current.
// ---------------------------------------------------------------------------
constexpr int kScratchMaxN = D3GS_SCAN_NOALLOC_MAX_N;
constexpr size_t kScratchBytes =
    ((size_t)((kScratchMaxN + d3gs::kGatherScanChunk - 1) / d3gs::kGatherScanChunk) * sizeof(unsigned long long) +
     2 * sizeof(uint32_t) + 255) / 256 * 256;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

constexpr int kScratchMaxDevices = 64;
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[kScratchMaxDevices] = {};

// Device address of `scratch` on the current device (NULL and an error text on failure).  In host code the
// array's name is only a handle for the runtime: everything that touches the memory goes through this pointer.
static void* scratch_on_current_device(const char* who) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kScratchMaxDevices) {
        set_error("%s: cannot tell the current device (%s)", who, e != hipSuccess ? hipGetErrorString(e) : "index out of range");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !ptr) {
            set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(e));
            return nullptr;
        }
        g_scratch_ptr[dev] = ptr;
    }
    return g_scratch_ptr[dev];
}

extern "C" int d3gs_scan_gathered_noalloc(const int32_t* src, int32_t src_n, const int32_t* index, int32_t n,
                                          int32_t* out, int64_t* total_dev, int64_t* total_host,
                                          d3gs_stream_t stream) {
    if (n < 0 || src_n < 0 || !total_dev) {
        set_error("d3gs_scan_gathered_noalloc: bad argument");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (n > kScratchMaxN) {
        set_error("d3gs_scan_gathered_noalloc: n = %d exceeds the built-in scratch (at most %d elements); use "
                  "d3gs_scan_gathered with a caller workspace", n, kScratchMaxN);
        return D3GS_ERR_WORKSPACE_TOO_SMALL;
    }
    void* ws = scratch_on_current_device("d3gs_scan_gathered_noalloc");
    if (!ws) return D3GS_ERR_LAUNCH;
    // the array keeps the previous call's status words: workspace_is_zero = 0 clears the part this call uses,
    // with a fill kernel (not a memset node) so that the call can be captured in a graph
    return d3gs_scan_gathered(src, src_n, index, n, out, ws, kScratchBytes, /*workspace_is_zero=*/0, total_dev,
                              total_host, stream);
}

extern "C" int d3gs_scan_tiles(int32_t* tiles_touched, int32_t n, void* workspace, size_t workspace_bytes,
                               int64_t* total_dev, d3gs_stream_t stream) {
    if (n < 0 || !total_dev) { set_error("d3gs_scan_tiles: bad argument"); return D3GS_ERR_INVALID_ARGUMENT; }
    if (n == 0) {
        // a one-thread kernel rather than a memset node: safe under stream capture
        hipLaunchKernelGGL(scan_sums_kernel, dim3(1), dim3(kBlock), 0, (hipStream_t)stream, (int32_t*)nullptr, 0,
                           total_dev);
        return D3GS_OK;
    }
    if (!tiles_touched || !workspace) { set_error("d3gs_scan_tiles: NULL buffer"); return D3GS_ERR_INVALID_ARGUMENT; }
    if (workspace_bytes < scan_ws_bytes(n)) {
        set_error("d3gs_scan_tiles: workspace %zu < required %zu", workspace_bytes, scan_ws_bytes(n));
        return D3GS_ERR_WORKSPACE_TOO_SMALL;
    }
    int rc = launch_scan(tiles_touched, n, workspace, total_dev, (hipStream_t)stream);
    if (rc) set_error("d3gs_scan_tiles: launch failed: %s", hipGetErrorString(hipGetLastError()));
    return rc;
}

// keys: (tile << 32) | depth bits; tile_keys / tile_keys16: the tile id alone in 32 or 16 bits.  Exactly one is given.
static int make_keys_impl(const d3gs_params* p, const int32_t* radii, const float* uvs, const float* conic_opacity,
                          const float* depths, const int32_t* offsets, const int32_t* gaussian_order,
                          const uint32_t* ordered_depth_keys, const uint64_t* tile_masks, uint64_t* keys,
                          uint32_t* tile_keys, uint16_t* tile_keys16, int32_t* gaussian_idx, int64_t m,
                          d3gs_stream_t stream) {
    int rc = check_params(p, "d3gs_make_keys");
    if (rc) return rc;
    if (m < 0) { set_error("d3gs_make_keys: m < 0"); return D3GS_ERR_INVALID_ARGUMENT; }
    if (p->n == 0 || m == 0) return D3GS_OK;
    const int given = (keys != nullptr) + (tile_keys != nullptr) + (tile_keys16 != nullptr);
    if (!radii || !uvs || !conic_opacity || !depths || !offsets || given != 1 || !gaussian_idx) {
        set_error("d3gs_make_keys: NULL buffer (exactly one of keys / tile_keys must be given)");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (p->compact_items > 0 && p->batch_size > 1 && !tile_masks) {
        set_error("d3gs_make_keys: the compact rows of a bundle (compact_items) need tile_masks to name their camera");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if ((uintptr_t)tile_masks & 15u) {     // the two words of a gaussian are read as one 16-byte load
        set_error("d3gs_make_keys: tile_masks must be 16-byte aligned");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (tile_keys16 && (long long)p->tiles_x * p->tiles_y * batch_count(*p) > (1ll << 16)) {
        set_error("d3gs_make_keys: 16-bit tile ids need at most 2^16 tiles");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    const dim3 grid((item_count(*p) + kBlock - 1) / kBlock), block(kBlock);
    if (keys)
        hipLaunchKernelGGL(make_keys_kernel<uint64_t>, grid, block, 0, (hipStream_t)stream, *p, radii, uvs, conic_opacity,
                           depths, offsets, gaussian_order, ordered_depth_keys, (const unsigned long long*)tile_masks,
                           keys, gaussian_idx, (long long)m);
    else if (tile_keys)
        hipLaunchKernelGGL(make_keys_kernel<uint32_t>, grid, block, 0, (hipStream_t)stream, *p, radii, uvs, conic_opacity,
                           depths, offsets, gaussian_order, ordered_depth_keys, (const unsigned long long*)tile_masks,
                           tile_keys, gaussian_idx, (long long)m);
    else
        hipLaunchKernelGGL(make_keys_kernel<uint16_t>, grid, block, 0, (hipStream_t)stream, *p, radii, uvs, conic_opacity,
                           depths, offsets, gaussian_order, ordered_depth_keys, (const unsigned long long*)tile_masks,
                           tile_keys16, gaussian_idx, (long long)m);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_make_keys: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_make_keys(const d3gs_params* p, const int32_t* radii, const float* uvs, const float* conic_opacity,
                              const float* depths, const int32_t* offsets, const int32_t* gaussian_order,
                              const uint32_t* ordered_depth_keys, const uint64_t* tile_masks, uint64_t* keys,
                              uint32_t* tile_keys, int32_t* gaussian_idx, int64_t m, d3gs_stream_t stream) {
    return make_keys_impl(p, radii, uvs, conic_opacity, depths, offsets, gaussian_order, ordered_depth_keys, tile_masks,
                          keys, tile_keys, nullptr, gaussian_idx, m, stream);
}

int d3gs::make_tile_keys_u16(const d3gs_params* p, const int32_t* radii, const float* uvs, const float* conic_opacity,
                             const float* depths, const int32_t* offsets, const int32_t* gaussian_order,
                             const uint32_t* ordered_depth_keys, const uint64_t* tile_masks, uint16_t* tile_keys,
                             int32_t* gaussian_idx, int64_t m, d3gs_stream_t stream) {
    return make_keys_impl(p, radii, uvs, conic_opacity, depths, offsets, gaussian_order, ordered_depth_keys, tile_masks,
                          nullptr, nullptr, tile_keys, gaussian_idx, m, stream);
}

extern "C" int d3gs_depth_keys(const float* depths, int32_t n, uint64_t* keys, int32_t* gaussian_idx,
                               d3gs_stream_t stream) {
    if (n < 0) { set_error("d3gs_depth_keys: n < 0"); return D3GS_ERR_INVALID_ARGUMENT; }
    if (n == 0) return D3GS_OK;
    if (!depths || !keys || !gaussian_idx) { set_error("d3gs_depth_keys: NULL buffer"); return D3GS_ERR_INVALID_ARGUMENT; }
    hipLaunchKernelGGL(depth_keys_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, (hipStream_t)stream, depths,
                       (int)n, keys, gaussian_idx);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_depth_keys: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_gather_i32(const int32_t* src, int32_t src_n, const int32_t* index, int32_t n, int32_t* dst,
                               d3gs_stream_t stream) {
    if (n < 0 || src_n < 0) { set_error("d3gs_gather_i32: bad size"); return D3GS_ERR_INVALID_ARGUMENT; }
    if (n == 0) return D3GS_OK;
    if (!src || !index || !dst) { set_error("d3gs_gather_i32: NULL buffer"); return D3GS_ERR_INVALID_ARGUMENT; }
    hipLaunchKernelGGL(gather_i32_kernel, dim3((n + kBlock - 1) / kBlock), dim3(kBlock), 0, (hipStream_t)stream, src,
                       index, (int)n, (int)src_n, dst);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_gather_i32: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

template <typename Key>
static int tile_ranges_impl(const char* who, const Key* keys_sorted, int64_t m, const int64_t* m_device,
                            int32_t* workload_ranges, int32_t num_tiles, int32_t* tile_order, d3gs_stream_t stream,
                            BinStatus status = BinStatus{{nullptr, nullptr}, nullptr, nullptr, false}) {
    const bool report = status.publish_host ||
                        ((status.sort_error[0] || status.sort_error[1]) && (status.total_dev || status.total_host));
    if (m < 0 || num_tiles < 0) { set_error("%s: bad argument", who); return D3GS_ERR_INVALID_ARGUMENT; }
    if ((m > 0 && !keys_sorted) || (num_tiles > 0 && !workload_ranges)) {
        set_error("%s: NULL buffer", who);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (m > 0)
        hipLaunchKernelGGL(tile_ranges_kernel<Key>,
                           dim3((unsigned)((m + (long long)kBlock * range_items<Key>() - 1) / ((long long)kBlock * range_items<Key>()))), dim3(kBlock), 0,
                           (hipStream_t)stream, keys_sorted, (long long)m, (const long long*)m_device, workload_ranges,
                           (int)num_tiles);
    if (tile_order && num_tiles > 0) {
        if (num_tiles <= kOrderThreads * kOrderPerThread)
            hipLaunchKernelGGL(tile_order_kernel<kOrderPerThread>, dim3(1), dim3(kOrderThreads), 0, (hipStream_t)stream,
                               workload_ranges, (int)num_tiles, tile_order, status);
        else
            hipLaunchKernelGGL(tile_order_kernel<kOrderPerThreadLarge>, dim3(1), dim3(kOrderThreads), 0,
                               (hipStream_t)stream, workload_ranges, (int)num_tiles, tile_order, status);
    }
    else if (report)
        hipLaunchKernelGGL(bin_status_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream, status);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", who, hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_tile_ranges(const uint64_t* keys_sorted, int64_t m, int32_t* workload_ranges, int32_t num_tiles,
                                int32_t* tile_order, d3gs_stream_t stream) {
    return tile_ranges_impl<uint64_t>("d3gs_tile_ranges", keys_sorted, m, nullptr, workload_ranges, num_tiles, tile_order,
                                      stream);
}

namespace d3gs {
int tile_ranges_u16_with_status(const uint16_t* tile_keys_sorted, int64_t m, const int64_t* m_device,
                                int32_t* workload_ranges, int32_t num_tiles, int32_t* tile_order,
                                const uint32_t* sort_error_a, const uint32_t* sort_error_b, int64_t* total_dev,
                                int64_t* total_host, bool publish_host, d3gs_stream_t stream) {
    return tile_ranges_impl<uint16_t>("d3gs_bin_pairs (tile ranges)", tile_keys_sorted, m, m_device, workload_ranges,
                                      num_tiles, tile_order, stream,
                                      BinStatus{{sort_error_a, sort_error_b}, total_dev, total_host,
                                                publish_host && total_host != nullptr});
}
int tile_ranges_u32_with_status(const uint32_t* tile_keys_sorted, int64_t m, const int64_t* m_device,
                                int32_t* workload_ranges, int32_t num_tiles, int32_t* tile_order,
                                const uint32_t* sort_error_a, const uint32_t* sort_error_b, int64_t* total_dev,
                                int64_t* total_host, bool publish_host, d3gs_stream_t stream) {
    return tile_ranges_impl<uint32_t>("d3gs_bin_pairs (tile ranges)", tile_keys_sorted, m, m_device, workload_ranges,
                                      num_tiles, tile_order, stream,
                                      BinStatus{{sort_error_a, sort_error_b}, total_dev, total_host,
                                                publish_host && total_host != nullptr});
}
}  // namespace d3gs

extern "C" int d3gs_tile_ranges_u32(const uint32_t* tile_keys_sorted, int64_t m, const int64_t* m_device,
                                    int32_t* workload_ranges, int32_t num_tiles, int32_t* tile_order,
                                    d3gs_stream_t stream) {
    return tile_ranges_impl<uint32_t>("d3gs_tile_ranges_u32", tile_keys_sorted, m, m_device, workload_ranges, num_tiles,
                                      tile_order, stream);
}
