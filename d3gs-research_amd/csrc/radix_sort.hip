// Stable LSD radix sort of (u64 key, i32 value) pairs on a bit range — the gfx950
// replacement of the reference's CUB DeviceRadixSort wrapper
// (d3sim/csrc/devsort.py:38-129, call site d3sim/algos/d3gs/render.py:846-887).
//
// Single-sweep design: one kernel histograms every digit of every pass in one
// read of the keys; then each pass (one 8- or 9-bit digit) is ONE kernel that reads a pair once
// and writes it once (24 B per pair per pass).  A workgroup owns 4096
// consecutive keys, ranks them in LDS, and learns where its digits start in the
// output from the workgroups before it through a decoupled look-back over
// per-(tile, digit) status words instead of a separate scan kernel.
//
// Stability: wave w of a workgroup owns the w-th eighth of the tile and walks it
// 64 keys at a time, so (wave, step, lane) order is input order; the rank of a
// key among equal digits is (keys of earlier waves) + (earlier steps of this
// wave) + (lower lanes of this step, by ballot matching).
//
// Coalescing: ranked pairs are first placed at their tile-local sorted position
// in LDS, then written out by consecutive threads, so equal-digit runs leave as
// contiguous segments.
//
// Look-back protocol: a workgroup's tile is its id, and workgroups are dispatched in
// id order, so a workgroup only ever waits on tiles that started before it.  A status word is 0 (not
// published), bit 30 + this tile's count of the digit (at most kOsTile), or bit 31 + the 31-bit inclusive
// prefix up to this tile; words are read and written with relaxed device-scope atomics.
// Polling is bounded: past the limit the workgroup raises an error flag and
// stops waiting, so the grid always drains.
#include "device_math.h"

namespace d3gs {

constexpr int kOsTile = 4096;  // pairs per workgroup
// Threads per workgroup of a pass: one thread owns one digit, so 9-bit digits take 512 threads (8 keys per thread);
// 7- and 8-bit digits run 256 threads with 16 keys each: half the wavefronts per workgroup lets six workgroups
// instead of four share a CU, which covers the 1500 tiles of a 6M-pair sort in one round of workgroups instead of
// one and a half (pair sort of the benchmark view: 0.121 -> 0.111 ms; with 2048-pair tiles it was slower).
template <int kBits> constexpr int os_threads() { return kBits > 8 ? 512 : 256; }
// Digits are 7, 8 or 9 bits wide: the narrowest width that reaches the fewest passes.  9 saves a pass on 18 or 27
// key bits (the depth keys of the gaussians); 7 costs none on 9 to 14 bits (the tile ids of an image of up to
// 16384 tiles) and makes the ranking one ballot shorter and a digit's run in the output twice as long.
constexpr int kOsMaxRadix = 512;
static inline int os_digit_bits(int begin_bit, int end_bit) {
    const int bits = end_bit - begin_bit;
    const int fewest = (bits + 8) / 9;
    for (int d = 7; d < 9; ++d)
        if ((bits + d - 1) / d == fewest) return d;
    return 9;
}
constexpr int kPeersAndAgree = 0x90;  // v_bitop3 truth table of a & ~(b ^ c): rows (a,b,c) = (1,0,0) and (1,1,1)
constexpr int kIcmpSlt = 40;                                  // "signed less than"
constexpr int kIcmpNe = 33;                                   // LLVM integer predicate "not equal", for lane-mask compares
constexpr uint32_t kFlagAggregate = 1u << 30;               // + a tile's own count, below 2^30
constexpr uint32_t kFlagPrefix = 1u << 31;                  // + an inclusive prefix, below 2^31
constexpr uint32_t kAggregateMask = kFlagAggregate - 1u, kPrefixMask = kFlagPrefix - 1u;
constexpr long long kOsMaxPairs = D3GS_MAX_PAIRS;           // positions and counts stay inside 31 bits
constexpr int kSpinLimit = 1 << 22;
// predecessor tiles polled per look-back step: 4 measured faster than 8, 16, 32 or 64 (0.121 -> 0.112 ms on 6M
// pairs, 0.075 -> 0.071 ms on 1M keys): the polls of a step are issued by every digit's thread, and what a wider
// window saves in steps it costs in loads that come back "not published yet"
constexpr int kLookWindow = 4;

struct SortWorkspace {
    uint32_t* hist;     // [passes][radix] digit totals of the whole input
    uint32_t* error;    // [1] set when a look-back gave up
    uint32_t* status;   // [passes][ntiles][radix]
};

__device__ __forceinline__ int os_wave_incl_scan(int v, int lane) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        int t = __shfl_up(v, off, 64);
        if (lane >= off) v += t;
    }
    return v;
}

// exclusive scan of one int per thread over a workgroup of kWaves wavefronts
template <int kWaves>
__device__ __forceinline__ int os_block_excl_scan(int v, int* smem /* kWaves ints */) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int incl = os_wave_incl_scan(v, lane);
    if (lane == 63) smem[wave] = incl;
    __syncthreads();
    int base = 0;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) base += (w < wave) ? smem[w] : 0;
    __syncthreads();
    return base + incl - v;
}

__global__ __launch_bounds__(kBlock) void os_clear_kernel(uint32_t* __restrict__ p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) p[i] = 0u;
}

// All passes' digit histograms in one read of the keys.  Few, large workgroups: every workgroup
// ends with one global atomic per (pass, digit), and atomics to one address from the whole chip
// serialise, so their number (workgroups x passes x 256) is what has to stay small.  Inside a
// workgroup each group of 8 lanes adds into its own LDS copy of the table, which divides the
// same-address conflicts of skewed digits (the exponent byte of a depth takes a handful of values).
constexpr int kHistThreads = 1024;
constexpr int kHistCopies = 8;
constexpr int kHistMaxBlocks = 256, kHistKeysPerThread = 4;   // 128 workgroups were no faster, 64 slower
template <typename Key, int kBits>
__global__ __launch_bounds__(kHistThreads) void os_hist_kernel(const Key* __restrict__ keys, long long m,
                                                                const long long* __restrict__ m_device,
                                                                int begin_bit, int end_bit, int passes, int copies,
                                                                uint32_t* __restrict__ hist) {
    constexpr int kRadix = 1 << kBits;
    if (m_device) m = min(m, max(*m_device, 0ll));   // m is then the capacity of the buffers
    extern __shared__ uint32_t h[];  // [copies][passes][kRadix]; copies is a power of two
    const int table = passes * kRadix;
    for (int k = threadIdx.x; k < copies * table; k += kHistThreads) h[k] = 0u;
    __syncthreads();
    uint32_t* mine = h + (threadIdx.x & (copies - 1)) * table;
    const long long stride = (long long)gridDim.x * kHistThreads;
    auto count = [&](Key key) {
        for (int p = 0; p < passes; ++p) {
            const int bit = begin_bit + kBits * p;
            const int nb = min(kBits, end_bit - bit);
            atomicAdd(&mine[p * kRadix + ((uint32_t)(key >> bit) & ((1u << nb) - 1u))], 1u);
        }
    };
    // Independent loads in flight per thread: with one, a workgroup per CU waits a memory round trip per key.  The
    // body of the input goes in 16-byte loads, two in flight (the bytes a CU has under way set its rate here);
    // the last few keys, and an input that is not 16-byte aligned, go one key at a time, four in flight.
    long long i = (long long)blockIdx.x * kHistThreads + threadIdx.x;
    if constexpr (sizeof(Key) <= 4) {
        if ((reinterpret_cast<uintptr_t>(keys) & 15u) == 0) {
            constexpr int kPerQuad = 16 / (int)sizeof(Key);       // keys in a 16-byte load: four, or eight 16-bit ones
            const uint4* quads = reinterpret_cast<const uint4*>(keys);
            const long long nq = m / kPerQuad;
            auto count_quad = [&](const uint4& a) {
                if constexpr (sizeof(Key) == 4) {
                    count(a.x); count(a.y); count(a.z); count(a.w);
                } else {
                    count((Key)(a.x & 0xFFFFu)); count((Key)(a.x >> 16)); count((Key)(a.y & 0xFFFFu)); count((Key)(a.y >> 16));
                    count((Key)(a.z & 0xFFFFu)); count((Key)(a.z >> 16)); count((Key)(a.w & 0xFFFFu)); count((Key)(a.w >> 16));
                }
            };
            long long q = i;
            for (; q + stride < nq; q += 2 * stride) {
                const uint4 a = quads[q], b = quads[q + stride];
                count_quad(a);
                count_quad(b);
            }
            for (; q < nq; q += stride) count_quad(quads[q]);
            i += nq * kPerQuad;      // the few keys behind the last whole quad
        }
    }
    for (; i + 3 * stride < m; i += 4 * stride) {
        const Key k0 = keys[i], k1 = keys[i + stride], k2 = keys[i + 2 * stride], k3 = keys[i + 3 * stride];
        count(k0);
        count(k1);
        count(k2);
        count(k3);
    }
    for (; i < m; i += stride) count(keys[i]);
    __syncthreads();
    for (int k = threadIdx.x; k < table; k += kHistThreads) {
        uint32_t c = 0;
        for (int q = 0; q < copies; ++q) c += h[q * table + k];
        if (c) atomicAdd(&hist[k], c);
    }
}

template <typename Key, int kBits>
__global__ __launch_bounds__(os_threads<kBits>()) void os_pass_kernel(const Key* __restrict__ keys_in,
                                                              const int32_t* __restrict__ vals_in,
                                                              Key* __restrict__ keys_out,
                                                              int32_t* __restrict__ vals_out, long long m,
                                                              const long long* __restrict__ m_device, int shift,
                                                              uint32_t mask, int ntiles,
                                                              const uint32_t* __restrict__ hist /* this pass, [radix] */,
                                                              uint32_t* __restrict__ status,
                                                              uint32_t* __restrict__ error) {
    constexpr int kRadix = 1 << kBits;
    constexpr int kOsThreads = os_threads<kBits>(), kOsWaves = kOsThreads / 64, kOsItems = kOsTile / kOsThreads;
    static_assert(kRadix <= kOsThreads && kRadix <= kOsMaxRadix, "one thread owns one digit");
    __shared__ int wave_cnt[kOsWaves][kRadix];  // running, then exclusive-over-waves, per-wave digit counts
    __shared__ int digit_out[kRadix];  // global position of tile-local sorted index 0, per digit (m < 2^31)
    __shared__ Key s_keys[kOsTile];
    __shared__ uint16_t s_src[kOsTile];  // tile-local input index of the pair at each sorted position
    __shared__ int s_scan[kOsWaves];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    for (int k = tid; k < kOsWaves * kRadix; k += kOsThreads) (&wave_cnt[0][0])[k] = 0;
    __syncthreads();
    // Tile = workgroup id.  Workgroups of a 1-D grid are dispatched in id order (per XCD, which gets
    // every 8th id), so every tile this one waits on has been dispatched before it; an atomic ticket
    // would add one chip-wide same-address atomic per workgroup to the start of every pass.
    const int tile = blockIdx.x;
    if (tile >= ntiles) return;
    // with a device-side count the grid covers the buffers' capacity: tiles past the count hold no pair,
    // nobody looks back at them, and they leave at once
    if (m_device) m = min(m, max(*m_device, 0ll));
    if ((long long)tile * kOsTile >= m) return;

    const long long tile_begin = (long long)tile * kOsTile;
    const int wave_begin = wave * (kOsTile / kOsWaves);
    Key key[kOsItems];
    int rank[kOsItems];
    const uint64_t lt_mask = (1ull << lane) - 1ull;
#pragma unroll
    for (int k = 0; k < kOsItems; ++k) {
        const long long idx = tile_begin + wave_begin + k * 64 + lane;
        const bool in = idx < m;
        key[k] = in ? keys_in[idx] : (Key)~(Key)0;
    }
    // pairs of the input from this lane's first one on, as far as it matters (a tile holds fewer than 2^16)
    const int left = (int)min(m - (tile_begin + wave_begin + lane), (long long)kOsTile);
#pragma unroll
    for (int k = 0; k < kOsItems; ++k) {
        const bool in = k * 64 < left;
        const uint32_t d = (uint32_t)(key[k] >> shift) & mask;
        // lanes whose digit equals this lane's: per bit, the lanes that agree with this lane on it.  The bit is
        // extracted as 0 / -1, which serves as the ballot's operand and as the mask that turns the ballot
        // into "agrees with me" (one three-input bit operation per half).
        const uint64_t live = __builtin_amdgcn_sicmp(k * 64, left, kIcmpSlt);
        uint32_t peers_lo = (uint32_t)live, peers_hi = (uint32_t)(live >> 32);
#pragma unroll
        for (int b = 0; b < kBits; ++b) {
            const int set = __builtin_amdgcn_sbfe((int)d, b, 1);
            const uint64_t bal = __builtin_amdgcn_sicmp(set, 0, kIcmpNe);
            peers_lo = __builtin_amdgcn_bitop3_b32(peers_lo, (uint32_t)set, (uint32_t)bal, kPeersAndAgree);
            peers_hi = __builtin_amdgcn_bitop3_b32(peers_hi, (uint32_t)set, (uint32_t)(bal >> 32), kPeersAndAgree);
        }
        const uint64_t peers = ((uint64_t)peers_hi << 32) | peers_lo;
        int before = 0;
        if (in) before = wave_cnt[wave][d];
        __builtin_amdgcn_wave_barrier();
        if (in && (peers & lt_mask) == 0) wave_cnt[wave][d] = before + __popcll(peers);
        __builtin_amdgcn_wave_barrier();
        rank[k] = before + __popcll(peers & lt_mask);
        // The pair sort's kernels (7- and 8-bit digits, many rounds of tiles) form the rank here, one register per
        // key: left alone the compiler keeps the masked ballot (two registers) and `before` alive instead and
        // counts the bits after the look-back, 114 registers instead of 84, which costs a wavefront per SIMD.  The
        // depth sort's (9 bits, one round of tiles, bound by latency) gains nothing from it.
        if constexpr (kBits < 9) asm volatile("" : "+v"(rank[k]));
    }
    __syncthreads();

    // the first kRadix threads each own one digit
    const bool owner = tid < kRadix;
    int c[kOsWaves];
    uint32_t total = 0;
    uint32_t* my_status = status + (size_t)tile * kRadix + (owner ? tid : 0);
    if (owner) {
#pragma unroll
        for (int w = 0; w < kOsWaves; ++w) {
            c[w] = wave_cnt[w][tid];
            total += (uint32_t)c[w];
        }
        if (tile > 0) __hip_atomic_store(my_status, kFlagAggregate | total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    // where each digit starts in the whole output, and inside this tile
    const int excl_global = os_block_excl_scan<kOsWaves>(owner ? (int)hist[tid] : 0, s_scan);
    const int excl_local = os_block_excl_scan<kOsWaves>((int)total, s_scan);
    if (owner) {    // where each wavefront's keys of the digit start inside the tile
        int running = excl_local;
#pragma unroll
        for (int w = 0; w < kOsWaves; ++w) {
            wave_cnt[w][tid] = running;
            running += c[w];
        }
    }
    __syncthreads();

    // Place every pair at its tile-local sorted position, read the sorted keys back and request the values: none
    // of this needs the earlier tiles, so the values' round trip through memory runs while the look-back below
    // makes its own.
#pragma unroll
    for (int k = 0; k < kOsItems; ++k) {
        const int local = wave_begin + k * 64 + lane;
        if (tile_begin + local < m) {
            const uint32_t d = (uint32_t)(key[k] >> shift) & mask;
            const int pos = wave_cnt[wave][d] + rank[k];
            s_keys[pos] = key[k];
            s_src[pos] = (uint16_t)local;
        }
    }
    __syncthreads();
    // consecutive threads take consecutive sorted positions: equal-digit runs leave as contiguous segments.
    // All of a thread's values are fetched before the first is stored (positions past the count read the tile's
    // first pair instead and store nothing), so the gathers' latencies overlap instead of adding up.
    const int count = (int)min((long long)kOsTile, m - tile_begin);
    Key sorted_key[kOsItems];
    int32_t sorted_val[kOsItems];
#pragma unroll
    for (int k = 0; k < kOsItems; ++k) {
        const int i = k * kOsThreads + tid;
        const int ii = i < count ? i : 0;
        sorted_key[k] = s_keys[ii];
        sorted_val[k] = (int32_t)s_src[ii];
    }
    // without an input value array the values are the pairs' own indices
    if (vals_in) {
#pragma unroll
        for (int k = 0; k < kOsItems; ++k) sorted_val[k] = vals_in[tile_begin + sorted_val[k]];
    } else {
#pragma unroll
        for (int k = 0; k < kOsItems; ++k) sorted_val[k] += (int32_t)tile_begin;
    }

    if (owner) {
        // digits of earlier tiles: walk back until a tile that already knows its inclusive prefix.
        // kLookWindow predecessors are polled per step with independent loads, so the serial depth of
        // the walk is a fraction of the tiles in flight.
        uint32_t prev = 0;
        if (tile > 0) {
            int t = tile - 1;
            int spins = 0;
            bool finished = false;
            while (!finished) {
                uint32_t s[kLookWindow];
#pragma unroll
                for (int i = 0; i < kLookWindow; ++i) {
                    const int tt = t - i;
                    s[i] = tt >= 0 ? __hip_atomic_load(status + (size_t)tt * kRadix + tid, __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT)
                                   : kFlagPrefix;  // before the first tile: an empty inclusive prefix
                }
                int consumed = kLookWindow;
#pragma unroll
                for (int i = 0; i < kLookWindow; ++i) {
                    if (consumed != kLookWindow) continue;
                    if (s[i] == 0u) {
                        consumed = i;  // not published yet: poll again from this tile
                    } else if (s[i] & kFlagPrefix) {
                        prev += s[i] & kPrefixMask;
                        finished = true;
                        consumed = i + 1;
                    } else {
                        prev += s[i] & kAggregateMask;
                    }
                }
                t -= consumed;
                if (!finished && consumed < kLookWindow) {
                    if (++spins > kSpinLimit) {
                        atomicOr(error, 1u);
                        finished = true;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
            }
        }
        __hip_atomic_store(my_status, kFlagPrefix | ((prev + total) & kPrefixMask), __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
        digit_out[tid] = excl_global + (int)prev - excl_local;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < kOsItems; ++k) {
        const int i = k * kOsThreads + tid;
        if (i < count) {
            const uint32_t d = (uint32_t)(sorted_key[k] >> shift) & mask;
            const long long pos = (long long)digit_out[d] + i;
            keys_out[pos] = sorted_key[k];
            vals_out[pos] = sorted_val[k];
        }
    }
}

// Reports a finished sort's error word: 0, or D3GS_ERR_SORT_LOOKBACK when a workgroup's bounded wait ran out
// (the output is then not sorted).  One thread; the host word is pinned, device-mapped memory.
__global__ void os_status_kernel(const uint32_t* __restrict__ error, int32_t* __restrict__ status_dev,
                                 int32_t* __restrict__ status_host) {
    const int32_t st = __hip_atomic_load(error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ? D3GS_ERR_SORT_LOOKBACK : 0;
    if (status_dev) *status_dev = st;
    if (status_host) *status_host = st;
}

static inline size_t os_align(size_t v) { return (v + 255) / 256 * 256; }
static inline int os_tiles(int64_t m) { return (int)((m + kOsTile - 1) / kOsTile); }
static inline int os_passes(int begin_bit, int end_bit) {
    const int digit = os_digit_bits(begin_bit, end_bit);
    return (end_bit - begin_bit + digit - 1) / digit;
}

static size_t os_layout(int64_t m, int passes, int radix, SortWorkspace* ws, void* base) {
    const int ntiles = os_tiles(m) > 0 ? os_tiles(m) : 1;
    size_t off = 0;
    char* b = (char*)base;
    if (ws) ws->hist = (uint32_t*)(b + off);
    off += os_align((size_t)passes * radix * 4);
    if (ws) ws->error = (uint32_t*)(b + off);
    off += 256;
    if (ws) ws->status = (uint32_t*)(b + off);
    off += os_align((size_t)passes * ntiles * radix * 4);
    return off;
}

}  // namespace d3gs

using namespace d3gs;

extern "C" int d3gs_sort_workspace_bytes(int64_t m, int begin_bit, int end_bit, size_t* bytes_out_host) {
    if (m < 0 || begin_bit < 0 || end_bit > 64 || begin_bit > end_bit || !bytes_out_host) {
        set_error("d3gs_sort_workspace_bytes: bad argument");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    const int passes = os_passes(begin_bit, end_bit) > 0 ? os_passes(begin_bit, end_bit) : 1;
    *bytes_out_host = os_layout(m, passes, 1 << os_digit_bits(begin_bit, end_bit), nullptr, nullptr);
    return D3GS_OK;
}

extern "C" int d3gs_sort_error_offset(int64_t m, int begin_bit, int end_bit, size_t* offset_out_host) {
    if (m < 0 || begin_bit < 0 || end_bit > 64 || begin_bit > end_bit || !offset_out_host) {
        set_error("d3gs_sort_error_offset: bad argument");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    const int passes = os_passes(begin_bit, end_bit) > 0 ? os_passes(begin_bit, end_bit) : 1;
    // the error word follows the digit histograms (os_layout)
    *offset_out_host = os_align((size_t)passes * (1 << os_digit_bits(begin_bit, end_bit)) * 4);
    return D3GS_OK;
}

extern "C" int d3gs_sort_status(const void* workspace, size_t workspace_bytes, int64_t m, int begin_bit, int end_bit,
                                int32_t* status_dev, int32_t* status_host, d3gs_stream_t stream) {
    size_t off = 0;
    int rc = d3gs_sort_error_offset(m, begin_bit, end_bit, &off);
    if (rc) return rc;
    if (!workspace || workspace_bytes < off + sizeof(uint32_t) || (!status_dev && !status_host)) {
        set_error("d3gs_sort_status: NULL or short workspace, or no status word to write");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    hipLaunchKernelGGL(os_status_kernel, dim3(1), dim3(1), 0, (hipStream_t)stream,
                       (const uint32_t*)((const char*)workspace + off), status_dev, status_host);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_sort_status: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

template <typename Key>
static int sort_pairs_impl(const char* who, int key_bits, Key* keys_a, Key* keys_b, int32_t* vals_a, int32_t* vals_b,
                           void* workspace, size_t workspace_bytes, int64_t m, const int64_t* m_device,
                           int values_are_indices, int workspace_is_zero, int begin_bit, int end_bit,
                           int* result_in_b_host, d3gs_stream_t stream) {
    if (m < 0 || begin_bit < 0 || end_bit > key_bits || begin_bit > end_bit || !result_in_b_host) {
        set_error("%s: bad argument (m=%lld bits=[%d,%d))", who, (long long)m, begin_bit, end_bit);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    if (m > kOsMaxPairs) { set_error("%s: more than 2^31 - 1024 pairs are not supported", who); return D3GS_ERR_UNSUPPORTED; }
    *result_in_b_host = 0;
    if (m == 0 || begin_bit == end_bit) return D3GS_OK;
    if (!keys_a || !keys_b || !vals_a || !vals_b || !workspace) {
        set_error("%s: NULL buffer", who);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    const int passes = os_passes(begin_bit, end_bit);
    const int digit = os_digit_bits(begin_bit, end_bit), radix = 1 << digit;
    SortWorkspace ws;
    const size_t need = os_layout(m, passes, radix, &ws, workspace);
    if (workspace_bytes < need) {
        set_error("%s: workspace %zu < required %zu", who, workspace_bytes, need);
        return D3GS_ERR_WORKSPACE_TOO_SMALL;
    }
    hipStream_t s = (hipStream_t)stream;
    const int ntiles = os_tiles(m);
    // a fill kernel, not a memset node, so the call can be captured in a graph
    if (!workspace_is_zero)
        hipLaunchKernelGGL(os_clear_kernel, dim3(512), dim3(kBlock), 0, s, (uint32_t*)workspace, need / 4);
    const int hist_blocks = (int)std::min<int64_t>(kHistMaxBlocks, (m + kHistThreads * kHistKeysPerThread - 1) / (kHistThreads * kHistKeysPerThread));
    // as many LDS copies of the histogram table as fit in 64 KB (a power of two, at most kHistCopies)
    int copies = kHistCopies;
    while (copies > 1 && (size_t)copies * passes * radix * sizeof(uint32_t) > 64 * 1024) copies >>= 1;
    const size_t hist_lds = (size_t)copies * passes * radix * sizeof(uint32_t);
    auto hist_kernel = digit == 9 ? os_hist_kernel<Key, 9> : digit == 8 ? os_hist_kernel<Key, 8> : os_hist_kernel<Key, 7>;
    auto pass_kernel = digit == 9 ? os_pass_kernel<Key, 9> : digit == 8 ? os_pass_kernel<Key, 8> : os_pass_kernel<Key, 7>;
    hipLaunchKernelGGL(hist_kernel, dim3(hist_blocks), dim3(kHistThreads), hist_lds, s, keys_a, (long long)m,
                       (const long long*)m_device, begin_bit, end_bit, passes, copies, ws.hist);
    Key* kin = keys_a;
    Key* kout = keys_b;
    const int32_t* vin = values_are_indices ? nullptr : vals_a;   // first pass only
    int32_t* vout = vals_b;
    int in_b = 0;
    for (int p = 0; p < passes; ++p) {
        const int bit = begin_bit + digit * p;
        const int nb = std::min(digit, end_bit - bit);
        const uint32_t mask = (1u << nb) - 1u;
        const uint32_t* pass_hist = ws.hist + (size_t)p * radix;
        uint32_t* pass_status = ws.status + (size_t)p * ntiles * radix;
        hipLaunchKernelGGL(pass_kernel, dim3(ntiles), dim3(digit == 9 ? os_threads<9>() : os_threads<8>()), 0, s, kin, vin,
                           kout, vout, (long long)m,
                           (const long long*)m_device, bit, mask, ntiles, pass_hist, pass_status, ws.error);
        std::swap(kin, kout);
        vin = vout;
        vout = in_b ? vals_b : vals_a;
        in_b ^= 1;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("%s: launch failed: %s", who, hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    *result_in_b_host = in_b;
    return D3GS_OK;
}

extern "C" int d3gs_sort_pairs(uint64_t* keys_a, uint64_t* keys_b, int32_t* vals_a, int32_t* vals_b, void* workspace,
                               size_t workspace_bytes, int64_t m, int begin_bit, int end_bit, int* result_in_b_host,
                               d3gs_stream_t stream) {
    return sort_pairs_impl<uint64_t>("d3gs_sort_pairs", 64, keys_a, keys_b, vals_a, vals_b, workspace, workspace_bytes, m,
                                     nullptr, 0, 0, begin_bit, end_bit, result_in_b_host, stream);
}

// The pair sort of the one-call binning on 16-bit tile ids (at most 2^16 tiles): the same kernels over keys half as
// wide, a quarter less to move per pass.
int d3gs::sort_pairs_u16(uint16_t* keys_a, uint16_t* keys_b, int32_t* vals_a, int32_t* vals_b, void* workspace,
                         size_t workspace_bytes, int64_t m, const int64_t* m_device, int workspace_is_zero, int end_bit,
                         int* result_in_b_host, d3gs_stream_t stream) {
    return sort_pairs_impl<uint16_t>("d3gs_bin_pairs (pair sort, 16-bit tile ids)", 16, keys_a, keys_b, vals_a, vals_b,
                                     workspace, workspace_bytes, m, m_device, 0, workspace_is_zero, 0, end_bit,
                                     result_in_b_host, stream);
}

extern "C" int d3gs_sort_pairs_u32(uint32_t* keys_a, uint32_t* keys_b, int32_t* vals_a, int32_t* vals_b, void* workspace,
                                   size_t workspace_bytes, int64_t m, const int64_t* m_device, int values_are_indices,
                                   int workspace_is_zero, int begin_bit, int end_bit, int* result_in_b_host,
                                   d3gs_stream_t stream) {
    return sort_pairs_impl<uint32_t>("d3gs_sort_pairs_u32", 32, keys_a, keys_b, vals_a, vals_b, workspace,
                                     workspace_bytes, m, m_device, values_are_indices, workspace_is_zero, begin_bit,
                                     end_bit, result_in_b_host, stream);
}
