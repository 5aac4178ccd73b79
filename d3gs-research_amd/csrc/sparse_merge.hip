// Sparse-mode bundles: the gradient rows of a gaussian that several cameras accepted are merged into one row.
//
// The reference deduplicates the accepted ids with a device hash table (insert, collect, query) and adds the rows
// with atomics (d3sim/algos/d3gs/render.py:2864-2903).  Here the ids are sorted with the library's radix sort
// (value = row), runs of equal ids are numbered by a scan of their first-element flags, and each merged row is the
// sum of its run's rows taken in sorted order by one thread per (merged row, column): no atomics, the same sums on
// every run, and the merged rows come out in ascending id order.
#include "device_math.h"

namespace d3gs {

constexpr int kMergeBlock = 256;

__global__ __launch_bounds__(kMergeBlock) void copy_ids_kernel(const int32_t* __restrict__ ids, int n,
                                                                uint32_t* __restrict__ keys) {
    const int i = blockIdx.x * kMergeBlock + threadIdx.x;
    if (i < n) keys[i] = (uint32_t)ids[i];
}

__global__ __launch_bounds__(kMergeBlock) void run_flags_kernel(const uint32_t* __restrict__ sorted, int n,
                                                                 int32_t* __restrict__ flags) {
    const int i = blockIdx.x * kMergeBlock + threadIdx.x;
    if (i < n) flags[i] = (i == 0 || sorted[i] != sorted[i - 1]) ? 1 : 0;
}

// scan: inclusive scan of the flags, so run number = scan - 1
__global__ __launch_bounds__(kMergeBlock) void run_scatter_kernel(const uint32_t* __restrict__ sorted,
                                                                   const int32_t* __restrict__ rows_sorted,
                                                                   const int32_t* __restrict__ flags,
                                                                   const int32_t* __restrict__ scan, int n,
                                                                   int32_t* __restrict__ unique_ids,
                                                                   int32_t* __restrict__ inverse,
                                                                   int32_t* __restrict__ run_rows,
                                                                   int32_t* __restrict__ run_starts) {
    const int i = blockIdx.x * kMergeBlock + threadIdx.x;
    if (i >= n) return;
    const int run = scan[i] - 1;
    const int row = rows_sorted[i];
    if (flags[i]) {
        unique_ids[run] = (int32_t)sorted[i];
        run_starts[run] = i;
    }
    if ((unsigned)row < (unsigned)n) inverse[row] = run;
    run_rows[i] = row;
    if (i == n - 1) run_starts[run + 1] = n;
}

__global__ __launch_bounds__(kMergeBlock) void merge_rows_kernel(const float* __restrict__ rows, int width, int n_rows,
                                                                  const int32_t* __restrict__ run_rows,
                                                                  const int32_t* __restrict__ run_starts, int n_runs,
                                                                  float* __restrict__ merged) {
    const long long e = (long long)blockIdx.x * kMergeBlock + threadIdx.x;
    if (e >= (long long)n_runs * width) return;
    const int run = (int)(e / width), col = (int)(e - (long long)run * width);
    const int lo = run_starts[run], hi = run_starts[run + 1];
    float sum = 0.0f;
    for (int k = lo; k < hi; ++k) {
        const int row = run_rows[k];
        if ((unsigned)row < (unsigned)n_rows) sum += rows[(size_t)row * width + col];
    }
    merged[e] = sum;
}

struct UniqueLayout { size_t keys_a, keys_b, vals_a, vals_b, flags, scan, sort_ws, scan_ws, total; size_t sort_bytes, scan_bytes; };

static int unique_layout(int32_t count, int32_t id_limit, UniqueLayout* L) {
    const size_t slice = (((size_t)count * 4) + 255) / 256 * 256;
    size_t sort_bytes = 0, scan_bytes = 0;
    int rc = d3gs_sort_workspace_bytes(count, 0, d3gs_higher_msb((uint32_t)id_limit), &sort_bytes);
    if (rc) return rc;
    rc = d3gs_scan_gathered_workspace_bytes(count, &scan_bytes);
    if (rc) return rc;
    L->keys_a = 0; L->keys_b = slice; L->vals_a = 2 * slice; L->vals_b = 3 * slice; L->flags = 4 * slice; L->scan = 5 * slice;
    L->sort_ws = 6 * slice;
    L->scan_ws = L->sort_ws + (sort_bytes + 255) / 256 * 256;
    L->total = L->scan_ws + (scan_bytes + 255) / 256 * 256;
    L->sort_bytes = sort_bytes; L->scan_bytes = scan_bytes;
    return D3GS_OK;
}

}  // namespace d3gs

using namespace d3gs;

extern "C" int d3gs_unique_ids_workspace_bytes(int32_t count, int32_t id_limit, size_t* bytes_out_host) {
    if (count < 0 || id_limit < 0 || !bytes_out_host) { set_error("d3gs_unique_ids_workspace_bytes: bad argument"); return D3GS_ERR_INVALID_ARGUMENT; }
    UniqueLayout L;
    int rc = unique_layout(count, id_limit, &L);
    if (rc) return rc;
    *bytes_out_host = L.total;
    return D3GS_OK;
}

extern "C" int d3gs_unique_ids(const int32_t* ids, int32_t count, int32_t id_limit, int32_t* unique_ids, int32_t* inverse,
                               int32_t* run_rows, int32_t* run_starts, void* workspace, size_t workspace_bytes,
                               int64_t* unique_count_dev, int64_t* unique_count_host, d3gs_stream_t stream) {
    if (count < 0 || id_limit < 0 || !unique_count_dev) { set_error("d3gs_unique_ids: bad argument"); return D3GS_ERR_INVALID_ARGUMENT; }
    hipStream_t s = (hipStream_t)stream;
    if (count == 0)     // the scan of nothing stores a zero total (and the host word)
        return d3gs_scan_gathered(nullptr, 0, nullptr, 0, nullptr, nullptr, 0, 0, unique_count_dev, unique_count_host, stream);
    if (!ids || !unique_ids || !inverse || !run_rows || !run_starts || !workspace) {
        set_error("d3gs_unique_ids: NULL buffer");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    UniqueLayout L;
    int rc = unique_layout(count, id_limit, &L);
    if (rc) return rc;
    if (workspace_bytes < L.total || ((uintptr_t)workspace & 255u)) {
        set_error("d3gs_unique_ids: workspace of %zu bytes needed (256-byte aligned), %zu given", L.total, workspace_bytes);
        return D3GS_ERR_WORKSPACE_TOO_SMALL;
    }
    char* w = (char*)workspace;
    uint32_t *keys_a = (uint32_t*)(w + L.keys_a), *keys_b = (uint32_t*)(w + L.keys_b);
    int32_t *vals_a = (int32_t*)(w + L.vals_a), *vals_b = (int32_t*)(w + L.vals_b);
    int32_t *flags = (int32_t*)(w + L.flags), *scan = (int32_t*)(w + L.scan);
    const dim3 grid((count + kMergeBlock - 1) / kMergeBlock), block(kMergeBlock);
    hipLaunchKernelGGL(copy_ids_kernel, grid, block, 0, s, ids, (int)count, keys_a);
    int in_b = 0;
    rc = d3gs_sort_pairs_u32(keys_a, keys_b, vals_a, vals_b, w + L.sort_ws, L.sort_bytes, count, nullptr,
                             /*values_are_indices=*/1, /*workspace_is_zero=*/0, 0, d3gs_higher_msb((uint32_t)id_limit), &in_b,
                             stream);
    if (rc) return rc;
    const uint32_t* sorted = in_b ? keys_b : keys_a;
    const int32_t* rows_sorted = in_b ? vals_b : vals_a;
    hipLaunchKernelGGL(run_flags_kernel, grid, block, 0, s, sorted, (int)count, flags);
    rc = d3gs_scan_gathered(flags, count, nullptr, count, scan, w + L.scan_ws, L.scan_bytes, 0, unique_count_dev,
                            unique_count_host, stream);
    if (rc) return rc;
    hipLaunchKernelGGL(run_scatter_kernel, grid, block, 0, s, sorted, rows_sorted, flags, scan, (int)count, unique_ids,
                       inverse, run_rows, run_starts);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_unique_ids: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}

extern "C" int d3gs_merge_rows(const float* rows, int32_t n_rows, int32_t width, const int32_t* run_rows,
                               const int32_t* run_starts, int32_t n_runs, float* merged, d3gs_stream_t stream) {
    if (n_rows < 0 || width < 0 || n_runs < 0) { set_error("d3gs_merge_rows: bad argument"); return D3GS_ERR_INVALID_ARGUMENT; }
    if (n_runs == 0 || width == 0) return D3GS_OK;
    if (!rows || !run_rows || !run_starts || !merged) { set_error("d3gs_merge_rows: NULL buffer"); return D3GS_ERR_INVALID_ARGUMENT; }
    const long long elems = (long long)n_runs * width;
    hipLaunchKernelGGL(merge_rows_kernel, dim3((unsigned)((elems + kMergeBlock - 1) / kMergeBlock)), dim3(kMergeBlock), 0,
                       (hipStream_t)stream, rows, (int)width, (int)n_rows, run_rows, run_starts, (int)n_runs, merged);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) { set_error("d3gs_merge_rows: launch failed: %s", hipGetErrorString(e)); return D3GS_ERR_LAUNCH; }
    return D3GS_OK;
}
