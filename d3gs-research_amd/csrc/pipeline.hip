// Composite entry point: the whole binning of one view (depth order, offsets, key expansion, pair sort,
// tile ranges and launch order) enqueued by one call.  Every step is one of the library's own entry points,
// in the order a caller would issue them; doing it here takes the caller's per-launch cost (argument
// marshalling in an interpreter, allocation between launches) off the stream's critical path, where the
// kernels of this phase are short enough for that cost to leave the GPU idle between them.
#include "device_math.h"

using namespace d3gs;

extern "C" int d3gs_bin_pairs(const d3gs_params* p, const int32_t* radii, const float* uvs, const float* conic_opacity,
                              const float* depths, const int32_t* tiles_touched, const uint64_t* tile_masks,
                              uint32_t* depth_keys_a, uint32_t* depth_keys_b, int32_t* order_a, int32_t* order_b,
                              void* depth_sort_ws, size_t depth_sort_ws_bytes, int32_t* offsets, void* scan_ws,
                              size_t scan_ws_bytes, int64_t* total_dev, int64_t* total_host, int64_t capacity,
                              uint32_t* tile_keys_a, uint32_t* tile_keys_b, int32_t* idx_a, int32_t* idx_b,
                              void* pair_sort_ws, size_t pair_sort_ws_bytes, int32_t* workload_ranges,
                              int32_t* tile_order, int32_t flags, int32_t* order_in_b,
                              int32_t* pairs_in_b, d3gs_stream_t stream) {
    if (!p || !order_in_b || !pairs_in_b || !total_dev || capacity < 0) {
        set_error("d3gs_bin_pairs: bad argument");
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    const int32_t n = item_count(*p);                               // render items: gaussians x cameras of a bundle
    const int32_t num_tiles = p->tiles_x * p->tiles_y * batch_count(*p);
    const int32_t workspaces_are_zero = flags & D3GS_BIN_WORKSPACES_ARE_ZERO;
    const bool host_word_at_end = (flags & D3GS_BIN_HOST_COUNT_AT_END) != 0;
    const bool narrow = (flags & D3GS_BIN_KEYS_16BIT) != 0;
    if (narrow && num_tiles > (1 << 16)) {
        set_error("d3gs_bin_pairs: D3GS_BIN_KEYS_16BIT needs at most 2^16 tiles (this call has %d)", num_tiles);
        return D3GS_ERR_INVALID_ARGUMENT;
    }
    int rc = d3gs_sort_pairs_u32(depth_keys_a, depth_keys_b, order_a, order_b, depth_sort_ws, depth_sort_ws_bytes, n,
                                 nullptr, /*values_are_indices=*/1, workspaces_are_zero, 0,
                                 d3gs_depth_key_bits(p), order_in_b, stream);
    if (rc) return rc;
    const uint32_t* depth_keys_sorted = *order_in_b ? depth_keys_b : depth_keys_a;
    const int32_t* order = *order_in_b ? order_b : order_a;
    // the pair count also goes to the host word, written by the scan itself (or, with D3GS_BIN_HOST_COUNT_AT_END, by
    // the last kernel of the call only); nothing here waits for it
    rc = d3gs_scan_gathered(tiles_touched, n, order, n, offsets, scan_ws, scan_ws_bytes, workspaces_are_zero, total_dev,
                            host_word_at_end ? nullptr : total_host, stream);
    if (rc) return rc;
    const int tile_bits = d3gs_higher_msb((uint32_t)num_tiles);
    // With D3GS_BIN_KEYS_16BIT the pair keys are 16-bit tile ids, stored in the front half of the caller's key
    // buffers: key expansion writes, both sort passes move and the ranges kernel reads half as many key bytes.
    if (narrow) {
        uint16_t* keys16_a = reinterpret_cast<uint16_t*>(tile_keys_a);
        uint16_t* keys16_b = reinterpret_cast<uint16_t*>(tile_keys_b);
        rc = make_tile_keys_u16(p, radii, uvs, conic_opacity, depths, offsets, order, depth_keys_sorted, tile_masks,
                                keys16_a, idx_a, capacity, stream);
        if (rc) return rc;
        rc = sort_pairs_u16(keys16_a, keys16_b, idx_a, idx_b, pair_sort_ws, pair_sort_ws_bytes, capacity, total_dev,
                            workspaces_are_zero ? kSortWorkspaceIsZero : 0, tile_bits, pairs_in_b, stream);
    } else {
        rc = d3gs_make_keys(p, radii, uvs, conic_opacity, depths, offsets, order, depth_keys_sorted, tile_masks, nullptr,
                            tile_keys_a, idx_a, capacity, stream);
        if (rc) return rc;
        rc = d3gs_sort_pairs_u32(tile_keys_a, tile_keys_b, idx_a, idx_b, pair_sort_ws, pair_sort_ws_bytes, capacity,
                                 total_dev, /*values_are_indices=*/0, workspaces_are_zero, 0, tile_bits, pairs_in_b, stream);
    }
    if (rc) return rc;
    // the last kernel replaces the pair count by D3GS_COUNT_SORT_GAVE_UP when either sort raised its error word
    size_t err_depth = 0, err_pairs = 0;
    d3gs_sort_error_offset(n, 0, d3gs_depth_key_bits(p), &err_depth);
    d3gs_sort_error_offset(capacity, 0, d3gs_higher_msb((uint32_t)num_tiles), &err_pairs);
    const uint32_t* e_depth = n > 0 && depth_sort_ws ? (const uint32_t*)((const char*)depth_sort_ws + err_depth) : nullptr;
    const uint32_t* e_pairs = capacity > 0 && pair_sort_ws ? (const uint32_t*)((const char*)pair_sort_ws + err_pairs) : nullptr;
    if (narrow)
        return tile_ranges_u16_with_status(reinterpret_cast<const uint16_t*>(*pairs_in_b ? tile_keys_b : tile_keys_a),
                                           capacity, total_dev, workload_ranges, num_tiles, tile_order, e_depth, e_pairs,
                                           total_dev, total_host, host_word_at_end, stream);
    return tile_ranges_u32_with_status(*pairs_in_b ? tile_keys_b : tile_keys_a, capacity, total_dev, workload_ranges,
                                       num_tiles, tile_order, e_depth, e_pairs, total_dev, total_host, host_word_at_end,
                                       stream);
}
