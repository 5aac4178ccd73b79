"""The reference's own call sequence through the C ABI, without any of the optional accelerations:
fused preprocess (SH colours included, no kept-tile record), scan of the tile counts in gaussian
order, key expansion without an order table, one radix sort over the whole (tile, depth) key, tile
ranges and the blend in raster order (render.py:629-681, 694-695, 839-840, 845-887, 937-939,
2304-2309).  Every buffer must equal the CPU oracle's and therefore the operator's fast path."""
import ctypes as C

import numpy as np
import pytest

from helpers import gen_scene, op_config, oracle_forward, torch_model

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cfg_id,n,wh,filt", [(0, None, None, 1), (1, 20000, (250, 190), 4), (2, 100000, (640, 360), 3)])
def test_reference_call_sequence(oracle, cfg_id, n, wh, filt):
    import torch
    from d3gs_research_amd import _capi
    from d3gs_research_amd.render import GaussianSplatOp
    scene = gen_scene(cfg_id, n=n, wh=wh)
    print(f"reference sequence cfg={cfg_id} n={scene.n} filter={filt}", flush=True)
    P_ref, ref = oracle_forward(oracle, scene, filt)
    op = GaussianSplatOp(op_config(scene, filt))
    model = torch_model(scene)
    P = op.make_params(model, scene.camera(), True)
    L = _capi.lib()
    p = _capi.ptr
    N, dev = scene.n, "cuda"
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    f32, i32 = torch.float32, torch.int32
    depths, radii = torch.empty(N, dtype=f32, device=dev), torch.empty(N, dtype=i32, device=dev)
    uvs, conic = torch.empty((N, 2), dtype=f32, device=dev), torch.empty((N, 4), dtype=f32, device=dev)
    touched, rgb = torch.empty(N, dtype=i32, device=dev), torch.empty((N, 3), dtype=f32, device=dev)
    cov2d, ne0 = torch.empty((N, 3), dtype=f32, device=dev), torch.empty(N, dtype=torch.uint8, device=dev)
    _capi.check(L.d3gs_preprocess_fwd(C.byref(P), p(model.xyz), p(model.quaternion_xyzw), p(model.scale), p(model.opacity),
                                      p(model.color_sh), None, None, p(depths), p(radii), p(uvs), p(conic), p(touched),
                                      p(rgb), p(cov2d), p(ne0), None, None, None, s), "preprocess")
    cpu = lambda t: t.cpu().numpy()
    assert np.array_equal(cpu(touched), ref["tiles_touched"])
    assert np.array_equal(cpu(rgb).view(np.uint32), ref["rgb_gaussian"].view(np.uint32))
    assert np.array_equal(cpu(ne0), ref["sh_to_rgb_ne_0"])

    nbytes = C.c_size_t(0)
    _capi.check(L.d3gs_scan_workspace_bytes(N, C.byref(nbytes)), "scan ws")
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
    total = torch.zeros(1, dtype=torch.int64, device=dev)
    _capi.check(L.d3gs_scan_tiles(p(touched), N, p(ws), nbytes.value, p(total), s), "scan")
    M = int(total.item())
    assert M == ref["num_rendered"]

    keys, vals = torch.empty(M, dtype=torch.int64, device=dev), torch.empty(M, dtype=i32, device=dev)
    _capi.check(L.d3gs_make_keys(C.byref(P), p(radii), p(uvs), p(conic), p(depths), p(touched), None, None, None,
                                 p(keys), None, p(vals), M, s), "make_keys")
    assert np.array_equal(cpu(keys).view(np.uint64), ref["keys"])
    assert np.array_equal(cpu(vals), ref["vals"])

    tiles = P.tiles_x * P.tiles_y
    end_bit = 32 + L.d3gs_higher_msb(tiles)
    kb, vb = torch.empty_like(keys), torch.empty_like(vals)
    _capi.check(L.d3gs_sort_workspace_bytes(M, 0, end_bit, C.byref(nbytes)), "sort ws")
    sws = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
    in_b = C.c_int(0)
    _capi.check(L.d3gs_sort_pairs(p(keys), p(kb), p(vals), p(vb), p(sws), nbytes.value, M, 0, end_bit, C.byref(in_b), s),
                "sort")
    ks, vs = (kb, vb) if in_b.value else (keys, vals)
    assert np.array_equal(cpu(ks).view(np.uint64), ref["keys_sorted"])
    assert np.array_equal(cpu(vs), ref["gaussian_idx_sorted"])

    ranges = torch.zeros((tiles, 2), dtype=i32, device=dev)
    _capi.check(L.d3gs_tile_ranges(p(ks), M, p(ranges), tiles, None, s), "tile_ranges")
    assert np.array_equal(cpu(ranges), ref["workload_ranges"])

    H, W = scene.height, scene.width
    color = torch.empty((H, W, 3), dtype=f32, device=dev)
    T, nc = torch.empty((H, W), dtype=f32, device=dev), torch.empty((H, W), dtype=i32, device=dev)
    scratch = torch.full((4096 + 3,), 7.0, dtype=f32, device=dev)[:4096]     # a region for the kernel to clear
    _capi.check(L.d3gs_blend_fwd(C.byref(P), p(ranges), p(vs), p(uvs), p(conic), p(rgb), None, None, p(color), p(T), p(nc),
                                 None, p(scratch), 4096 * 4, s), "blend_fwd")
    torch.cuda.synchronize()
    assert np.array_equal(cpu(nc), ref["n_contrib"])
    assert np.array_equal(cpu(color).view(np.uint32), ref["color"].view(np.uint32))
    assert np.array_equal(cpu(T).view(np.uint32), ref["T"].view(np.uint32))
    assert float(scratch.abs().max()) == 0.0

    # and the operator's fast path gives the same image
    out, ctx = op.forward(model, scene.camera(), training=True)
    assert torch.equal(out.color[0], color) and torch.equal(out.T[0], T) and torch.equal(out.n_contrib[0], nc)
    assert torch.equal(ctx.gaussian_idx_sorted, vs) and torch.equal(ctx.workload_ranges, ranges)

    # the same binning through the one-call entry point (depth-first factorisation, 32-bit tile keys): the sorted
    # gaussian indices, the ranges and the pair count must equal the plain sequence's
    tile_masks = torch.empty((N, 2), dtype=torch.int64, device=dev)
    dkeys_a, dkeys_b = torch.empty(N, dtype=i32, device=dev), torch.empty(N, dtype=i32, device=dev)
    _capi.check(L.d3gs_preprocess_fwd(C.byref(P), p(model.xyz), p(model.quaternion_xyzw), p(model.scale), p(model.opacity),
                                      p(model.color_sh), None, None, p(depths), p(radii), p(uvs), p(conic), p(touched),
                                      p(rgb), p(cov2d), p(ne0), p(tile_masks), p(dkeys_a), None, s), "preprocess (masks, keys)")
    cap = M + 1000
    ord_a, ord_b, offs = (torch.empty(N, dtype=i32, device=dev) for _ in range(3))
    tk_a, tk_b, ix_a, ix_b = (torch.empty(cap, dtype=i32, device=dev) for _ in range(4))
    tile_bits = L.d3gs_higher_msb(tiles)
    sizes = []
    for call, args in ((L.d3gs_sort_workspace_bytes, (N, 0, L.d3gs_depth_key_bits(C.byref(P)))),
                       (L.d3gs_scan_gathered_workspace_bytes, (N,)),
                       (L.d3gs_sort_workspace_bytes, (cap, 0, tile_bits))):
        _capi.check(call(*args, C.byref(nbytes)), "workspace size")
        sizes.append(nbytes.value)
    ws1, ws2, ws3 = (torch.full((b,), 0x5A, dtype=torch.uint8, device=dev) for b in sizes)   # not zero: the library clears
    ranges2, order2 = torch.zeros((tiles, 2), dtype=i32, device=dev), torch.empty(tiles, dtype=i32, device=dev)
    total2 = torch.empty(1, dtype=torch.int64, device=dev)
    host_total = torch.full((1,), -1, dtype=torch.int64).pin_memory()
    order_in_b, pairs_in_b = C.c_int(-1), C.c_int(-1)
    _capi.check(L.d3gs_bin_pairs(C.byref(P), p(radii), p(uvs), p(conic), p(depths), p(touched), p(tile_masks), p(dkeys_a),
                                 p(dkeys_b), p(ord_a), p(ord_b), p(ws1), sizes[0], p(offs), p(ws2), sizes[1], p(total2),
                                 C.c_void_p(host_total.data_ptr()), cap, p(tk_a), p(tk_b), p(ix_a), p(ix_b), p(ws3), sizes[2],
                                 p(ranges2), p(order2), 0, C.byref(order_in_b), C.byref(pairs_in_b), s), "bin_pairs")
    torch.cuda.synchronize()
    assert int(total2.item()) == M and int(host_total[0]) == M
    assert order_in_b.value in (0, 1) and pairs_in_b.value in (0, 1)
    vs2 = (ix_b if pairs_in_b.value else ix_a)[:M]
    tks = (tk_b if pairs_in_b.value else tk_a)[:M]
    assert np.array_equal(cpu(vs2), ref["gaussian_idx_sorted"])
    assert np.array_equal(cpu(tks).astype(np.uint64), ref["keys_sorted"] >> np.uint64(32))
    assert np.array_equal(cpu(ranges2), ref["workload_ranges"])
    assert np.array_equal(np.sort(cpu(order2)), np.arange(tiles))

    # single-stream fused preprocess through the operator (overlap_sh_colors off)
    op2 = GaussianSplatOp(op_config(scene, filt))
    op2.overlap_sh_colors = False
    out2, ctx2 = op2.forward(model, scene.camera(), training=True)
    assert torch.equal(out2.color, out.color) and torch.equal(ctx2.rgb_gaussian, ctx.rgb_gaussian)
    assert torch.equal(ctx2.sh_to_rgb_ne_0, ctx.sh_to_rgb_ne_0)
