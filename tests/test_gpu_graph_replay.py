"""The library's calls under HIP graph capture: one view, forward and backward (clear, K1 with the colours, the
one-call binning, both blend kernels, K9), captured once through the C ABI and replayed while the model moves.

Nothing in these calls allocates, synchronises or records a memset node (workspaces are cleared by fill kernels),
and the host values they return (which buffer of a pair holds the result) depend on sizes only, so a captured view
stays valid as long as its pair count fits the captured capacity.  Every replay is checked against the same calls
issued eagerly on the same inputs, with unrelated eager work and a synchronisation between the replays."""
import ctypes as C

import numpy as np
import pytest

from helpers import gen_scene, op_config, torch_model

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cfg_id,n,wh", [(0, None, None), (1, 30000, (320, 240))])
def test_captured_view_replays_like_eager_calls(cfg_id, n, wh):
    import torch
    from d3gs_research_amd import _capi
    from d3gs_research_amd.render import GaussianSplatOp
    scene = gen_scene(cfg_id, n=n, wh=wh)
    print(f"graph replay cfg={cfg_id} n={scene.n}", flush=True)
    op = GaussianSplatOp(op_config(scene, 4))
    model = torch_model(scene)
    P = op.make_params(model, scene.camera(), True)
    L, p = _capi.lib(), _capi.ptr
    N, dev, H, W = scene.n, "cuda", scene.height, scene.width
    tiles = P.tiles_x * P.tiles_y
    f32, i32, u8 = torch.float32, torch.int32, torch.uint8
    rng = np.random.default_rng(7)

    # capacity of the pair buffers: the first view's count with head room (what the operator does from view to view)
    _, ctx0 = op.forward(model, scene.camera(), training=True)
    cap = int(ctx0.gaussian_idx_sorted.numel()) * 5 // 4 + 4096
    depths, radii, touched_tiles = (torch.empty(N, dtype=t, device=dev) for t in (f32, i32, i32))
    uvs, conic = torch.empty((N, 2), dtype=f32, device=dev), torch.empty((N, 4), dtype=f32, device=dev)
    rgb, cov2d, ne0 = torch.empty((N, 3), dtype=f32, device=dev), torch.empty((N, 3), dtype=f32, device=dev), torch.empty(N, dtype=u8, device=dev)
    tile_masks = torch.empty((N, 2), dtype=torch.int64, device=dev)
    dk_a, dk_b, ord_a, ord_b, offs = (torch.empty(N, dtype=i32, device=dev) for _ in range(5))
    tk_a, tk_b, ix_a, ix_b = (torch.empty(cap, dtype=i32, device=dev) for _ in range(4))
    nbytes, sizes = C.c_size_t(0), []
    for call, args in ((L.d3gs_sort_workspace_bytes, (N, 0, L.d3gs_depth_key_bits(C.byref(P)))),
                       (L.d3gs_scan_gathered_workspace_bytes, (N,)),
                       (L.d3gs_sort_workspace_bytes, (cap, 0, L.d3gs_higher_msb(tiles)))):
        _capi.check(call(*args, C.byref(nbytes)), "workspace size")
        sizes.append((nbytes.value + 255) // 256 * 256)
    # everything that has to be zero when a view starts, in one buffer and one fill
    rec = _capi.GRAD_RECORD_FLOATS
    zero_sizes = sizes + [tiles * 8, N * rec * 4, (N + 255) // 256 * 256] + [model_t.numel() * 4 for model_t in
                                                                             (model.xyz, model.quaternion_xyzw, model.scale, model.opacity, model.color_sh)]
    zero_sizes = [(b + 255) // 256 * 256 for b in zero_sizes]
    zero = torch.empty(sum(zero_sizes), dtype=u8, device=dev)
    parts, at = [], 0
    for b in zero_sizes:
        parts.append(zero[at:at + b])
        at += b
    ws1, ws2, ws3 = parts[:3]
    ranges = parts[3][:tiles * 8].view(i32).view(tiles, 2)
    records = parts[4][:N * rec * 4].view(f32).view(N, rec)
    touched = parts[5][:N]
    grads = [parts[6 + k][:t.numel() * 4].view(f32).view(t.shape) for k, t in
             enumerate((model.xyz, model.quaternion_xyzw, model.scale, model.opacity, model.color_sh))]
    order = torch.empty(tiles, dtype=i32, device=dev)
    total = torch.empty(1, dtype=torch.int64, device=dev)
    host_total = torch.full((1,), -1, dtype=torch.int64).pin_memory()
    color = torch.empty((H, W, 3), dtype=f32, device=dev)
    T, nc = torch.empty((H, W), dtype=f32, device=dev), torch.empty((H, W), dtype=i32, device=dev)
    drgb = torch.from_numpy(rng.standard_normal((H, W, 3)).astype(np.float32)).cuda()
    dT = torch.from_numpy(rng.standard_normal((H, W)).astype(np.float32)).cuda()
    picked = {}

    def view():
        """One view on the current stream: no allocation, no synchronisation."""
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        zero.zero_()
        _capi.check(L.d3gs_preprocess_fwd(C.byref(P), p(model.xyz), p(model.quaternion_xyzw), p(model.scale), p(model.opacity),
                                          p(model.color_sh), None, None, p(depths), p(radii), p(uvs), p(conic),
                                          p(touched_tiles), p(rgb), p(cov2d), p(ne0), p(tile_masks), p(dk_a), None, s), "K1")
        order_in_b, pairs_in_b = C.c_int(-1), C.c_int(-1)
        _capi.check(L.d3gs_bin_pairs(C.byref(P), p(radii), p(uvs), p(conic), p(depths), p(touched_tiles), p(tile_masks),
                                     p(dk_a), p(dk_b), p(ord_a), p(ord_b), p(ws1), sizes[0], p(offs), p(ws2), sizes[1],
                                     p(total), C.c_void_p(host_total.data_ptr()), cap, p(tk_a), p(tk_b), p(ix_a), p(ix_b),
                                     p(ws3), sizes[2], p(ranges), p(order), _capi.BIN_WORKSPACES_ARE_ZERO,
                                     C.byref(order_in_b), C.byref(pairs_in_b), s), "bin_pairs")
        idx = ix_b if pairs_in_b.value else ix_a
        picked["idx"] = idx
        _capi.check(L.d3gs_blend_fwd(C.byref(P), p(ranges), p(idx), p(uvs), p(conic), p(rgb), None, p(order), p(color), p(T),
                                     p(nc), None, None, 0, s), "blend_fwd")
        _capi.check(L.d3gs_blend_bwd(C.byref(P), p(ranges), p(idx), p(uvs), p(conic), p(rgb), None, p(order), p(T), p(nc),
                                     p(color), None, p(drgb), p(dT), None, p(records), p(touched), s), "blend_bwd")
        _capi.check(L.d3gs_preprocess_bwd(C.byref(P), p(model.xyz), p(model.quaternion_xyzw), p(model.scale), p(model.opacity),
                                          p(model.color_sh), p(radii), p(cov2d), p(ne0), p(records), p(touched), 0, 1,
                                          p(grads[0]), p(grads[1]), p(grads[2]), p(grads[3]), p(grads[4]), None, None, s), "K9")

    def results():
        m = int(host_total[0])
        return dict(m=m, color=color.clone(), T=T.clone(), nc=nc.clone(), idx=picked["idx"][:m].clone(),
                    ranges=ranges.clone(), grads=[g.clone() for g in grads])

    view()                                  # (the library's one-time set-up happens outside the capture)
    torch.cuda.synchronize()
    first = results()
    assert 0 < first["m"] <= cap
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        view()
    busy = torch.randn(512, 512, device=dev)
    for replay in range(4):
        if replay:      # the model moves between the views, as under an optimizer
            model.xyz.add_(torch.from_numpy((0.02 * rng.standard_normal(model.xyz.shape)).astype(np.float32)).cuda())
        view()
        torch.cuda.synchronize()
        eager = results()
        for t in (color, T, records, *grads):      # nothing of the eager view may pass for the replay's result
            t.fill_(float("nan"))
        nc.fill_(-1)
        host_total[0] = -7
        busy = busy @ busy.T * 1e-3                 # unrelated eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = results()
        assert got["m"] == eager["m"] and 0 < got["m"] <= cap, (replay, got["m"], eager["m"])
        if replay:
            assert eager["m"] != first["m"] or not torch.equal(eager["color"], first["color"])    # the view did change
        for key in ("color", "T", "nc", "idx", "ranges"):
            assert torch.equal(got[key], eager[key]), (replay, key)
        for k, (a, b) in enumerate(zip(got["grads"], eager["grads"])):      # sums of atomics: equal to their order
            assert bool(torch.isfinite(a).all())
            assert float((a - b).abs().max()) <= 1e-3 * float(b.abs().max()) + 1e-30, (replay, k)

    # what the capture buys a small view, whose launches cost more than its kernels (printed, not asserted)
    def timed(fn, reps=30):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / reps
    print(f"  view of {scene.n} gaussians, M={first['m']}: {timed(view):.3f} ms as eager calls, "
          f"{timed(graph.replay):.3f} ms as a graph replay", flush=True)
