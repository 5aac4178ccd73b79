"""Sparse mode (config sparse_mode; render.py:234-238, 478-500, 622-640, 2857-2918): everything behind the preprocess
works on the accepted gaussians only.  The render must be the dense one bit for bit, the compact arrays the dense ones'
accepted rows, and the sparse gradient the dense gradient's rows of the accepted gaussians."""
import numpy as np
import pytest

from helpers import gen_scene, grad_close, op_config, oracle_forward, torch_model

pytestmark = pytest.mark.gpu


def _narrow_scene():
    """A view that sees a part of the model: half of the gaussians are moved behind the camera or far to the side."""
    scene = gen_scene(1, n=30000, wh=(320, 240))
    rng = np.random.default_rng(12)
    away = rng.random(scene.n) < 0.5
    scene.xyz[away, 2] -= 20.0
    scene.xyz[rng.random(scene.n) < 0.1, 0] += 50.0
    return scene


@pytest.mark.parametrize("filt,views", [(1, 1), (4, 2)])
def test_sparse_equals_dense(oracle, filt, views):
    import torch
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    scene = _narrow_scene()
    model = torch_model(scene)
    mask = torch.from_numpy(np.random.default_rng(2).random(scene.n) < 0.1).cuda()
    dT = torch.from_numpy(np.random.default_rng(7).standard_normal(scene.dT.shape).astype(np.float32)).cuda()
    grads = GaussianSplatGradients(drgb=torch.from_numpy(scene.drgb).cuda(), dT=dT)
    res = {}
    for sparse in (False, True):
        op = GaussianSplatOp(op_config(scene, filt, sparse_mode=sparse))
        for _ in range(views):
            out, ctx = op.forward(model, scene.camera(), training=True, mask=mask)
        gm, duv, _ = op.backward(model, scene.camera(), ctx, out, grads, return_uv_grad=True)
        torch.cuda.synchronize()
        res[sparse] = (op, out, ctx, gm, duv, op._last_keys_sorted.clone())
    (_, out_d, ctx_d, gm_d, duv_d, keys_d), (op_s, out_s, ctx_s, gm_s, duv_s, keys_s) = res[False], res[True]
    ids = out_s.sparse_gaussian_ids.long()
    accepted = torch.nonzero(out_d.radii > 0).squeeze(1)
    assert 0 < ids.numel() < scene.n // 2 and torch.equal(ids, accepted)           # ascending, exactly the accepted
    assert torch.equal(out_s.sparse_batch_ids, torch.zeros_like(out_s.sparse_batch_ids))
    assert not bool(mask[ids].any())
    # image and per-pixel outputs: the dense render, bit for bit
    for name in ("color", "T", "n_contrib"):
        assert torch.equal(getattr(out_s, name), getattr(out_d, name)), name
    # compact arrays = accepted rows of the dense ones
    assert torch.equal(out_s.radii, out_d.radii[ids])
    for name in ("depths", "uvs", "conic_opacity", "rgb_gaussian", "cov2d_vecs", "sh_to_rgb_ne_0"):
        assert torch.equal(getattr(ctx_s, name), getattr(ctx_d, name)[ids]), name
    # the same lists: sorted keys, ranges, and the sorted rows name the same gaussians
    assert torch.equal(keys_s, keys_d) and torch.equal(ctx_s.workload_ranges, ctx_d.workload_ranges)
    assert torch.equal(ids[ctx_s.gaussian_idx_sorted.long()], ctx_d.gaussian_idx_sorted.long())
    # sparse gradient: one row per accepted gaussian = the dense gradient's rows; the rest of the dense one is zero
    assert tuple(duv_s.shape) == (1, ids.numel(), 2)
    top = float(duv_d.abs().max())
    assert float((duv_s[0] - duv_d[0][ids]).abs().max()) <= 1e-4 * top
    rest = torch.ones(scene.n, dtype=torch.bool, device="cuda")
    rest[ids] = False
    for name in ("xyz", "quaternion_xyzw", "scale", "opacity", "color_sh"):
        a, b = getattr(gm_s, name).double(), getattr(gm_d, name).double()
        assert a.shape[0] == ids.numel() and tuple(a.shape[1:]) == tuple(b.shape[1:]), name
        err = (a - b[ids]).abs().reshape(-1)
        scale = float(b.abs().max())
        assert float(torch.quantile(err[:: max(1, err.numel() // 1_000_000)], 0.999)) <= 1e-4 * scale and float(err.max()) <= 1e-3 * scale, name
        assert float(b[rest].abs().max()) == 0.0, name
    # and against the oracle (dense), gathered
    P, ref = oracle_forward(oracle, scene, filt)
    ref = oracle.forward(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                         invalid_mask=mask.cpu().numpy())
    assert np.array_equal(out_s.color.cpu().numpy()[0].view(np.uint32), ref["color"].view(np.uint32))
    g_ref, pb_ref = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                                    scene.drgb[0], dT.cpu().numpy()[0])
    ok, worst, nbad = grad_close(gm_s.xyz.cpu().numpy(), pb_ref["dxyz"][ids.cpu().numpy()], rel=1e-3, abs_frac=1e-4)
    assert ok, (worst, nbad)


def test_sparse_inference_and_empty_view():
    import torch
    from d3gs_research_amd.render import GaussianSplatOp
    scene = _narrow_scene()
    model = torch_model(scene)
    op_d = GaussianSplatOp(op_config(scene, 4, bg_color=np.array([0.2, 0.4, 0.6], np.float32)))
    op_s = GaussianSplatOp(op_config(scene, 4, sparse_mode=True, bg_color=np.array([0.2, 0.4, 0.6], np.float32)))
    out_d, _ = op_d.forward(model, scene.camera(), training=False)
    out_s, ctx = op_s.forward(model, scene.camera(), training=False)
    assert ctx is None and torch.equal(out_s.color, out_d.color) and out_s.sparse_gaussian_ids.numel() > 0
    # nothing accepted: every gaussian masked out
    everything = torch.ones(scene.n, dtype=torch.bool, device="cuda")
    out_e, ctx_e = op_s.forward(model, scene.camera(), training=True, mask=everything)
    assert ctx_e is None and out_e.sparse_gaussian_ids.numel() == 0 and out_e.radii.numel() == 0
    assert float(out_e.T.min()) == 1.0 and float(out_e.color.abs().max()) == 0.0


@pytest.mark.parametrize("one_pass", [True, False])
def test_sparse_bundle_merges_the_cameras_rows(one_pass):
    """A sparse bundle, in one pass over the B * N items (compact rows behind K1, K9 with a camera per row) and
    camera by camera: the dense bundle's images, its accepted items' rows, and gradients merged per gaussian."""
    import torch
    from d3gs_research_amd.render import CameraBundle, GaussianSplatGradients, GaussianSplatOp
    from test_gpu_camera_bundle import _cameras
    scene = _narrow_scene()
    cams = _cameras(scene)
    B = len(cams)
    model = torch_model(scene)
    bundle = CameraBundle.from_pinhole_cams(cams)
    rng = np.random.default_rng(4)
    res = {}
    for sparse in (False, True):
        op = GaussianSplatOp(op_config(scene, 4, sparse_mode=sparse))
        op.bundle_in_one_pass = one_pass or not sparse
        for _ in range(2):      # the second view takes the one-call binning
            out, ctx = op.forward(model, bundle, training=True)
        if sparse:
            from d3gs_research_amd.render import GaussianSplatOpBatchContext
            assert isinstance(ctx, GaussianSplatOpBatchContext) != one_pass
        if not res:
            drgb = torch.from_numpy(rng.standard_normal(out.color.shape).astype(np.float32)).cuda()
            dT = torch.from_numpy(rng.standard_normal(out.T.shape).astype(np.float32)).cuda()
        gm, duv, _ = op.backward(model, bundle, ctx, out, GaussianSplatGradients(drgb=drgb, dT=dT), return_uv_grad=True)
        torch.cuda.synchronize()
        res[sparse] = (op, out, gm, duv)
    (_, out_d, gm_d, duv_d), (op_s, out_s, gm_s, duv_s) = res[False], res[True]
    assert torch.equal(out_s.color, out_d.color) and torch.equal(out_s.n_contrib, out_d.n_contrib)
    # rows of camera 0, then camera 1, ...: exactly the accepted (camera, gaussian) items of the dense bundle
    items = torch.nonzero(out_d.radii > 0).squeeze(1)
    assert torch.equal(out_s.sparse_batch_ids.long() * scene.n + out_s.sparse_gaussian_ids.long(), items)
    assert torch.equal(out_s.radii, out_d.radii[items])
    top = float(duv_d.abs().max())
    assert float((duv_s[0] - duv_d.reshape(B * scene.n, 2)[items]).abs().max()) <= 1e-4 * top
    unique = op_s.last_sparse_unique_ids.long()
    assert torch.equal(unique, torch.unique(out_s.sparse_gaussian_ids.long()))
    for name in ("xyz", "quaternion_xyzw", "scale", "opacity", "color_sh"):
        a, b = getattr(gm_s, name).double(), getattr(gm_d, name).double()
        assert a.shape[0] == unique.numel(), name
        err = (a - b[unique]).abs().reshape(-1)
        scale = float(b.abs().max())
        assert float(torch.quantile(err[:: max(1, err.numel() // 1_000_000)], 0.999)) <= 1e-4 * scale and float(err.max()) <= 1e-3 * scale, name


@pytest.mark.parametrize("count,id_limit", [(0, 10), (1, 1), (257, 40), (100_003, 30_000), (1_000_000, 3_000_000)])
def test_unique_ids_and_merge_rows_c_abi(count, id_limit):
    """d3gs_unique_ids / d3gs_merge_rows (the deduplication of a sparse bundle's rows, render.py:2864-2903) against
    numpy.unique and a sequential float32 sum of each run's rows in run order."""
    import torch
    from d3gs_research_amd.render import GaussianSplatOp
    scene = gen_scene(0, n=16)
    op = GaussianSplatOp(op_config(scene, 1))
    rng = np.random.default_rng(count)
    ids = rng.integers(0, id_limit, count).astype(np.int32)
    unique, run_rows, run_starts = op.unique_ids(torch.from_numpy(ids).cuda(), id_limit)
    torch.cuda.synchronize()
    want, inverse = np.unique(ids, return_inverse=True)
    U = want.size
    assert np.array_equal(unique.cpu().numpy(), want)
    if count == 0:
        return
    assert np.array_equal(op.last_unique_inverse.cpu().numpy(), inverse)
    rr, rs = run_rows.cpu().numpy(), run_starts.cpu().numpy()[:U + 1]
    assert rs[0] == 0 and rs[U] == count and (np.diff(rs) > 0).all()
    assert np.array_equal(ids[rr], np.sort(ids, kind="stable"))
    assert np.array_equal(rr, np.argsort(ids, kind="stable"))         # rows of equal id keep their input order
    for width in (1, 3, 48):
        if count * width > 4_000_000:
            continue
        rows = rng.standard_normal((count, width)).astype(np.float32)
        merged = op.merge_rows(torch.from_numpy(rows).cuda(), run_rows, run_starts, U).cpu().numpy()
        ref = np.zeros((U, width), np.float32)
        longest = int(np.diff(rs).max())
        for k in range(longest):                                       # k-th row of every run that has one
            has = rs[:-1] + k < rs[1:]
            ref[has] = ref[has] + rows[rr[rs[:-1][has] + k]]
        assert np.array_equal(merged.view(np.uint32), ref.view(np.uint32))


@pytest.mark.parametrize("one_pass", [True, False])
def test_sparse_bundle_with_a_camera_that_renders_no_pair(one_pass):
    """A camera can accept gaussians (their 3-sigma rect meets the image) and still end without a single (tile,
    gaussian) pair (OBB keeps no tile of any of them): it has rows in out.radii / out.sparse_gaussian_ids but no
    context.  The rows of the cameras behind it must still line up, its own duv rows are zero."""
    import torch
    from d3gs_research_amd.camera import BasicPinholeCamera
    from d3gs_research_amd.render import CameraBundle, GaussianSplatGradients, GaussianSplatOp
    scene = gen_scene(1, n=4000, wh=(320, 240))
    # three faint gaussians just left of the image as the FIRST camera sees it: their 3-sigma rect reaches into
    # tile column 0, the ellipse of alpha >= 1/255 (opacity barely above 1/255) does not
    z = 4.0
    for k in range(3):
        scene.xyz[k] = [(-164.0 - k) * z / scene.fx, (k - 1) * 20.0 * z / scene.fy, 0.0]
        scene.scale[k] = np.log(4.0 * z / scene.fx)
        scene.opacity[k] = np.log(0.0046 / (1 - 0.0046))
    model = torch_model(scene)
    mask0 = np.ones(scene.n, bool)
    mask0[:3] = False                          # camera 0 sees only the three
    mask = np.concatenate([mask0, np.zeros(scene.n, bool), np.zeros(scene.n, bool)])
    tw = np.array(scene.to_world, np.float64)
    cams = []
    for dx in (0.0, 0.25, -0.25):
        t = tw.copy()
        t[0, 3] += dx
        cams.append(BasicPinholeCamera.from_params(scene.fx, scene.fy, scene.cx, scene.cy, scene.width, scene.height, t))
    bundle = CameraBundle.from_pinhole_cams(cams)
    mask_t = torch.from_numpy(mask).cuda()
    rng = np.random.default_rng(5)
    res = {}
    for sparse in (False, True):
        op = GaussianSplatOp(op_config(scene, 3, sparse_mode=sparse))
        op.bundle_in_one_pass = one_pass or not sparse
        out, ctx = op.forward(model, bundle, training=True, mask=mask_t)
        if not res:
            drgb = torch.from_numpy(rng.standard_normal(out.color.shape).astype(np.float32)).cuda()
            dT = torch.zeros_like(out.T)
        gm, duv, _ = op.backward(model, bundle, ctx, out, GaussianSplatGradients(drgb=drgb, dT=dT), return_uv_grad=True)
        torch.cuda.synchronize()
        res[sparse] = (op, out, ctx, gm, duv)
    (_, out_d, _, gm_d, duv_d), (op_s, out_s, ctx_s, gm_s, duv_s) = res[False], res[True]
    B = 3
    items = torch.nonzero(out_d.radii > 0).squeeze(1)
    first = items[items < scene.n]
    assert first.numel() == 3                                                  # accepted, and no pair:
    if one_pass:
        assert int((ctx_s.workload_ranges[:ctx_s.workload_ranges.shape[0] // B, 1] - ctx_s.workload_ranges[:ctx_s.workload_ranges.shape[0] // B, 0]).sum()) == 0
    else:
        assert ctx_s.per_camera[0] is None and ctx_s.rows_per_camera[0] == 3
    assert float(out_s.T[0].min()) == 1.0
    assert torch.equal(out_s.sparse_batch_ids.long() * scene.n + out_s.sparse_gaussian_ids.long(), items)
    assert torch.equal(out_s.color, out_d.color)
    assert tuple(duv_s.shape) == (1, items.numel(), 2) and float(duv_s[0, :3].abs().max()) == 0.0
    B = 3
    top = float(duv_d.abs().max())
    assert float((duv_s[0] - duv_d.reshape(B * scene.n, 2)[items]).abs().max()) <= 1e-4 * top
    unique = op_s.last_sparse_unique_ids.long()
    # camera by camera the first camera contributes no gradient row; in one pass its three rows are there, and zero
    seen = torch.unique(out_s.sparse_gaussian_ids.long() if one_pass else out_s.sparse_gaussian_ids[3:].long())
    assert torch.equal(unique, seen)
    for name in ("xyz", "scale", "opacity", "color_sh"):
        a, b = getattr(gm_s, name).double(), getattr(gm_d, name).double()
        scale = float(b.abs().max())
        assert float((a - b[unique]).abs().max()) <= 1e-3 * scale, name


def test_sparse_mode_with_instances(oracle):
    """sparse_mode with instance poses: the compact pass must equal the dense instance render (bit for bit) and the
    oracle's, and its sparse gradient the oracle's rows of the accepted gaussians."""
    import torch
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    from helpers import oracle_params
    from test_gpu_instances import _setup
    scene = _narrow_scene()
    K = 5
    T, ids_np, model, cam = _setup(scene, K, 77)
    T_dev = torch.from_numpy(T).cuda()
    grads = GaussianSplatGradients(drgb=torch.from_numpy(scene.drgb).cuda(), dT=torch.from_numpy(scene.dT).cuda())
    res = {}
    for sparse in (False, True):
        op = GaussianSplatOp(op_config(scene, 4, sparse_mode=sparse))
        for _ in range(2):
            out, ctx = op.forward(model, cam, training=True, instance2world_T=T_dev)
        gm, duv, _ = op.backward(model, cam, ctx, out, grads, return_uv_grad=True)
        torch.cuda.synchronize()
        res[sparse] = (op, out, ctx, gm, duv)
    (op_d, out_d, ctx_d, gm_d, _), (_, out_s, ctx_s, gm_s, _) = res[False], res[True]
    ids = out_s.sparse_gaussian_ids.long()
    assert 0 < ids.numel() < scene.n and torch.equal(ids, torch.nonzero(out_d.radii > 0).squeeze(1))
    for name in ("color", "T", "n_contrib"):
        assert torch.equal(getattr(out_s, name), getattr(out_d, name)), name
    for name in ("uvs", "conic_opacity", "rgb_gaussian", "cov2d_vecs"):
        assert torch.equal(getattr(ctx_s, name), getattr(ctx_d, name)[ids]), name
    _, table = op_d.instance_table(model, cam, T_dev)
    inst = (ids_np, table.cpu().numpy())
    P = oracle_params(oracle, scene, 4)
    args = (scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    ref = oracle.forward(P, *args, instances=inst)
    assert np.array_equal(out_s.color.cpu().numpy()[0].view(np.uint32), ref["color"].view(np.uint32))
    _, pb_ref = oracle.backward(P, ref, *args, scene.drgb[0], scene.dT[0], instances=inst)
    sel = ids.cpu().numpy()
    for name, got in (("dxyz", gm_s.xyz), ("dscale", gm_s.scale), ("dopacity", gm_s.opacity), ("dsh", gm_s.color_sh)):
        ok, worst, nbad = grad_close(got.cpu().numpy(), pb_ref[name][sel], rel=1e-3, abs_frac=1e-4)
        assert ok, (name, worst, nbad)
