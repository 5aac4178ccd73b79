"""A bundle rendered in one pass (B * N render items, the reference's way, render.py:314-326) against the same bundle
rendered camera by camera, over randomised option combinations: depth / RGBA / NCHW / anti-aliasing / 32-bit sort /
custom features / instance poses with a frame per camera / reject mask / disable_builtin_rgb, training or inference.
Images must be identical, gradients equal to the order of their sums.  Each way is checked against the oracle
elsewhere (test_gpu_camera_bundle.py, test_gpu_instances.py); this file is about the combinations."""
import numpy as np
import pytest

from helpers import gen_scene, op_config, torch_model
from test_gpu_camera_bundle import _cameras
from test_oracle_instances import _poses

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(12))
def test_one_pass_equals_camera_by_camera(seed):
    import torch
    from d3gs_research_amd.render import CameraBundle, GaussianSplatGradients, GaussianSplatOp
    scene = gen_scene(1, n=15000, wh=(250, 190))
    cams = _cameras(scene)
    B, n = len(cams), scene.n
    r = np.random.default_rng(100 + seed)
    f = {k: bool(r.integers(0, 2)) for k in ("depth", "rgba", "nchw", "aa", "s32", "feat", "inst", "mask", "norgb", "infer")}
    if f["feat"] or f["norgb"]:
        f["nchw"] = False      # not combined in the reference either
    print(f"seed {seed}: " + " ".join(k for k, v in f.items() if v), flush=True)
    over = dict(render_depth=f["depth"], render_rgba=f["rgba"], use_nchw=f["nchw"], enable_anti_aliasing=f["aa"],
                enable_32bit_sort=f["s32"], depth_32bit_prec=0.01, disable_builtin_rgb=f["norgb"])
    model = torch_model(scene)
    bundle = CameraBundle.from_pinhole_cams(cams)
    T_dev = None
    if f["inst"]:
        K = 3
        T = np.stack([_poses(r, K, angle=0.1, shift=0.1)[3] for _ in range(2)], 0)      # two frames of K poses
        model.instance_id = torch.from_numpy(r.integers(-1, K, n).astype(np.int32)).cuda()
        T_dev = torch.from_numpy(T.astype(np.float32)).cuda()
        bundle.frame_ids = torch.tensor([0, 1, 0], dtype=torch.int64, device="cuda")
    feat = torch.from_numpy(r.standard_normal((B * n, 4)).astype(np.float32)).cuda() if f["feat"] else None
    mask = torch.from_numpy(r.random(B * n) < 0.2).cuda() if f["mask"] else None
    t = lambda shape: torch.from_numpy(r.standard_normal(tuple(shape)).astype(np.float32)).cuda()
    res, g = [], None
    for one_pass in (True, False):
        op = GaussianSplatOp(op_config(scene, 4, **over))
        op.bundle_in_one_pass = one_pass
        op.bundle_k9_in_one_launch = bool(seed % 2)      # the preprocess backward: one launch, or one per camera
        out, ctx = op.forward(model, bundle, training=not f["infer"], instance2world_T=T_dev, custom_features=feat,
                              mask=mask)
        gm = duv = dcf = None
        if not f["infer"]:
            if g is None:
                g = GaussianSplatGradients(drgb=t(out.color.shape), dT=t(out.T.shape),
                                           ddepth=t(out.T.shape) if f["depth"] else None,
                                           dcustom_features=t(out.custom_features.shape) if f["feat"] else None)
            gm, duv, dcf = op.backward(model, bundle, ctx, out, g, return_uv_grad=True, instance2world_T=T_dev)
        res.append((out, gm, duv, dcf))
    (o1, g1, d1, c1), (o2, g2, d2, c2) = res
    assert torch.equal(o1.color, o2.color) and torch.equal(o1.T, o2.T) and torch.equal(o1.n_contrib, o2.n_contrib)
    assert torch.equal(o1.radii, o2.radii)
    if f["depth"]:      # inference divides by 1 - T: pixels nothing reached hold 0 / 0 on both sides
        assert torch.equal(torch.nan_to_num(o1.depth, nan=-1.0), torch.nan_to_num(o2.depth, nan=-1.0))
    if f["feat"]:
        assert torch.equal(o1.custom_features, o2.custom_features)
    if f["infer"]:
        return
    assert float((d1 - d2).abs().max()) <= 1e-4 * float(d2.abs().max())
    if f["feat"]:
        assert float((c1 - c2).abs().max()) <= 1e-4 * float(c2.abs().max())
    for k in ("xyz", "scale", "quaternion_xyzw", "opacity", "color_sh"):
        a, b = getattr(g1, k).double(), getattr(g2, k).double()
        assert float((a - b).abs().max()) <= 2e-3 * float(b.abs().max()) + 1e-30, k


@pytest.mark.parametrize("seed", range(8))
def test_sparse_bundle_one_pass_equals_camera_by_camera_and_dense(seed):
    """sparse_mode bundles over the options sparse mode takes (render.py:234-238 excludes custom features): the one
    pass over compact rows, the camera-by-camera path and the dense bundle give the same images; the sparse rows are
    the dense arrays at the accepted items; merged gradients are the dense ones at the distinct gaussians."""
    import torch
    from d3gs_research_amd.render import CameraBundle, GaussianSplatGradients, GaussianSplatOp
    scene = gen_scene(1, n=15000, wh=(250, 190))
    cams = _cameras(scene)
    B, n = len(cams), scene.n
    r = np.random.default_rng(500 + seed)
    f = {k: bool(r.integers(0, 2)) for k in ("depth", "rgba", "nchw", "aa", "s32", "inst", "mask", "infer")}
    print(f"seed {seed}: " + " ".join(k for k, v in f.items() if v), flush=True)
    over = dict(render_depth=f["depth"], render_rgba=f["rgba"], use_nchw=f["nchw"], enable_anti_aliasing=f["aa"],
                enable_32bit_sort=f["s32"], depth_32bit_prec=0.01)
    model = torch_model(scene)
    bundle = CameraBundle.from_pinhole_cams(cams)
    T_dev = None
    if f["inst"]:
        K = 3
        T = np.stack([_poses(r, K, angle=0.1, shift=0.1)[3] for _ in range(2)], 0)
        model.instance_id = torch.from_numpy(r.integers(-1, K, n).astype(np.int32)).cuda()
        T_dev = torch.from_numpy(T.astype(np.float32)).cuda()
        bundle.frame_ids = torch.tensor([0, 1, 0], dtype=torch.int64, device="cuda")
    mask = torch.from_numpy(r.random(B * n) < 0.2).cuda() if f["mask"] else None
    t = lambda shape: torch.from_numpy(r.standard_normal(tuple(shape)).astype(np.float32)).cuda()
    res, g = {}, None
    for name, sparse, one_pass in (("dense", False, True), ("one", True, True), ("each", True, False)):
        op = GaussianSplatOp(op_config(scene, 4, sparse_mode=sparse, **over))
        op.bundle_in_one_pass = one_pass
        for _ in range(2):      # the second view of an op takes the one-call binning with buffers sized by the first
            out, ctx = op.forward(model, bundle, training=not f["infer"], instance2world_T=T_dev, mask=mask)
        gm = duv = None
        if not f["infer"]:
            if g is None:
                g = GaussianSplatGradients(drgb=t(out.color.shape), dT=t(out.T.shape),
                                           ddepth=t(out.T.shape) if f["depth"] else None)
            gm, duv, _ = op.backward(model, bundle, ctx, out, g, return_uv_grad=True, instance2world_T=T_dev)
        torch.cuda.synchronize()
        res[name] = (op, out, gm, duv)
    (_, od, gd, dd), (op1, o1, g1, d1), (op2, o2, g2, d2) = res["dense"], res["one"], res["each"]
    for o in (o1, o2):
        assert torch.equal(o.color, od.color) and torch.equal(o.T, od.T) and torch.equal(o.n_contrib, od.n_contrib)
        if f["depth"]:
            assert torch.equal(torch.nan_to_num(o.depth, nan=-1.0), torch.nan_to_num(od.depth, nan=-1.0))
    items = o1.sparse_batch_ids.long() * n + o1.sparse_gaussian_ids.long()
    assert torch.equal(o1.sparse_gaussian_ids, o2.sparse_gaussian_ids) and torch.equal(o1.sparse_batch_ids, o2.sparse_batch_ids)
    assert bool((items[1:] > items[:-1]).all())
    assert torch.equal(o1.radii, od.radii.reshape(-1)[items]) and torch.equal(o2.radii, o1.radii)
    if f["infer"]:
        return
    top = float(dd.abs().max())
    dense_rows = dd.reshape(-1, 2)[items]
    for d in (d1, d2):
        assert tuple(d.shape) == (1, items.numel(), 2)
        assert float((d[0] - dense_rows).abs().max()) <= 1e-4 * top
    unique = op1.last_sparse_unique_ids.long()
    assert torch.equal(unique, torch.unique(o1.sparse_gaussian_ids.long()))
    for k in ("xyz", "scale", "quaternion_xyzw", "opacity", "color_sh"):
        want = getattr(gd, k).double()[unique]
        bar = 2e-3 * float(want.abs().max()) + 1e-30
        assert float((getattr(g1, k).double() - want).abs().max()) <= bar, k
        # camera by camera the merged rows only name gaussians of cameras that rendered a pair
        rows2 = op2.last_sparse_unique_ids.long()
        assert float((getattr(g2, k).double() - getattr(gd, k).double()[rows2]).abs().max()) <= bar, k
