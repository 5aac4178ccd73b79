"""rasterize_backward_algo = PER_GAUSSIAN (render.py:2319-2776): the second backward algorithm, lanes = gaussians,
pixels handed from lane to lane, state in front of each bucket from the forward's snapshots.  Same gradient as the
default kernel: judged against the oracle with the default kernel's bars, and against the default kernel itself."""
import numpy as np
import pytest

from helpers import gen_scene, grad_close, k9_noise_spread, op_config, oracle_forward, per_gaussian_rel_err, torch_model

pytestmark = pytest.mark.gpu

NONE, AABB, OBB, DFVT = 0, 1, 3, 4


@pytest.mark.parametrize("cfg_id,n,wh,filt,views", [(0, None, None, AABB, 1), (1, 20000, (250, 190), OBB, 2),
                                                    (2, 100000, (640, 360), DFVT, 2), (4, 30000, (960, 540), AABB, 1),
                                                    (1, None, None, DFVT, 2), (2, None, None, DFVT, 2)])
def test_per_gaussian_backward_parity(oracle, cfg_id, n, wh, filt, views):
    import torch
    from d3gs_research_amd.config_def import RasterizeBackwardAlgo
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    scene = gen_scene(cfg_id, n=n, wh=wh)
    print(f"per-gaussian case cfg={cfg_id} n={scene.n} wh={scene.width}x{scene.height} filter={filt} views={views}", flush=True)
    dT = np.random.default_rng(7).standard_normal(scene.dT.shape).astype(np.float32)
    P, ref = oracle_forward(oracle, scene, filt)
    g_ref, pb_ref = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity,
                                    scene.color_sh, scene.drgb[0], dT[0])
    model = torch_model(scene)
    grads = GaussianSplatGradients(drgb=torch.from_numpy(scene.drgb).cuda(), dT=torch.from_numpy(dT).cuda())
    cpu = lambda t: t.detach().cpu().numpy()
    results = {}
    for algo in (RasterizeBackwardAlgo.PER_GAUSSIAN, RasterizeBackwardAlgo.DEFAULT):
        op = GaussianSplatOp(op_config(scene, filt, rasterize_backward_algo=algo))
        for _ in range(views):
            out, ctx = op.forward(model, scene.camera(), training=True)
        assert (ctx.per_gaussian_snap is not None) == (algo == RasterizeBackwardAlgo.PER_GAUSSIAN)
        # the forward that stores snapshots renders the same image, bit for bit
        assert np.array_equal(cpu(out.color)[0].view(np.uint32), ref["color"].view(np.uint32))
        assert np.array_equal(cpu(out.n_contrib)[0], ref["n_contrib"])
        gm, duv, _ = op.backward(model, scene.camera(), ctx, out, grads, return_uv_grad=True)
        torch.cuda.synchronize()
        results[algo] = (op.last_raster_grads, gm)
    g, gm = results[RasterizeBackwardAlgo.PER_GAUSSIAN]
    g_def, gm_def = results[RasterizeBackwardAlgo.DEFAULT]
    # The bar.  dcolor = sum of w * drgb does not involve the pixels' colour state: the default kernel's bar,
    # 1e-4 * sum|terms|.  duv, dconic and dopacity go through dL/dalpha = drgb . (T c - colour behind) / (1 - alpha),
    # and this algorithm rebuilds "colour behind" in front of a bucket as final colour - snapshot, two float32 sums
    # rounded at the magnitude of the final colour (render.py:2601 does the same), where the default kernel and the
    # oracle subtract term by term: the two differ by a few ulp of the final colour per pixel, however small the
    # difference T c - colour behind is.  The oracle reports that sensitivity ("statemass": sum over pixels of
    # |d term / d dl| * sum_ch |drgb| |final colour|); measured, the deviation stays under 9 * 2^-24 * statemass with
    # a median of 0.1, which is what some hundred roundings of either sum amount to.  Bar: 16 * 2^-24 * statemass
    # on top of the default's.
    mass = np.array(g_ref["absmass"][:, :9])
    tol = 1e-4 * mass + 1e-30
    tol[:, :6] += 16 * 2.0 ** -24 * g_ref["statemass"]
    for name, got, cols in (("duv", g.duv, slice(0, 2)), ("dconic", g.dconic, slice(2, 5)),
                            ("dopacity", g.dopacity, slice(5, 6)), ("dcolor", g.dcolor, slice(6, 9))):
        a, b = cpu(got).astype(np.float64).reshape(scene.n, -1), g_ref[name].reshape(scene.n, -1)
        excess = np.abs(a - b) - tol[:, cols]
        assert (excess <= 0).all(), f"{name}: {int((excess > 0).sum())} values beyond the bar"
        assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(b), f"{name}: relative L2 error {np.linalg.norm(a - b) / np.linalg.norm(b):.2e}"
    ok, worst, nbad = grad_close(cpu(g.dcolor), g_ref["dcolor"])
    assert ok, f"dcolor: {nbad} elements outside tolerance (worst {worst:.2f}x)"
    # the same gaussians receive a gradient under both algorithms
    assert torch.equal(g.touched != 0, g_def.touched != 0)
    spread = k9_noise_spread(oracle, P, scene, ref, g_ref, pb_ref, state_ulps=4.0)
    for name, got in (("dxyz", gm.xyz), ("dquat", gm.quaternion_xyzw), ("dscale", gm.scale),
                      ("dopacity", gm.opacity), ("dsh", gm.color_sh)):
        med, p99 = np.quantile(per_gaussian_rel_err(cpu(got), pb_ref[name]), [0.5, 0.99])
        m_med, m_p99 = spread[name]
        assert med <= 2 * m_med and p99 <= 2 * m_p99, \
            f"{name}: per-gaussian relative error median {med:.2e} p99 {p99:.2e}; noise model {m_med:.2e} {m_p99:.2e}"


def test_bucket_offsets_c_abi():
    import ctypes as C
    import torch
    from d3gs_research_amd import _capi
    L = _capi.lib()
    rng = np.random.default_rng(3)
    for tiles in (1, 63, 1024, 1025, 32400):
        lens = rng.integers(0, 700, size=tiles).astype(np.int32)
        lens[rng.random(tiles) < 0.2] = 0
        start = np.concatenate([[0], np.cumsum(lens)[:-1]]).astype(np.int32)
        ranges = np.stack([start, start + lens], 1).astype(np.int32)
        ranges[lens == 0] = 0         # untouched tiles read [0, 0)
        out = torch.full((tiles + 1,), -1, dtype=torch.int32, device="cuda")
        s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
        _capi.check(L.d3gs_bucket_offsets(_capi.ptr(torch.from_numpy(ranges).cuda()), tiles, _capi.ptr(out), s), "buckets")
        want = np.concatenate([[0], np.cumsum((lens + 63) // 64)])
        assert np.array_equal(out.cpu().numpy(), want.astype(np.int32))


def test_per_gaussian_backward_on_a_bundle():
    """The second algorithm over a bundle rendered in one pass (B * N render items, the camera in the tile id):
    same images, and gradients that agree with the default algorithm's to the order of their sums."""
    import torch
    from d3gs_research_amd.config_def import RasterizeBackwardAlgo
    from d3gs_research_amd.render import CameraBundle, GaussianSplatGradients, GaussianSplatOp
    from test_gpu_camera_bundle import _cameras
    scene = gen_scene(1, n=20000, wh=(250, 190))
    bundle = CameraBundle.from_pinhole_cams(_cameras(scene))
    model = torch_model(scene)
    rng = np.random.default_rng(0)
    res, drgb, dT = [], None, None
    for algo in (RasterizeBackwardAlgo.DEFAULT, RasterizeBackwardAlgo.PER_GAUSSIAN):
        op = GaussianSplatOp(op_config(scene, 4, rasterize_backward_algo=algo))
        out, ctx = op.forward(model, bundle, training=True)
        assert ctx.batch_size == len(bundle)
        if drgb is None:
            drgb = torch.from_numpy(rng.standard_normal(out.color.shape).astype(np.float32)).cuda()
            dT = torch.from_numpy(rng.standard_normal(out.T.shape).astype(np.float32)).cuda()
        gm, duv, _ = op.backward(model, bundle, ctx, out, GaussianSplatGradients(drgb=drgb, dT=dT), return_uv_grad=True)
        res.append((out, gm, duv))
    (o1, g1, d1), (o2, g2, d2) = res
    assert torch.equal(o1.color, o2.color) and torch.equal(o1.T, o2.T) and torch.equal(o1.n_contrib, o2.n_contrib)
    assert float((d1 - d2).abs().max()) <= 1e-5 * float(d1.abs().max())
    for k in ("xyz", "scale", "quaternion_xyzw", "opacity", "color_sh"):
        a, b = getattr(g1, k).double(), getattr(g2, k).double()
        assert float((a - b).abs().max()) <= 1e-3 * float(b.abs().max()), k


@pytest.mark.parametrize("depth,rgba,nchw", [(True, False, False), (False, True, False), (True, True, True)])
def test_per_gaussian_backward_with_depth_and_alpha_channels(oracle, depth, rgba, nchw):
    """The second algorithm with a depth and / or an alpha channel (render.py:2364-2398, 2412-2415, 2490-2528) and in
    the NCHW layout: the snapshots carry the channels' running sums, the gradient (dz included) is the oracle's to
    the bars of the plain per-gaussian test."""
    import torch
    from d3gs_research_amd.config_def import RasterizeBackwardAlgo
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    scene = gen_scene(1, n=30000, wh=(250, 190))
    print(f"per-gaussian channels depth={depth} rgba={rgba} nchw={nchw}", flush=True)
    filt = DFVT
    rng = np.random.default_rng(9)
    over = dict(render_depth=depth, render_rgba=rgba, use_nchw=nchw)
    P, ref = oracle_forward(oracle, scene, filt, **over)
    C_ = 3 + int(rgba)
    shape = (C_, scene.height, scene.width) if nchw else (scene.height, scene.width, C_)
    drgb = rng.standard_normal(shape).astype(np.float32)
    dT = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    ddepth = rng.standard_normal((scene.height, scene.width)).astype(np.float32) if depth else None
    g_ref, pb_ref = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity,
                                    scene.color_sh, drgb, dT, ddepth=ddepth)
    model = torch_model(scene)
    grads = GaussianSplatGradients(drgb=torch.from_numpy(drgb[None]).cuda(), dT=torch.from_numpy(dT[None]).cuda(),
                                   ddepth=None if ddepth is None else torch.from_numpy(ddepth[None]).cuda())
    cpu = lambda t: t.detach().cpu().numpy()
    op = GaussianSplatOp(op_config(scene, filt, rasterize_backward_algo=RasterizeBackwardAlgo.PER_GAUSSIAN, **over))
    for _ in range(2):
        out, ctx = op.forward(model, scene.camera(), training=True)
    assert ctx.per_gaussian_snap is not None and ctx.per_gaussian_snap[1].shape[-1] == 8
    assert np.array_equal(cpu(out.color)[0].view(np.uint32), ref["color"].view(np.uint32))
    if depth:
        assert np.array_equal(cpu(out.depth)[0].view(np.uint32), ref["depth"].view(np.uint32))
    gm, duv, _ = op.backward(model, scene.camera(), ctx, out, grads, return_uv_grad=True)
    torch.cuda.synchronize()
    g = op.last_raster_grads
    cols = 10 if depth else 9
    mass = np.array(g_ref["absmass"][:, :cols])
    tol = 1e-4 * mass + 1e-30
    tol[:, :6] += 16 * 2.0 ** -24 * g_ref["statemass"]
    checks = [("duv", g.duv, slice(0, 2)), ("dconic", g.dconic, slice(2, 5)), ("dopacity", g.dopacity, slice(5, 6)),
              ("dcolor", g.dcolor, slice(6, 9))]
    if depth:
        checks.append(("dz", g.dz, slice(9, 10)))
    for name, got, sl in checks:
        a, b = cpu(got).astype(np.float64).reshape(scene.n, -1), g_ref[name].reshape(scene.n, -1)
        excess = np.abs(a - b) - tol[:, sl]
        assert (excess <= 0).all(), f"{name}: {int((excess > 0).sum())} values beyond the bar"
        assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(b), f"{name}: relative L2 error {np.linalg.norm(a - b) / np.linalg.norm(b):.2e}"
    spread = k9_noise_spread(oracle, P, scene, ref, g_ref, pb_ref, state_ulps=4.0)
    for name, got in (("dxyz", gm.xyz), ("dscale", gm.scale), ("dopacity", gm.opacity), ("dsh", gm.color_sh)):
        med, p99 = np.quantile(per_gaussian_rel_err(cpu(got), pb_ref[name]), [0.5, 0.99])
        m_med, m_p99 = spread[name]
        print(f"  {name}: median {med:.2e} p99 {p99:.2e}; noise model {m_med:.2e} {m_p99:.2e}", flush=True)
        assert med <= 2 * m_med and p99 <= 2 * m_p99, f"{name}: median {med:.2e} p99 {p99:.2e}; noise model {m_med:.2e} {m_p99:.2e}"
        # the depth and alpha sums are rounded at the magnitude of their final values (a few units and up to one,
        # where most colours stay far below one), and so is the state this algorithm rebuilds from them
        # (final - snapshot): a wider fixed bar with either channel; the noise model above prices it in
        assert med <= 1e-4 and p99 <= 1e-2, f"{name}: median {med:.2e} p99 {p99:.2e}"


def test_per_gaussian_backward_with_custom_features(oracle):
    """Custom feature channels under rasterize_backward_algo = PER_GAUSSIAN: the colour pass runs the second
    algorithm, the feature passes add their share (render.py:1892-1895, 1952-1955); gradients against the oracle."""
    import torch
    from d3gs_research_amd.config_def import RasterizeBackwardAlgo
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    scene = gen_scene(1, n=20000, wh=(250, 190))
    rng = np.random.default_rng(3)
    F = 5
    feat = rng.standard_normal((scene.n, F)).astype(np.float32)
    P, ref = oracle_forward(oracle, scene, DFVT)
    feat_img = oracle.blend_custom_features(P, ref, feat)
    dfeat = rng.standard_normal(feat_img.shape).astype(np.float32)
    g_ref, pb_ref = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                                    scene.drgb[0], scene.dT[0], custom_features=feat, custom_feature_image=feat_img,
                                    dcustom_features=dfeat)
    model = torch_model(scene)
    op = GaussianSplatOp(op_config(scene, DFVT, rasterize_backward_algo=RasterizeBackwardAlgo.PER_GAUSSIAN))
    feat_t = torch.from_numpy(feat).cuda()
    out, ctx = op.forward(model, scene.camera(), training=True, custom_features=feat_t)
    assert ctx.per_gaussian_snap is not None
    assert np.array_equal(out.custom_features.cpu().numpy()[0].view(np.uint32), feat_img.view(np.uint32))
    grads = GaussianSplatGradients(drgb=torch.from_numpy(scene.drgb).cuda(), dT=torch.from_numpy(scene.dT).cuda(),
                                   dcustom_features=torch.from_numpy(dfeat[None]).cuda())
    gm, duv, dcf = op.backward(model, scene.camera(), ctx, out, grads, return_uv_grad=True)
    torch.cuda.synchronize()
    cpu = lambda t: t.detach().cpu().numpy()
    a, b = cpu(dcf).astype(np.float64), g_ref["dcustom_features"]
    assert (np.abs(a - b) <= 1e-4 * g_ref["absmass_features"] + 1e-30).all()
    tol = 1e-4 * np.array(g_ref["absmass"][:, :6]) + 16 * 2.0 ** -24 * g_ref["statemass"] + 1e-30
    g = op.last_raster_grads
    for name, got, sl in (("duv", g.duv, slice(0, 2)), ("dconic", g.dconic, slice(2, 5)), ("dopacity", g.dopacity, slice(5, 6))):
        a, b = cpu(got).astype(np.float64).reshape(scene.n, -1), g_ref[name].reshape(scene.n, -1)
        assert (np.abs(a - b) <= tol[:, sl]).all(), name
    for name, got in (("dxyz", gm.xyz), ("dscale", gm.scale), ("dsh", gm.color_sh)):
        med, p99 = np.quantile(per_gaussian_rel_err(cpu(got), pb_ref[name]), [0.5, 0.99])
        assert med <= 1e-5 and p99 <= 2e-3, f"{name}: median {med:.2e} p99 {p99:.2e}"
