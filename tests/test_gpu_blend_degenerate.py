"""d3gs_blend_fwd / d3gs_blend_bwd are public entry points that take any conic_opacity array.  The staging cull of
the kernels (a bounding box and a per-patch minimum of the quadratic form) assumes an ellipse; for a conic that is
not positive definite -- a zero or negative diagonal, b^2 >= a c -- it must stand aside and let the exact per-pixel
sequence decide (render.py:1765-1792: power > 0 is skipped AFTER the transmittance test).  Hand-made conics through
the C ABI against the oracle, image bit for bit and gradients to the blend's bar.  What the entry points do ask for
is that the power -1/2 (a dx^2 + c dy^2) - b dx dy stays below 80 for every pixel of a listed tile (the exp of the
blend is evaluated without an overflow guard; any positive semi-definite conic satisfies it)."""
import ctypes as C

import numpy as np
import pytest

from helpers import gen_scene, grad_close, op_config, oracle_params, torch_model

pytestmark = pytest.mark.gpu


def _conics(rng, G):
    co = np.zeros((G, 4), np.float32)
    kinds = []
    for g in range(G):
        kind = g % 8
        a, c = rng.uniform(0.002, 0.2, 2)
        b = rng.uniform(-0.9, 0.9) * np.sqrt(a * c)
        if kind in (3, 4):
            a, c = rng.uniform(0.002, 0.012, 2)       # keeps power below 80 over the image (the entry points' bound)
            b = rng.uniform(-0.9, 0.9) * np.sqrt(a * c)
        if kind == 1:
            a = 0.0                                   # degenerate: a parabolic cylinder
        elif kind == 2:
            c = 0.0
        elif kind == 3:
            a, c = -a, -c                             # negative definite: power > 0 away from the centre
        elif kind == 4:
            b = 1.5 * np.sqrt(a * c) * np.sign(b or 1.0)   # indefinite: b^2 > a c
        elif kind == 5:
            b = np.sqrt(np.float32(a) * np.float32(c))     # b^2 == a c up to rounding: a strip
        elif kind == 6:
            a, b, c = 0.0, 0.0, 0.0                   # constant alpha = opacity everywhere
        elif kind == 7:
            a, c = 1e-6, 40.0                         # extremely elongated, still positive definite
            b = 0.0
        co[g] = [a, b, c, rng.uniform(0.05, 0.9)]
        kinds.append(kind)
    return co, kinds


@pytest.mark.parametrize("seed", [0, 1])
def test_blend_with_conics_that_are_not_ellipses(oracle, seed):
    import torch
    from d3gs_research_amd import _capi
    from d3gs_research_amd.render import GaussianSplatOp
    W, H, G = 48, 32, 96
    scene = gen_scene(0, n=G, wh=(W, H))
    rng = np.random.default_rng(seed)
    co, kinds = _conics(rng, G)
    uvs = np.stack([rng.uniform(-8, W + 8, G), rng.uniform(-8, H + 8, G)], 1).astype(np.float32)
    rgb = rng.uniform(0, 1, (G, 3)).astype(np.float32)
    depths = np.sort(rng.uniform(1, 5, G)).astype(np.float32)
    tiles = ((W + 15) // 16) * ((H + 15) // 16)
    idx = np.tile(np.arange(G, dtype=np.int32), tiles)                  # every tile lists every gaussian, in order
    ranges = np.stack([np.arange(tiles) * G, (np.arange(tiles) + 1) * G], 1).astype(np.int32)
    ys, xs = np.mgrid[0:H, 0:W]
    dx, dy = uvs[:, 0, None, None] - xs, uvs[:, 1, None, None] - ys
    form = lambda: -0.5 * (co[:, 0, None, None] * dx * dx + co[:, 2, None, None] * dy * dy) - co[:, 1, None, None] * dx * dy
    top = form().reshape(G, -1).max(1)
    co[:, :3] *= np.where(top > 60.0, 60.0 / np.maximum(top, 1.0), 1.0).astype(np.float32)[:, None]   # the entry points' bound
    power = form()
    assert power.max() < 80.0 and power.max() > 30.0         # positive powers occur, inside the stated bound
    P = oracle_params(oracle, scene, 1)
    color, T, nc, _ = oracle.blend_fwd(P, ranges, idx, uvs, co, rgb)
    drgb = rng.standard_normal((H, W, 3)).astype(np.float32)
    dT = rng.standard_normal((H, W)).astype(np.float32)
    g_ref = oracle.blend_bwd(P, ranges, idx, uvs, co, rgb, T, nc, color, drgb, dT)
    print(f"degenerate conics seed={seed}: T in [{T.min():.3g}, {T.max():.3g}], contributors up to {nc.max()}", flush=True)
    assert T.min() < 0.5 and nc.max() > 10            # the hand-made gaussians do blend

    op = GaussianSplatOp(op_config(scene, 1))
    Pg = op.make_params(torch_model(scene), scene.camera(), True)
    L, p = _capi.lib(), _capi.ptr
    dev = "cuda"
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    d_ranges, d_idx, d_uvs, d_co, d_rgb = t(ranges), t(idx), t(uvs), t(co), t(rgb)
    o_color = torch.empty((H, W, 3), dtype=torch.float32, device=dev)
    o_T = torch.empty((H, W), dtype=torch.float32, device=dev)
    o_nc = torch.empty((H, W), dtype=torch.int32, device=dev)
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _capi.check(L.d3gs_blend_fwd(C.byref(Pg), p(d_ranges), p(d_idx), p(d_uvs), p(d_co), p(d_rgb), None, None, p(o_color),
                                 p(o_T), p(o_nc), None, None, 0, s), "d3gs_blend_fwd")
    torch.cuda.synchronize()
    assert np.array_equal(o_nc.cpu().numpy(), nc)
    assert np.array_equal(o_T.cpu().numpy().view(np.uint32), T.view(np.uint32))
    assert np.array_equal(o_color.cpu().numpy().view(np.uint32), color.view(np.uint32))

    rec = torch.zeros((G, _capi.GRAD_RECORD_FLOATS), dtype=torch.float32, device=dev)
    d_drgb, d_dT = t(drgb), t(dT)
    _capi.check(L.d3gs_blend_bwd(C.byref(Pg), p(d_ranges), p(d_idx), p(d_uvs), p(d_co), p(d_rgb), None, None, p(o_T),
                                 p(o_nc), p(o_color), None, p(d_drgb), p(d_dT), None, p(rec), None, s), "d3gs_blend_bwd")
    torch.cuda.synchronize()
    r = rec.cpu().numpy().astype(np.float64)
    mass = g_ref["absmass"]
    for name, cols in (("duv", slice(0, 2)), ("dconic", slice(2, 5)), ("dopacity", slice(5, 6)), ("dcolor", slice(6, 9))):
        a, b = r[:, cols], g_ref[name].reshape(G, -1)
        excess = np.abs(a - b) - (1e-4 * mass[:, cols] + 1e-30)
        bad = np.argwhere(excess > 0)
        assert bad.size == 0, f"{name}: gaussians {sorted(set(bad[:, 0]))} (kinds {sorted({kinds[g] for g in bad[:, 0]})})"
        ok, worst, nbad = grad_close(a, b)
        assert ok, f"{name}: {nbad} outside tolerance (worst {worst:.2f}x)"
