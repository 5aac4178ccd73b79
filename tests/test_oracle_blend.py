"""Pins the oracle's blend forward (K6) against a float64 per-pixel restatement
and the compositing invariants."""
import numpy as np
import pytest

from f64_reference import blend_pixel_f64
from helpers import gen_scene, oracle_forward


@pytest.mark.parametrize("cfg_id,n,wh,filt", [(0, None, None, 1), (1, 30000, (256, 256), 0), (4, 3000, (480, 270), 3)])
def test_blend_forward_matches_float64(oracle, cfg_id, n, wh, filt):
    scene = gen_scene(cfg_id, n=n, wh=wh)
    ref = oracle_forward(oracle, scene, filt)[1]
    tiles_x = (scene.width + 15) // 16
    uvs = ref["uvs"].astype(np.float64)
    co = ref["conic_opacity"].astype(np.float64)
    rgb = ref["rgb_gaussian"].astype(np.float64)
    rng = np.random.default_rng(3)
    checked = mism = 0
    for _ in range(600):
        px, py = int(rng.integers(scene.width)), int(rng.integers(scene.height))
        t = (py // 16) * tiles_x + px // 16
        r0, r1 = ref["workload_ranges"][t]
        col, T, last, ws = blend_pixel_f64(px, py, ref["gaussian_idx_sorted"][r0:r1], uvs, co, rgb)
        checked += 1
        # float32 rounding can flip a threshold decision (alpha vs 1/255, T vs 1e-4) for a rare pixel
        if last != ref["n_contrib"][py, px]:
            mism += 1
            continue
        assert np.abs(col - ref["color"][py, px]).max() <= 2e-5
        assert abs(T - ref["T"][py, px]) <= 1e-5
        assert abs(sum(ws) + T - 1.0) <= 1e-9           # partition of unity in exact arithmetic
    assert mism <= checked * 0.01


def test_compositing_invariants(oracle):
    scene = gen_scene(1, n=50000, wh=(320, 320))
    ref = oracle_forward(oracle, scene, 1)[1]
    T, color = ref["T"], ref["color"]
    assert T.min() >= 0 and T.max() <= 1
    assert color.min() >= 0
    # colour is a convex combination of gaussian colours scaled by (1 - T)
    assert (color.max(axis=2) <= (1 - T) * ref["rgb_gaussian"].max() + 1e-5).all()
    # n_contrib is the list index of the last contributor (render.py:1836): inside the tile's list
    tiles_x = (scene.width + 15) // 16
    lens = (ref["workload_ranges"][:, 1] - ref["workload_ranges"][:, 0]).reshape(-1, tiles_x)
    per_pixel_len = np.kron(lens, np.ones((16, 16), int))[:scene.height, :scene.width]
    assert (ref["n_contrib"] <= np.maximum(per_pixel_len - 1, 0)).all()
    # pixels with an empty list are untouched
    empty = per_pixel_len == 0
    assert (T[empty] == 1).all() and (color[empty] == 0).all()


def test_inference_background_and_clamp(oracle):
    """render.py:2258-2263: inference output is clamp(rgb + T * bg, 0, 1)."""
    scene = gen_scene(0)
    bg = (0.3, 0.6, 0.9)
    tr = oracle_forward(oracle, scene, 1, training=True)[1]
    inf = oracle_forward(oracle, scene, 1, training=False, bg=bg)[1]
    want = np.clip(tr["color"].astype(np.float64) + tr["T"][..., None] * np.array(bg, np.float32).astype(np.float64), 0, 1)
    assert np.abs(inf["color"] - want).max() <= 1e-6
    assert np.array_equal(inf["T"], tr["T"])


def test_extra_channels_layouts_and_inference_depth(oracle):
    """render_rgba: alpha = sum of weights = 1 - T in exact arithmetic and no background in inference
    (render.py:1899-1906, 2227-2229); use_nchw is the same image transposed (render.py:702, 2272-2294);
    render_depth in inference is normalised by the opacity (render.py:2244-2250)."""
    from helpers import oracle_params
    scene = gen_scene(1, n=30000, wh=(200, 136))
    args = (scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    base = oracle.forward(oracle_params(oracle, scene, 1), *args)

    P = oracle_params(oracle, scene, 1)
    P.render_rgba, P.render_depth = 1, 1
    full = oracle.forward(P, *args)
    assert np.array_equal(full["color"][..., :3], base["color"]) and np.array_equal(full["T"], base["T"])
    assert np.abs(full["color"][..., 3] + full["T"] - 1.0).max() <= 2e-6
    # depth is a convex-ish combination of the member depths: bounded by alpha * max depth
    assert (full["depth"] >= 0).all()
    assert (full["depth"] <= full["color"][..., 3] * full["depths"].max() * (1 + 1e-5) + 1e-6).all()

    P.use_nchw = 1
    nchw = oracle.forward(P, *args)
    assert nchw["color"].shape == (4, scene.height, scene.width)
    assert np.array_equal(nchw["color"].transpose(1, 2, 0), full["color"])
    assert np.array_equal(nchw["depth"], full["depth"])

    bg = (0.3, 0.6, 0.1)
    Pi = oracle_params(oracle, scene, 1, training=False, bg=bg)
    Pi.render_rgba, Pi.render_depth = 1, 1
    inf = oracle.forward(Pi, *args)
    assert np.array_equal(inf["T"], full["T"])
    want_rgb = np.clip(full["color"][..., :3] + full["T"][..., None] * np.array(bg, np.float32), 0, 1)
    assert np.abs(inf["color"][..., :3] - want_rgb).max() <= 1e-6
    assert np.abs(inf["color"][..., 3] - np.clip(full["color"][..., 3], 0, 1)).max() == 0
    want_depth = full["depth"] / (np.float32(1.0) - full["T"])
    seen = full["T"] < 1
    assert np.allclose(inf["depth"][seen], want_depth[seen], rtol=1e-6, atol=0)
    assert (inf["depth"][~seen] == 0).all() or np.isnan(inf["depth"][~seen]).all()


def test_statemass_bounds_the_effect_of_rounding_the_colour_state(oracle):
    """`statemass` (the bar of the per-gaussian backward's test) is the sensitivity of duv / dconic / dopacity to
    the pixels' running colour state: moving the final colour the backward starts from by one float32 ulp-scale
    step per pixel and channel (which only shifts that state, every alpha and T stays the same) must move each
    value by no more than 2^-24 * statemass, and does move some by a good part of it."""
    O = oracle
    scene = gen_scene(1, n=20000, wh=(250, 190))
    P, ref = oracle_forward(O, scene, 1)
    args = (P, ref["workload_ranges"], ref["gaussian_idx_sorted"], ref["uvs"], ref["conic_opacity"], ref["rgb_gaussian"],
            ref["T"], ref["n_contrib"])
    g0 = O.blend_bwd(*args, ref["color"], scene.drgb[0], scene.dT[0])
    rng = np.random.default_rng(5)
    step = (2.0 ** -24) * np.abs(ref["color"].astype(np.float64)) * rng.choice([-1.0, 1.0], size=ref["color"].shape)
    moved = (ref["color"].astype(np.float64) + step).astype(np.float32)
    moved_by = np.abs(moved.astype(np.float64) - ref["color"])          # what float32 made of the step
    assert moved_by.max() <= 2.0 ** -23 * np.abs(ref["color"]).max()
    g1 = O.blend_bwd(*args, moved, scene.drgb[0], scene.dT[0])
    assert np.array_equal(g0["dcolor"], g1["dcolor"])                   # w * drgb does not see the colour state
    got = np.concatenate([g1[k].reshape(scene.n, -1) - g0[k].reshape(scene.n, -1) for k in ("duv", "dconic", "dopacity")], 1)
    # float32 rounds the step to 0, 1 or 2 ulp of the colour: bound with 2^-22 instead of 2^-24, plus the float32
    # rounding of the terms themselves
    bound = 2.0 ** -22 * g0["statemass"] + 1e-5 * g0["absmass"][:, :6] + 1e-30
    assert (np.abs(got) <= bound).all()
    live = g0["statemass"] > 0
    assert live.any() and np.quantile((np.abs(got) / (2.0 ** -24 * g0["statemass"] + 1e-300))[live], 0.9) > 0.05
