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
