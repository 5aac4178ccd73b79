"""Pins the oracle's preprocess forward (K1) against float64 closed forms built
with scipy rotations and numpy matrix products, including a rotated, translated
camera so that a transposed matrix or a swapped quaternion order fails."""
import numpy as np
import pytest
from scipy.spatial.transform import Rotation

from f64_reference import preprocess_f64
from helpers import gen_scene, oracle_params


def _posed_scene(cfg_id, n, wh=None):
    s = gen_scene(cfg_id, n=n, wh=wh)
    Rc = Rotation.from_euler("xyz", [0.2, -0.35, 0.5]).as_matrix()
    tw = np.eye(4)
    tw[:3, :3] = Rc
    tw[:3, 3] = [0.3, -0.2, s.to_world[2, 3] - 0.5]
    s.to_world = tw
    return s


@pytest.mark.parametrize("make", [lambda: gen_scene(0), lambda: gen_scene(1, n=20000), lambda: _posed_scene(1, 20000),
                                  lambda: _posed_scene(2, 30000, (640, 360)), lambda: gen_scene(4, n=20000, wh=(960, 540))])
def test_preprocess_matches_float64_closed_forms(oracle, make):
    scene = make()
    P = oracle_params(oracle, scene, 0)
    got = oracle.preprocess_fwd(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    ref = preprocess_f64(scene)
    valid = got["radii"] > 0
    assert valid.sum() > 0.3 * scene.n
    # everything the oracle rejected must be rejected by the float64 rules too (allowing threshold ties)
    in_depth = (ref["z"] >= scene.near) & (ref["z"] <= scene.far)
    assert not (valid & ~in_depth).any()
    v = valid
    rel = lambda a, b: np.abs(a - b) / (np.abs(b) + 1e-12)
    assert np.abs(got["depths"][v] - ref["z"][v]).max() <= 2e-6 * np.abs(ref["z"][v]).max()
    assert np.abs(got["uvs"][v] - ref["uv"][v]).max() <= 2e-3            # pixels; |uv| up to ~1e4
    assert np.median(np.abs(got["uvs"][v] - ref["uv"][v])) <= 5e-5
    # matrix entries relative to the matrix scale (the off-diagonal may be ~0)
    mrel = lambda a, b: np.abs(a - b) / np.abs(b).max(axis=1, keepdims=True)
    assert mrel(got["cov2d_vecs"][v], ref["cov2d"][v]).max() <= 1e-4
    assert np.median(mrel(got["cov2d_vecs"][v], ref["cov2d"][v])) <= 2e-7
    assert mrel(got["conic_opacity"][v, :3], ref["conic"][v]).max() <= 1e-3
    assert np.median(mrel(got["conic_opacity"][v, :3], ref["conic"][v])) <= 1e-6
    assert rel(got["conic_opacity"][v, 3], ref["opacity"][v]).max() <= 1e-6
    # radius = ceil(3 sqrt(lambda_max)): equal except where float32 rounding crosses an integer
    rf = np.ceil(ref["radius_f"][v])
    diff = got["radii"][v] - rf
    assert np.abs(diff).max() <= 1 and (diff != 0).mean() < 2e-3
    # colour: clamp at zero and the clamp mask, r -> bit 2, g -> bit 1, b -> bit 0 (render.py:608)
    want_rgb = np.maximum(ref["rgb"][v], 0)
    assert np.abs(got["rgb_gaussian"][v] - want_rgb).max() <= 2e-6
    neg = ref["rgb"][v] < 0
    mask = (neg[:, 0] << 2) | (neg[:, 1] << 1) | neg[:, 2]
    near_zero = (np.abs(ref["rgb"][v]) < 1e-6).any(1)
    assert np.array_equal(got["sh_to_rgb_ne_0"][v][~near_zero], mask[~near_zero])
    # rejected gaussians are zero-filled
    for k in ("depths", "uvs", "conic_opacity", "rgb_gaussian", "cov2d_vecs", "tiles_touched"):
        assert not got[k][~v].any()


def test_validity_rules(oracle):
    """render.py:475: det <= 0, z outside [near, far], empty rect or opacity <= 1/255 reject a gaussian."""
    scene = gen_scene(0, n=8)
    scene.xyz[:] = [0.0, 0.0, 4.0]
    scene.scale[:] = -3.0
    scene.opacity[:] = 1.0
    scene.xyz[1, 2] = 0.005          # nearer than near (0.01)
    scene.xyz[2, 2] = 150.0          # beyond far (100)
    scene.xyz[3, 2] = -4.0           # behind the camera
    scene.xyz[4, 0] = 40.0           # far off screen: empty tile rect
    scene.opacity[5] = -5.6          # sigmoid = 0.00368 <= 1/255
    scene.opacity[6] = -5.5          # sigmoid = 0.00407 >  1/255
    P = oracle_params(oracle, scene, 0)
    got = oracle.preprocess_fwd(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    assert (got["radii"] > 0).tolist() == [True, False, False, False, False, False, True, True]
    assert (got["tiles_touched"] > 0).tolist() == (got["radii"] > 0).tolist()


def test_on_axis_identity_closed_form(oracle):
    """Camera at the origin looking +z, identity rotation, point on the optical axis:
    cov2d = diag((fx s_x / z)^2, (fy s_y / z)^2) + 0.3 I and uv = principal point - 0.5."""
    scene = gen_scene(0, n=1)
    scene.xyz[0] = [0.0, 0.0, 4.0]
    scene.quaternion_xyzw[0] = [0.0, 0.0, 0.0, 2.0]     # unnormalised on purpose: the kernel normalises
    scene.scale[0] = np.log([0.05, 0.1, 0.2])
    scene.opacity[0] = 0.0
    P = oracle_params(oracle, scene, 0)
    got = oracle.preprocess_fwd(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    a = (128 * 0.05 / 4) ** 2 + 0.3
    c = (128 * 0.1 / 4) ** 2 + 0.3
    np.testing.assert_allclose(got["cov2d_vecs"][0], [a, 0.0, c], rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(got["uvs"][0], [63.5, 63.5], atol=1e-5)
    np.testing.assert_allclose(got["conic_opacity"][0], [1 / a, 0.0, 1 / c, 0.5], rtol=1e-5, atol=1e-7)
    assert got["radii"][0] == int(np.ceil(3 * np.sqrt(c)))
    assert abs(got["depths"][0] - 4.0) < 1e-6
    # degree 0: rgb = C0 * dc + 0.5, clamped at 0
    want = np.maximum(0.28209479177387814 * scene.color_sh[0, 0].astype(np.float64) + 0.5, 0)
    np.testing.assert_allclose(got["rgb_gaussian"][0], want, atol=1e-6)


def test_notebook_eigen_radius_value(oracle):
    """The reference's geometry notebook (scripts/geometry.ipynb, cell 3) inverts
    [[0.029680, 0.011789], [0.011789, 0.119252]]; the 3-sigma radius formula must agree with numpy's eigenvalues."""
    m = np.array([[0.029680, 0.011789], [0.011789, 0.119252]])
    cov = np.linalg.inv(m)
    lam = np.linalg.eigvalsh(cov).max()
    a, b, c = cov[0, 0], cov[0, 1], cov[1, 1]
    mid = 0.5 * (a + c)
    assert abs(mid + np.sqrt(max(0.1, mid * mid - (a * c - b * b))) - lam) < 1e-9
    # and through the oracle: build a gaussian whose projected covariance is `cov` (minus the low-pass)
    scene = gen_scene(0, n=1)
    w, V = np.linalg.eigh(cov - 0.3 * np.eye(2))
    assert (w > 0).all()
    z, f = 4.0, 128.0
    R3 = np.eye(3)
    R3[:2, :2] = V
    if np.linalg.det(R3) < 0:
        R3[:, 0] *= -1
    scene.xyz[0] = [0, 0, z]
    scene.quaternion_xyzw[0] = Rotation.from_matrix(R3).as_quat()
    scene.scale[0] = np.log([np.sqrt(w[0]) * z / f, np.sqrt(w[1]) * z / f, 1e-3])
    P = oracle_params(oracle, scene, 0)
    got = oracle.preprocess_fwd(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    np.testing.assert_allclose(got["cov2d_vecs"][0], [a, b, c], rtol=1e-4)
    assert got["radii"][0] == int(np.ceil(3 * np.sqrt(lam)))


def test_invalid_mask_equals_rendering_the_kept_subset(oracle):
    """render.py:306-308: mask[i] true rejects gaussian i.  The masked render must be the render of
    the scene with those gaussians removed, and the rejected records must be the zero records."""
    scene = gen_scene(0)
    rng = np.random.default_rng(5)
    mask = rng.random(scene.n) < 0.3
    P = oracle_params(oracle, scene, 0)
    got = oracle.forward(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                         invalid_mask=mask)
    keep = np.flatnonzero(~mask)
    Pk = oracle_params(oracle, scene, 0)
    Pk.n = len(keep)
    want = oracle.forward(Pk, scene.xyz[keep], scene.quaternion_xyzw[keep], scene.scale[keep], scene.opacity[keep],
                          scene.color_sh[keep])
    assert (got["radii"][mask] == 0).all() and (got["tiles_touched"][mask] == 0).all()
    assert np.array_equal(got["radii"][keep], want["radii"])
    assert np.array_equal(got["color"], want["color"]) and np.array_equal(got["T"], want["T"])
    assert np.array_equal(got["n_contrib"], want["n_contrib"])
    assert np.array_equal(keep[want["gaussian_idx_sorted"]], got["gaussian_idx_sorted"])
