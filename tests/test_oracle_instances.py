"""Pins the oracle's instance rendering (render.py:207-220, 346-356, 3031-3040): gaussians that carry an
instance id are given in their object's frame and seen by the camera expressed in that frame.

What fixes the result without retyping the formula:
  * identity poses, or negative ids, change nothing (bit for bit);
  * with every gaussian in one instance the render is the plain render by the composed camera (bit for bit):
    the per-gaussian substitution is a camera replacement and nothing else;
  * at SH degree 0 (colour independent of the viewing direction) rendering the instance-frame gaussians under
    their poses equals rendering the same gaussians moved into the world frame (xyz -> R xyz + t, the
    orientation composed with R), and the position gradient comes back rotated by R^T.  A transposed
    rotation, a wrong sign of the translation or a swapped composition order fails this one."""
import numpy as np

from helpers import gen_scene, oracle_params

AABB, DFVT = 1, 4


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint32)


def _quat_to_R(q):
    x, y, z, w = (float(v) for v in q)
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)],
                     [2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)],
                     [2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)]], np.float64)


def _quat_mul(a, b):
    """Hamilton product a (x) b of xyzw quaternions, rows of b."""
    ax, ay, az, aw = a
    bx, by, bz, bw = b[:, 0], b[:, 1], b[:, 2], b[:, 3]
    return np.stack([aw * bx + ax * bw + ay * bz - az * by,
                     aw * by - ax * bz + ay * bw + az * bx,
                     aw * bz + ax * by - ay * bx + az * bw,
                     aw * bw - ax * bx - ay * by - az * bz], 1)


def _poses(rng, count, angle=0.3, shift=0.25):
    """Random rigid poses: unit quaternions near identity, small translations.  Returns (quats, R, t, T[count,4,3])."""
    q = np.concatenate([rng.standard_normal((count, 3)) * angle, np.ones((count, 1))], 1)
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    R = np.stack([_quat_to_R(v) for v in q])
    t = rng.standard_normal((count, 3)) * shift
    T = np.concatenate([R.transpose(0, 2, 1), t[:, None, :]], 1)     # rows: columns of R, then t
    return q, R, t, T.astype(np.float32)


def _args(scene):
    return scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh


def _run(O, P, scene, instances, xyz=None, quat=None):
    a = list(_args(scene))
    if xyz is not None:
        a[0] = xyz
    if quat is not None:
        a[1] = quat
    fwd = O.forward(P, *a, instances=instances)
    g, pb = O.backward(P, fwd, *a, scene.drgb[0], scene.dT[0], instances=instances)
    return fwd, pb


def test_identity_poses_and_negative_ids_change_nothing(oracle):
    scene = gen_scene(1, n=6000, wh=(160, 120))
    P = oracle_params(oracle, scene, DFVT)
    rng = np.random.default_rng(5)
    plain_f, plain_b = _run(oracle, P, scene, None)
    eye = np.tile(np.concatenate([np.eye(3), np.zeros((1, 3))], 0)[None], (3, 1, 1)).astype(np.float32)
    cams = oracle.instance_cameras(scene.cam2world_T, eye)
    assert np.array_equal(_bits(cams[1]), _bits(scene.cam2world_T.reshape(-1)))
    ids = rng.integers(-1, 3, scene.n).astype(np.int32)
    _, _, _, T = _poses(rng, 3)
    for label, inst in (("identity", (ids, cams)),
                        ("negative ids", (np.full(scene.n, -1, np.int32), oracle.instance_cameras(scene.cam2world_T, T)))):
        f, b = _run(oracle, P, scene, inst)
        for k in ("color", "T", "radii", "uvs", "conic_opacity", "gaussian_idx_sorted", "workload_ranges"):
            assert np.array_equal(f[k], plain_f[k]), (label, k)
        for k in ("dxyz", "dquat", "dscale", "dopacity", "dsh"):
            assert np.array_equal(_bits(b[k]), _bits(plain_b[k])), (label, k)


def test_one_instance_is_the_composed_camera(oracle):
    scene = gen_scene(1, n=6000, wh=(160, 120))
    rng = np.random.default_rng(6)
    _, _, _, T = _poses(rng, 2)
    cams = oracle.instance_cameras(scene.cam2world_T, T)
    ids = np.ones(scene.n, np.int32)
    P = oracle_params(oracle, scene, DFVT)
    f, b = _run(oracle, P, scene, (ids, cams))
    Q = oracle_params(oracle, scene, DFVT, cam2world_T=cams[1].reshape(4, 3))
    f2, b2 = _run(oracle, Q, scene, None)
    assert f["num_rendered"] == f2["num_rendered"] > 0
    for k in ("color", "T", "radii", "uvs", "conic_opacity", "rgb_gaussian", "gaussian_idx_sorted", "workload_ranges"):
        assert np.array_equal(f[k], f2[k]), k
    for k in ("dxyz", "dquat", "dscale", "dopacity", "dsh"):
        assert np.array_equal(_bits(b[k]), _bits(b2[k])), k
    # and it is not the plain render
    f0, _ = _run(oracle, P, scene, None)
    assert not np.array_equal(f["uvs"], f0["uvs"])


def test_instance_render_equals_render_of_world_space_gaussians(oracle):
    scene = gen_scene(0)          # SH degree 0
    assert scene.sh_degree == 0
    rng = np.random.default_rng(7)
    K = 3
    q, R, t, T = _poses(rng, K)
    ids = rng.integers(-1, K, scene.n).astype(np.int32)
    P = oracle_params(oracle, scene, AABB)
    cams = oracle.instance_cameras(scene.cam2world_T, T)
    f_i, b_i = _run(oracle, P, scene, (ids, cams))

    # the same gaussians moved into the world frame (float64, rounded once)
    xyz_w = scene.xyz.astype(np.float64).copy()
    quat_w = scene.quaternion_xyzw.astype(np.float64).copy()
    for k in range(K):
        m = ids == k
        xyz_w[m] = xyz_w[m] @ R[k].T + t[k]
        quat_w[m] = _quat_mul(q[k], quat_w[m])
    f_w, b_w = _run(oracle, P, scene, None, xyz=xyz_w.astype(np.float32), quat=quat_w.astype(np.float32))

    moved = ids >= 0
    assert moved.sum() > scene.n // 2 and np.abs(f_i["uvs"] - oracle.forward(P, *_args(scene))["uvs"])[moved].max() > 1.0
    vis = (f_i["radii"] > 0) & (f_w["radii"] > 0)
    assert (f_i["radii"] > 0).sum() > 100 and ((f_i["radii"] > 0) != (f_w["radii"] > 0)).sum() <= 2
    assert np.abs(f_i["uvs"] - f_w["uvs"])[vis].max() < 2e-3
    assert np.abs(f_i["depths"] - f_w["depths"])[vis].max() < 1e-5 * np.abs(f_w["depths"]).max() + 1e-5
    rel = np.abs(f_i["conic_opacity"] - f_w["conic_opacity"])[vis] / (np.abs(f_w["conic_opacity"])[vis] + 1e-3)
    assert rel.max() < 2e-3
    err = np.abs(f_i["color"].astype(np.float64) - f_w["color"])
    assert np.quantile(err, 0.999) < 2e-4 and err.max() < 5e-2, (np.quantile(err, 0.999), err.max())

    # position gradient: d/dxyz_instance = R^T d/dxyz_world; scale, opacity and colour gradients carry over
    dx_w = b_w["dxyz"].astype(np.float64)
    expect = dx_w.copy()
    for k in range(K):
        m = ids == k
        expect[m] = dx_w[m] @ R[k]
    for got, ref, name in ((b_i["dxyz"], expect, "dxyz"), (b_i["dscale"], b_w["dscale"], "dscale"),
                           (b_i["dopacity"], b_w["dopacity"], "dopacity"), (b_i["dsh"], b_w["dsh"], "dsh")):
        e = np.abs(got.astype(np.float64) - ref).reshape(scene.n, -1).max(1)
        scale_ = np.abs(ref).max()
        assert np.quantile(e, 0.995) < 2e-3 * scale_, (name, np.quantile(e, 0.995) / scale_)
