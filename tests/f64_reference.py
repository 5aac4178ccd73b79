"""Independent float64 restatements used to pin the oracle: closed forms written
with numpy / scipy matrix algebra (not the oracle's scalar operation order)."""
from __future__ import annotations

import numpy as np
from scipy.spatial.transform import Rotation

# real SH constants as tabulated in the reference's in-tree Inria utility
# (d3sim/algos/d3gs/origin/data/utils/sh_utils.py:26-53)
C0 = 0.28209479177387814
C1 = 0.4886025119029199
C2 = [1.0925484305920792, -1.0925484305920792, 0.31539156525252005, -1.0925484305920792, 0.5462742152960396]
C3 = [-0.5900435899266435, 2.890611442640554, -0.4570457994644658, 0.3731763325901154, -0.4570457994644658,
      1.445305721320277, -0.5900435899266435]


def eval_sh(deg, sh, dirs):
    """sh [N,K,3], dirs [N,3] unit -> rgb [N,3] (before the +0.5 offset); follows the published
    3DGS eval_sh formula (sh_utils.py:55-116)."""
    x, y, z = dirs[:, 0:1], dirs[:, 1:2], dirs[:, 2:3]
    r = C0 * sh[:, 0]
    if deg > 0:
        r = r - C1 * y * sh[:, 1] + C1 * z * sh[:, 2] - C1 * x * sh[:, 3]
    if deg > 1:
        xx, yy, zz, xy, yz, xz = x * x, y * y, z * z, x * y, y * z, x * z
        r = (r + C2[0] * xy * sh[:, 4] + C2[1] * yz * sh[:, 5] + C2[2] * (2 * zz - xx - yy) * sh[:, 6]
             + C2[3] * xz * sh[:, 7] + C2[4] * (xx - yy) * sh[:, 8])
    if deg > 2:
        r = (r + C3[0] * y * (3 * xx - yy) * sh[:, 9] + C3[1] * xy * z * sh[:, 10]
             + C3[2] * y * (4 * zz - xx - yy) * sh[:, 11] + C3[3] * z * (2 * zz - 3 * xx - 3 * yy) * sh[:, 12]
             + C3[4] * x * (4 * zz - xx - yy) * sh[:, 13] + C3[5] * z * (xx - yy) * sh[:, 14]
             + C3[6] * x * (xx - 3 * yy) * sh[:, 15])
    return r


def preprocess_f64(scene, lowpass=0.3, eps=1e-6, clamp_factor=1.3, eigen_eps=0.1, sigma=3.0):
    """Projection, EWA covariance, conic, radius, colour in float64 matrix form."""
    X = scene.xyz.astype(np.float64)
    to_world = scene.to_world.astype(np.float64)
    Rc2w, c = to_world[:3, :3], to_world[:3, 3]
    W = Rc2w.T                                    # world -> camera
    pc = (X - c) @ W.T
    z = pc[:, 2]
    fx, fy, cx, cy = scene.fx, scene.fy, scene.cx, scene.cy
    uv = np.stack([fx * pc[:, 0] / z + cx - 0.5, fy * pc[:, 1] / z + cy - 0.5], 1)
    q = scene.quaternion_xyzw.astype(np.float64)
    q = q / np.linalg.norm(q, axis=1, keepdims=True)
    R = Rotation.from_quat(q).as_matrix()         # scipy: scalar-last (x, y, z, w)
    S = np.exp(scene.scale.astype(np.float64))
    M = R * S[:, None, :]
    Sigma3 = M @ M.transpose(0, 2, 1)
    tanx, tany = 0.5 * scene.width / fx, 0.5 * scene.height / fy
    lx, ly = np.abs(tanx * clamp_factor * z), np.abs(tany * clamp_factor * z)
    tx, ty = np.clip(pc[:, 0], -lx, lx), np.clip(pc[:, 1], -ly, ly)
    J = np.zeros((len(X), 2, 3))
    J[:, 0, 0] = fx / z
    J[:, 0, 2] = -fx * tx / z ** 2
    J[:, 1, 1] = fy / z
    J[:, 1, 2] = -fy * ty / z ** 2
    T = J @ W
    Sigma2 = T @ Sigma3 @ T.transpose(0, 2, 1)
    a, b, cc = Sigma2[:, 0, 0] + lowpass, Sigma2[:, 0, 1], Sigma2[:, 1, 1] + lowpass
    det = a * cc - b * b
    conic = np.stack([cc, -b, a], 1) / (det + eps)[:, None]
    opacity = 1.0 / (1.0 + np.exp(-scene.opacity.astype(np.float64)))
    mid = 0.5 * (a + cc)
    lam = mid + np.sqrt(np.maximum(eigen_eps, mid * mid - det))
    radius_f = sigma * np.sqrt(lam)
    d = X - c
    dirs = d / np.linalg.norm(d, axis=1, keepdims=True)
    rgb = eval_sh(scene.sh_degree, scene.color_sh.astype(np.float64), dirs) + 0.5
    return dict(pc=pc, z=z, uv=uv, cov2d=np.stack([a, b, cc], 1), det=det, conic=conic, opacity=opacity,
                radius_f=radius_f, rgb=rgb, Sigma3=Sigma3)


def blend_pixel_f64(px, py, idx, uvs, conic_opacity, rgb, alpha_eps=1 / 255.0, t_eps=1e-4):
    """Front-to-back compositing of one pixel over the gaussian ids `idx`; float64.
    Returns colour, final T, index of the last contributor and the weights."""
    T, col, last = 1.0, np.zeros(3), 0
    ws = []
    for k, g in enumerate(idx):
        dx, dy = uvs[g, 0] - px, uvs[g, 1] - py
        a, b, c, o = conic_opacity[g]
        power = -0.5 * (a * dx * dx + c * dy * dy) - b * dx * dy
        alpha = min(0.99, o * np.exp(power))
        if alpha < alpha_eps:
            continue
        nT = T * (1 - alpha)
        if nT < t_eps:
            break
        if power > 0:
            continue
        col += alpha * T * rgb[g]
        ws.append(alpha * T)
        T, last = nT, k
    return col, T, last, ws
