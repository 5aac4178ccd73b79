"""Seeded synthetic scenes for the five benchmark / parity configurations.

Each scene is drawn from one ``numpy.random.Generator(PCG64(1000 + config_id))``
in a fixed order (means, log-scales, quaternions, opacity logits, SH DC, SH
rest, dL/dimage) so that every consumer — parity tests, the CPU oracle, the
benchmark — sees identical inputs.
"""
from __future__ import annotations

import dataclasses

import numpy as np

from .camera import BasicPinholeCamera
from .config_def import EarlyFilterAlgo, GaussianSplatConfig


@dataclasses.dataclass
class Scene:
    config_id: int
    name: str
    xyz: np.ndarray          # [N,3]
    quaternion_xyzw: np.ndarray  # [N,4]
    scale: np.ndarray        # [N,3] log-scale
    opacity: np.ndarray      # [N] logit
    color_sh: np.ndarray     # [N,K,3]
    sh_degree: int
    width: int
    height: int
    fx: float
    fy: float
    cx: float
    cy: float
    to_world: np.ndarray     # 4x4 camera -> world
    near: float
    far: float
    drgb: np.ndarray         # [1,H,W,3]
    dT: np.ndarray           # [1,H,W]

    @property
    def n(self):
        return self.xyz.shape[0]

    def camera(self) -> BasicPinholeCamera:
        return BasicPinholeCamera.from_params(self.fx, self.fy, self.cx, self.cy, self.width, self.height, self.to_world)

    @property
    def cam2world_T(self) -> np.ndarray:
        """4x3 ``to_world[:3].T`` (rows 0-2: world->camera rotation, row 3: centre)."""
        return np.ascontiguousarray(self.to_world[:3].T.astype(np.float32))


_SPECS = {
    0: dict(name="tiny-4k-sh0-128", n=4096, wh=(128, 128), f=128.0, cam_z=0.0, sh_degree=0, near=0.01, far=100.0),
    1: dict(name="100k-sh3-512", n=100_000, wh=(512, 512), f=600.0, cam_z=-4.0, sh_degree=3, near=0.2, far=1e4),
    2: dict(name="1M-sh3-1080p", n=1_000_000, wh=(1920, 1080), f=1100.0, cam_z=-5.0, sh_degree=3, near=0.2, far=1e4),
    3: dict(name="3M-sh3-1080p-slab", n=3_000_000, wh=(1920, 1080), f=1100.0, cam_z=-5.0, sh_degree=3, near=0.2, far=1e4),
    4: dict(name="500k-sh3-4k-stress", n=500_000, wh=(3840, 2160), f=2200.0, cam_z=0.0, sh_degree=3, near=0.2, far=1e4),
}


def _normal(rng, shape, mean, std):
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(std) + np.float32(mean)).astype(np.float32)


def _uniform(rng, shape, lo, hi):
    return (rng.random(shape, dtype=np.float32) * np.float32(hi - lo) + np.float32(lo)).astype(np.float32)


def gen_scene(config_id: int, n: int | None = None, wh: tuple[int, int] | None = None, with_grad: bool = True) -> Scene:
    """Build configuration ``config_id`` (0..4).

    ``n`` / ``wh`` shrink the gaussian count / image size (focal length and
    principal point scale with the width) for fast parity cases that keep the
    configuration's distributions.
    """
    spec = _SPECS[config_id]
    rng = np.random.Generator(np.random.PCG64(1000 + config_id))
    N = int(n if n is not None else spec["n"])
    W0, H0 = spec["wh"]
    W, H = wh if wh is not None else (W0, H0)
    fscale = W / W0
    f = spec["f"] * fscale
    cx, cy = W / 2.0, H / 2.0

    # means
    if config_id == 0:
        xyz = np.stack([_uniform(rng, N, -1, 1), _uniform(rng, N, -1, 1), _uniform(rng, N, 2, 6)], 1)
    elif config_id == 1:
        xyz = _normal(rng, (N, 3), 0.0, 1.0)
    elif config_id == 2:
        centres = _uniform(rng, (8, 3), -2, 2)
        which = rng.integers(0, 8, size=N)
        xyz = centres[which] + _normal(rng, (N, 3), 0.0, 0.6)
    elif config_id == 3:
        xyz = np.stack([_uniform(rng, N, -10, 10), _uniform(rng, N, -10, 10), _uniform(rng, N, 1, 40) + np.float32(spec["cam_z"])], 1)
    else:
        xyz = np.stack([_uniform(rng, N, -3, 3), _uniform(rng, N, -3, 3), _uniform(rng, N, 3, 8)], 1)
    xyz = np.ascontiguousarray(xyz, np.float32)

    # log-scales
    if config_id == 0:
        scale = _normal(rng, (N, 3), -3.0, 0.5)
    elif config_id == 1:
        scale = _normal(rng, (N, 3), -4.0, 0.7)
    elif config_id in (2, 3):
        scale = _normal(rng, (N, 3), -4.5, 1.0)
    else:
        big = rng.random(N) < 0.05
        small_s = _normal(rng, (N, 3), -5.0, 0.5)
        big_s = _normal(rng, (N, 3), -1.5, 0.3)
        scale = np.where(big[:, None], big_s, small_s).astype(np.float32)

    # quaternions (x, y, z, w), normalised here; the kernels normalise again
    q = _normal(rng, (N, 4), 0.0, 1.0)
    q = (q / np.linalg.norm(q, axis=1, keepdims=True)).astype(np.float32)

    # opacity logits
    if config_id in (0, 1):
        opacity = _normal(rng, N, 0.0, 1.0)
    elif config_id in (2, 3):
        opacity = _normal(rng, N, 0.0, 1.5)
    else:
        opacity = _normal(rng, N, 2.0, 0.5)

    # SH
    deg = spec["sh_degree"]
    K = (deg + 1) ** 2
    sh = np.empty((N, K, 3), np.float32)
    sh[:, 0] = _normal(rng, (N, 3), 0.0, 0.5)
    if K > 1:
        sh[:, 1:] = _normal(rng, (N, K - 1, 3), 0.0, 0.05)

    if with_grad:
        drgb = _normal(rng, (1, H, W, 3), 0.0, 1.0)
    else:
        drgb = np.zeros((1, H, W, 3), np.float32)
    dT = np.zeros((1, H, W), np.float32)

    to_world = np.eye(4, dtype=np.float64)
    to_world[2, 3] = spec["cam_z"]
    return Scene(config_id=config_id, name=spec["name"], xyz=xyz, quaternion_xyzw=q, scale=scale, opacity=opacity,
                 color_sh=sh, sh_degree=deg, width=W, height=H, fx=float(f), fy=float(f), cx=float(cx), cy=float(cy),
                 to_world=to_world, near=spec["near"], far=spec["far"], drgb=drgb, dT=dT)


def scene_config(scene: Scene, filter_algo: int = int(EarlyFilterAlgo.OBB_DFVT), **over) -> GaussianSplatConfig:
    """Rasterizer configuration for a synthetic scene: reference defaults with the scene's near / far planes."""
    cfg = GaussianSplatConfig(near=scene.near, far=scene.far, early_filter_algo=EarlyFilterAlgo(int(filter_algo)))
    for k, v in over.items():
        setattr(cfg, k, v)
    return cfg


def scene_model(scene: Scene, device="cuda"):
    """The scene's gaussians as a fused-activation model on ``device``."""
    import torch
    from .model import GaussianModelOriginFused
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    return GaussianModelOriginFused(xyz=t(scene.xyz), quaternion_xyzw=t(scene.quaternion_xyzw), scale=t(scene.scale),
                                    opacity=t(scene.opacity), color_sh=t(scene.color_sh), color_sh_base=None,
                                    cur_sh_degree=scene.sh_degree, act_applied=True)
