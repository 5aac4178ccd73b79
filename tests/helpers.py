"""Shared helpers for the parity tests: scene -> oracle params / torch model."""
from __future__ import annotations

import numpy as np

from d3gs_research_amd.config_def import GaussianSplatConfig
from d3gs_research_amd.synthetic import Scene, gen_scene, scene_config, scene_model  # noqa: F401


def oracle_params(O, scene: Scene, filter_algo: int, training: bool = True, **over):
    return O.params_for_scene(scene, filter_algo, training, **over)


def op_config(scene: Scene, filter_algo: int, **over) -> GaussianSplatConfig:
    return scene_config(scene, filter_algo, **over)


def torch_model(scene: Scene, device="cuda"):
    return scene_model(scene, device)


def oracle_forward(O, scene: Scene, filter_algo: int, training=True, **over):
    P = oracle_params(O, scene, filter_algo, training, **over)
    return P, O.forward(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)


def grad_close(a, b, rel=1e-4, abs_frac=1e-5):
    """|a-b| <= rel*|b| + abs_frac*max|b| elementwise; returns (ok, worst excess ratio)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    scale = np.abs(b).max() if b.size else 0.0
    tol = rel * np.abs(b) + abs_frac * scale
    err = np.abs(a - b)
    bad = err > tol
    worst = float((err / np.maximum(tol, 1e-300)).max()) if b.size else 0.0
    return (not bad.any()), worst, int(bad.sum())
