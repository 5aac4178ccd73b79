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


def per_gaussian_rel_err(a, b):
    """Relative L2 error of each gaussian's gradient vector (rows of a against rows of b), over the gaussians
    whose reference gradient is not zero; the denominator has a floor of 1e-6 of the largest norm."""
    n = b.shape[0]
    a = np.asarray(a, np.float64).reshape(n, -1)
    b = np.asarray(b, np.float64).reshape(n, -1)
    rn = np.linalg.norm(b, axis=1)
    return (np.linalg.norm(a - b, axis=1) / (rn + 1e-6 * rn.max()))[rn > 0]


def rel_err_summary(e):
    """(median, 99th percentile, maximum, share of gaussians beyond 1e-4) of per-gaussian relative errors."""
    if e.size == 0:
        return 0.0, 0.0, 0.0, 0.0
    med, p99 = np.quantile(e, [0.5, 0.99])
    return float(med), float(p99), float(e.max()), float((e > 1e-4).mean())


def k9_noise_spread(O, P, scene, ref, g_ref, pb_ref, ulps=2.0, seed=11, state_ulps=0.0, tail=False):
    """What rounding noise in the blend backward's sums does to the preprocess backward, measured on the
    oracle.  A float32 sum of the per-pixel terms, in whatever order, carries an error of the order of
    2^-24 * sum|terms| ("absmass", which the oracle returns next to its float64 sums).  The oracle's own
    preprocess backward is run again on the screen-space gradients perturbed by N(0, 1) * ulps * 2^-24 * absmass;
    returned: {gradient name: (median, 99th percentile)} of the per-gaussian relative error it induces.  The
    spread beyond the input noise is the conditioning of the chain rule itself (near-degenerate projected
    covariances: gradients that are small differences of large terms).  With tail=True each entry is
    (median, 99th percentile, maximum, share of gaussians beyond 1e-4) instead."""
    rng = np.random.default_rng(seed)
    # state_ulps: on top of that, noise of state_ulps * 2^-24 * statemass in duv / dconic / dopacity, for a
    # backward whose per-pixel colour state is rounded differently from the oracle's (the per-gaussian algorithm)
    m = (ulps * 2.0 ** -24) * g_ref["absmass"][:, :9].copy()
    m[:, :6] += (state_ulps * 2.0 ** -24) * g_ref["statemass"]
    noisy = {"duv": g_ref["duv"] + rng.standard_normal(g_ref["duv"].shape) * m[:, 0:2],
             "dconic": g_ref["dconic"] + rng.standard_normal(g_ref["dconic"].shape) * m[:, 2:5],
             "dopacity": g_ref["dopacity"] + rng.standard_normal(g_ref["dopacity"].shape) * m[:, 5],
             "dcolor": g_ref["dcolor"] + rng.standard_normal(g_ref["dcolor"].shape) * m[:, 6:9]}
    dz = None
    if g_ref.get("dz") is not None:      # a depth channel: its gradient takes part, with its own summation noise
        dz = (g_ref["dz"] + rng.standard_normal(g_ref["dz"].shape) * (ulps * 2.0 ** -24) * g_ref["absmass"][:, 9]).astype(np.float32)
    pert = O.preprocess_bwd(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                            ref["radii"], ref["cov2d_vecs"], ref["sh_to_rgb_ne_0"],
                            *(noisy[k].astype(np.float32) for k in ("duv", "dconic", "dopacity", "dcolor")), dz=dz)
    names = ("dxyz", "dquat", "dscale", "dopacity", "dsh")
    if tail:
        return {k: rel_err_summary(per_gaussian_rel_err(pert[k], pb_ref[k])) for k in names}
    return {k: tuple(np.quantile(per_gaussian_rel_err(pert[k], pb_ref[k]), [0.5, 0.99])) for k in names}
