"""Data formats and helpers either side of the rasterizer: the Inria 3DGS point-cloud file, the
learning-rate schedule and the optimizer parameter groups of the reference trainer.

* PLY layout (d3sim/algos/d3gs/tools.py:20-62 reads it; the writer it must match is
  origin/data/scene/gaussian_model.py:177-208): one ``vertex`` element of float32 properties
  ``x y z nx ny nz f_dc_0..2 f_rest_0..44 opacity scale_0..2 rot_0..3``.  ``f_rest`` is stored
  channel-major (3 x 15) and becomes coefficient-major ``[15, 3]``; ``rot`` is stored ``wxyz`` and
  becomes ``xyzw``; scale and opacity stay raw (log-scale, logit).
* No third-party PLY package is needed: the header is parsed here and the body is read with a
  numpy structured dtype.
"""
from __future__ import annotations

import math

import numpy as np
import torch

from .model import GaussianModelOrigin, GaussianModelOriginBase, GaussianModelOriginFused

SH_C0 = 0.28209479177387814

_PLY_TYPES = {
    "char": "i1", "int8": "i1", "uchar": "u1", "uint8": "u1", "short": "i2", "int16": "i2", "ushort": "u2",
    "uint16": "u2", "int": "i4", "int32": "i4", "uint": "u4", "uint32": "u4", "float": "f4", "float32": "f4",
    "double": "f8", "float64": "f8",
}


def rgb_to_sh(rgb):
    """tools.py:14-15."""
    return (rgb - 0.5) / SH_C0


def inverse_sigmoid(x):
    """tools.py:17-18."""
    return torch.log(x / (1 - x))


def read_ply_vertices(path: str) -> dict[str, np.ndarray]:
    """Properties of the ``vertex`` element of a PLY file (ascii or binary, scalar properties only)."""
    with open(path, "rb") as f:
        if f.readline().strip() != b"ply":
            raise ValueError(f"{path}: not a PLY file")
        fmt = None
        elements: list[tuple[str, int, list[tuple[str, str]]]] = []
        while True:
            line = f.readline()
            if not line:
                raise ValueError(f"{path}: header without end_header")
            tok = line.decode("ascii", "replace").split()
            if not tok or tok[0] in ("comment", "obj_info"):
                continue
            if tok[0] == "format":
                fmt = tok[1]
            elif tok[0] == "element":
                elements.append((tok[1], int(tok[2]), []))
            elif tok[0] == "property":
                if tok[1] == "list":
                    if elements[-1][0] == "vertex":
                        raise ValueError(f"{path}: list property in the vertex element")
                    elements[-1][2].append((tok[-1], "list"))
                else:
                    if tok[1] not in _PLY_TYPES:
                        raise ValueError(f"{path}: unknown property type {tok[1]}")
                    elements[-1][2].append((tok[2], _PLY_TYPES[tok[1]]))
            elif tok[0] == "end_header":
                break
        if fmt not in ("ascii", "binary_little_endian", "binary_big_endian"):
            raise ValueError(f"{path}: unsupported PLY format {fmt}")
        if not elements or elements[0][0] != "vertex":
            raise ValueError(f"{path}: the first element must be 'vertex'")
        _, count, props = elements[0]
        if fmt == "ascii":
            data = np.loadtxt(f, dtype=np.float64, max_rows=count, ndmin=2)
            if data.shape != (count, len(props)):
                raise ValueError(f"{path}: vertex table has shape {data.shape}, expected {(count, len(props))}")
            return {name: data[:, k].astype(np.dtype(t)) for k, (name, t) in enumerate(props)}
        order = "<" if fmt == "binary_little_endian" else ">"
        dtype = np.dtype([(name, order + t) for name, t in props])
        body = np.fromfile(f, dtype=dtype, count=count)
        if body.shape[0] != count:
            raise ValueError(f"{path}: truncated vertex data ({body.shape[0]} of {count})")
        return {name: np.ascontiguousarray(body[name]) for name, _ in props}


def load_3dgs_origin_model(ply_path: str, fused: bool = True, split: bool = True, device="cuda") -> GaussianModelOriginBase:
    """tools.py:20-62: an Inria-format point cloud as a (fused or torch-activated) model, SH degree 3."""
    v = read_ply_vertices(ply_path)
    n = v["x"].shape[0]
    positions = np.stack([v["x"], v["y"], v["z"]], axis=1).astype(np.float32)
    f_dc = np.stack([v[f"f_dc_{i}"] for i in range(3)], axis=1)
    f_rest = np.stack([v[f"f_rest_{i}"] for i in range(45)], axis=1).reshape(-1, 3, 15).transpose(0, 2, 1).reshape(n, -1)
    sh = np.ascontiguousarray(np.concatenate([f_dc, f_rest], axis=1).astype(np.float32)).reshape(-1, 16, 3)
    rots = np.ascontiguousarray(np.stack([v[f"rot_{i}"] for i in range(4)], axis=1).astype(np.float32)[:, [1, 2, 3, 0]])
    scales = np.stack([v[f"scale_{i}"] for i in range(3)], axis=1).astype(np.float32)
    opacity = v["opacity"].astype(np.float32)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(device)
    sh_t = t(sh)
    base_t = None
    if split:
        base_t = sh_t[:, 0].contiguous()
        sh_t = sh_t[:, 1:].contiguous()
    cls = GaussianModelOriginFused if fused else GaussianModelOrigin
    model = cls(xyz=t(positions), quaternion_xyzw=t(rots), scale=t(scales), opacity=t(opacity), color_sh=sh_t,
                color_sh_base=base_t)
    model.cur_sh_degree = 3
    return model


def save_3dgs_origin_model(model: GaussianModelOriginBase, path: str) -> None:
    """Writes the layout ``load_3dgs_origin_model`` reads (origin/data/scene/gaussian_model.py:177-208):
    binary little endian, normals zero, raw scale / opacity, rotation wxyz, f_rest channel-major."""
    cpu = lambda x: x.detach().cpu().numpy().astype(np.float32)
    sh = cpu(model.color_sh)
    if model.color_sh_base is not None:
        sh = np.concatenate([cpu(model.color_sh_base)[:, None, :], sh], axis=1)
    n, k = sh.shape[0], sh.shape[1]
    names = ["x", "y", "z", "nx", "ny", "nz"] + [f"f_dc_{i}" for i in range(3)] + \
            [f"f_rest_{i}" for i in range(3 * (k - 1))] + ["opacity"] + [f"scale_{i}" for i in range(3)] + \
            [f"rot_{i}" for i in range(4)]
    table = np.concatenate([cpu(model.xyz), np.zeros((n, 3), np.float32), sh[:, 0, :],
                            sh[:, 1:, :].transpose(0, 2, 1).reshape(n, -1), cpu(model.opacity).reshape(n, 1),
                            cpu(model.scale), cpu(model.quaternion_xyzw)[:, [3, 0, 1, 2]]], axis=1).astype("<f4")
    header = "ply\nformat binary_little_endian 1.0\nelement vertex %d\n" % n + \
             "".join(f"property float {name}\n" for name in names) + "end_header\n"
    with open(path, "wb") as f:
        f.write(header.encode("ascii"))
        f.write(np.ascontiguousarray(table).tobytes())


def nearest_neighbour_distances(points: np.ndarray, k: int = 3) -> np.ndarray:
    """Distances [N, k] from every point to its k nearest other points (what the reference's ``simple_knn`` returns,
    d3sim/algos/d3gs/ops.py:185-214).  A k-d tree on the host: this runs once, when a model is initialised."""
    from scipy.spatial import cKDTree
    pts = np.ascontiguousarray(points, np.float64)
    assert pts.ndim == 2 and pts.shape[1] == 3 and pts.shape[0] > k, "points must be [N, 3] with N > k"
    dist, _ = cKDTree(pts).query(pts, k=k + 1)     # the nearest hit of a point is the point itself
    return dist[:, 1:].astype(np.float32)


def points_to_gaussian_init_scale(points: torch.Tensor) -> torch.Tensor:
    """tools.py:64-69: the log of the root mean square distance to the three nearest neighbours, the same on every
    axis, as the initial (raw) scale [N, 3]."""
    knn = torch.from_numpy(nearest_neighbour_distances(points.detach().cpu().numpy(), 3)).to(points.device)
    dist2 = torch.clamp_min(torch.square(knn).mean(1), 0.0000001)
    return torch.log(torch.sqrt(dist2))[..., None].repeat(1, 3)


def init_original_3dgs_model(model: GaussianModelOriginBase, points: np.ndarray, points_rgb: np.ndarray) -> None:
    """tools.py:71-90: the original recipe's start from a point cloud, written into an allocated model in place:
    positions = points, DC colour from the points' rgb in [0, 1], scale from the neighbour distances, identity
    rotations, opacity 0.1 (as a logit), SH degree 0."""
    with torch.no_grad():
        assert model.xyz.shape[0] == points.shape[0]
        dev = model.xyz.device
        pts = torch.from_numpy(points.astype(np.float32)).to(dev).contiguous()
        dc = rgb_to_sh(torch.from_numpy(points_rgb.astype(np.float32)).to(dev))
        if model.color_sh_base is None:
            model.color_sh[:, 0] = dc
        else:
            model.color_sh_base[:] = dc
        model.scale[:] = points_to_gaussian_init_scale(pts)
        quat = torch.zeros((pts.shape[0], 4), device=dev)
        quat[:, 3] = 1
        model.quaternion_xyzw[:] = quat
        model.opacity[:] = inverse_sigmoid(0.1 * torch.ones(pts.shape[0], dtype=torch.float32, device=dev))
        model.cur_sh_degree = 0
        model.xyz[:] = pts


def get_expon_lr_func(lr_init, lr_final, lr_delay_steps=0, lr_delay_mult=1.0, max_steps=1000000):
    """tools.py:92-126: log-linear interpolation from lr_init to lr_final with an optional sine warm-up."""
    def helper(step):
        if step < 0 or (lr_init == 0.0 and lr_final == 0.0):
            return 0.0
        if lr_delay_steps > 0:
            delay_rate = lr_delay_mult + (1 - lr_delay_mult) * math.sin(0.5 * math.pi * min(max(step / lr_delay_steps, 0), 1))
        else:
            delay_rate = 1.0
        t = min(max(step / max_steps, 0), 1)
        return delay_rate * math.exp(math.log(lr_init) * (1 - t) + math.log(lr_final) * t)
    return helper


def create_origin_3dgs_optimizer(model: GaussianModelOriginBase, optim_cfg, spatial_lr_scale: float):
    """tools.py:129-147: Adam parameter groups of the original 3DGS recipe and the position schedule.
    ``optim_cfg`` carries position_lr_init / position_lr_final / position_lr_delay_mult /
    position_lr_max_steps / feature_lr / opacity_lr / scaling_lr / rotation_lr."""
    groups = [{"params": [model.xyz], "lr": optim_cfg.position_lr_init * spatial_lr_scale, "name": "xyz"}]
    if model.color_sh_base is not None:
        groups.append({"params": [model.color_sh_base], "lr": optim_cfg.feature_lr, "name": "color_sh_base"})
    groups += [
        {"params": [model.color_sh], "lr": optim_cfg.feature_lr / 20.0, "name": "color_sh"},
        {"params": [model.opacity], "lr": optim_cfg.opacity_lr, "name": "opacity"},
        {"params": [model.scale], "lr": optim_cfg.scaling_lr, "name": "scale"},
        {"params": [model.quaternion_xyzw], "lr": optim_cfg.rotation_lr, "name": "quaternion_xyzw"},
    ]
    optim = torch.optim.Adam(groups, lr=0.0, eps=1e-15)
    schedule = get_expon_lr_func(lr_init=optim_cfg.position_lr_init * spatial_lr_scale,
                                 lr_final=optim_cfg.position_lr_final * spatial_lr_scale,
                                 lr_delay_mult=optim_cfg.position_lr_delay_mult,
                                 max_steps=optim_cfg.position_lr_max_steps)
    return optim, schedule


def create_origin_xyz_scheduler(optim_cfg, batch_size: int, spatial_lr_scale: float):
    """tools.py:175-181: the position schedule for a step over ``batch_size`` views (rates scaled by its root)."""
    bs_scale = math.sqrt(batch_size)
    return get_expon_lr_func(lr_init=optim_cfg.position_lr_init * spatial_lr_scale * bs_scale,
                             lr_final=optim_cfg.position_lr_final * spatial_lr_scale * bs_scale,
                             lr_delay_mult=optim_cfg.position_lr_delay_mult,
                             max_steps=optim_cfg.position_lr_max_steps)


def create_origin_3dgs_optimizers(model: GaussianModelOriginBase, optim_cfg, batch_size: int, spatial_lr_scale: float,
                                  fused: bool = True):
    """tools.py:146-173: one optimizer per parameter group for steps over ``batch_size`` views: rates scaled by
    sqrt(batch_size), eps by its inverse, and the betas of ``batch_size`` single-view steps folded into one,
    1 - batch_size (1 - beta).  The reference instantiates its own fused Adam kernel per group; here each group gets a
    ``torch.optim.Adam`` (``fused`` asks for torch's fused implementation).  Returns ({name: optimizer}, schedule)."""
    bs_scale = math.sqrt(batch_size)
    groups = [("xyz", model.xyz, optim_cfg.position_lr_init * spatial_lr_scale * bs_scale)]
    if model.color_sh_base is not None:
        groups.append(("color_sh_base", model.color_sh_base, optim_cfg.feature_lr * bs_scale))
    groups += [("color_sh", model.color_sh, optim_cfg.feature_lr * bs_scale / 20.0),
               ("opacity", model.opacity, optim_cfg.opacity_lr * bs_scale),
               ("scale", model.scale, optim_cfg.scaling_lr * bs_scale),
               ("quaternion_xyzw", model.quaternion_xyzw, optim_cfg.rotation_lr * bs_scale)]
    betas = (1 - batch_size * (1 - 0.9), 1 - batch_size * (1 - 0.999))
    optimizers = {}
    for name, tensor, lr in groups:
        use_fused = bool(fused and tensor.is_cuda)
        optimizers[name] = torch.optim.Adam([{"params": [tensor], "lr": lr, "name": name}], lr=lr, eps=1e-15 / bs_scale,
                                            betas=betas, fused=use_fused)
    return optimizers, create_origin_xyz_scheduler(optim_cfg, batch_size, spatial_lr_scale)
