"""Gaussian model containers with the reference's tensor layout.

``GaussianModelOriginFused`` mirrors d3sim/algos/d3gs/origin/model.py:34-48 and
435-465: raw (pre-activation) tensors whose activations — exp for scale,
normalize for the quaternion, sigmoid for opacity — are applied inside the
preprocess kernel.  ``GaussianModelOrigin`` (origin/model.py:249-270) applies the
same activations with torch before the operator runs, so autograd differentiates
them and the kernels see activated values.  Quaternions are stored (x, y, z, w).
"""
from __future__ import annotations

import dataclasses
import math

import torch


@dataclasses.dataclass(kw_only=True)
class GaussianModelOriginBase:
    xyz: torch.Tensor                    # [N, 3] f32
    quaternion_xyzw: torch.Tensor        # [N, 4] f32
    scale: torch.Tensor                  # [N, 3] f32 (log-scale)
    opacity: torch.Tensor                # [N]    f32 (logit)
    color_sh: torch.Tensor               # [N, K, 3] f32
    color_sh_base: torch.Tensor | None = None   # [N, 3] f32 when the DC term is split off
    instance_id: torch.Tensor | None = None
    act_applied: bool = False
    cur_sh_degree: int = 0

    def __len__(self):
        return self.xyz.shape[0]

    @property
    def color_sh_degree(self) -> int:
        dim = self.color_sh.shape[1]
        if self.color_sh_base is not None:
            dim += 1
        res = int(math.sqrt(dim)) - 1
        assert (res + 1) * (res + 1) == dim
        return res

    def get_proxy_field_dict(self):
        res = {"xyz": self.xyz, "quaternion_xyzw": self.quaternion_xyzw, "scale": self.scale,
               "opacity": self.opacity, "color_sh": self.color_sh}
        if self.color_sh_base is not None:
            res["color_sh_base"] = self.color_sh_base
        return res

    def set_requires_grad(self, requires_grad: bool):
        for t in self.get_proxy_field_dict().values():
            t.requires_grad_(requires_grad)

    def clear_grad(self):
        for t in self.get_proxy_field_dict().values():
            t.grad = None

    # activated views (origin/model.py:50-84); the base class has identity activations
    @property
    def xyz_act(self) -> torch.Tensor:
        return self.xyz

    @property
    def quaternion_xyzw_act(self) -> torch.Tensor:
        return self.quaternion_xyzw

    @property
    def scale_act(self) -> torch.Tensor:
        return self.scale

    @property
    def opacity_act(self) -> torch.Tensor:
        return self.opacity

    def create_model_with_act(self):
        """origin/model.py:144-156."""
        if self.act_applied:
            return dataclasses.replace(self)
        return dataclasses.replace(self, xyz=self.xyz_act, quaternion_xyzw=self.quaternion_xyzw_act,
                                   scale=self.scale_act, opacity=self.opacity_act, act_applied=True)

    def to_device(self, device):
        kw = {k: v.to(device) for k, v in self.get_proxy_field_dict().items()}
        return dataclasses.replace(self, **kw)

    @property
    def color_sh_act(self) -> torch.Tensor:
        return self.color_sh

    @property
    def color_sh_base_act(self) -> torch.Tensor | None:
        return self.color_sh_base

    # constructors (origin/model.py:158-246)
    @classmethod
    def _allocate(cls, make, N: int, max_num_degree: int, split: bool, dtype, device, opacity=None):
        coefficients = (max_num_degree + 1) * (max_num_degree + 1) - (1 if split else 0)
        return cls(xyz=make(N, 3, dtype=dtype, device=device), quaternion_xyzw=make(N, 4, dtype=dtype, device=device),
                   scale=make(N, 3, dtype=dtype, device=device),
                   opacity=opacity if opacity is not None else make(N, dtype=dtype, device=device),
                   color_sh_base=make(N, 3, dtype=dtype, device=device) if split else None,
                   color_sh=make(N, coefficients, 3, dtype=dtype, device=device), cur_sh_degree=0)

    @classmethod
    def empty(cls, N: int, max_num_degree: int, split: bool = False, dtype: torch.dtype = torch.float32,
              device: torch.device | str = "cuda"):
        """origin/model.py:158-178: uninitialised tensors for N gaussians with SH up to ``max_num_degree``; ``split``
        keeps the DC coefficient in ``color_sh_base``."""
        return cls._allocate(torch.empty, N, max_num_degree, split, dtype, device)

    @classmethod
    def zeros(cls, N: int, max_num_degree: int, split: bool = False, dtype: torch.dtype = torch.float32,
              device: torch.device | str = "cpu", opacity: torch.Tensor | None = None):
        """origin/model.py:208-229 (``opacity`` lets a caller hand in storage it already has)."""
        return cls._allocate(torch.zeros, N, max_num_degree, split, dtype, device, opacity)

    @classmethod
    def zeros_like_debug(cls, model: "GaussianModelOriginBase", opacity: torch.Tensor | None = None):
        """origin/model.py:231-246: zeros with the shapes of ``model``."""
        return cls.zeros(len(model), model.color_sh_degree, model.color_sh_base is not None, model.xyz.dtype,
                         model.xyz.device, opacity)

    @classmethod
    def create_from_points(cls, points, points_rgb, device: torch.device | str = "cuda"):
        """The original recipe's start from a point cloud (origin/model.py:180-206, ``create_from_dataset`` applied
        to the dataset's ``dataset_point_cloud.xyz`` / ``.rgb``; dataset readers are not part of this package):
        degree-3 storage with a split DC term, initialised by ``tools.init_original_3dgs_model``."""
        from . import tools
        model = cls.empty(points.shape[0], 3, True, device=device)
        model.color_sh.zero_()
        tools.init_original_3dgs_model(model, points, points_rgb)
        return model


@dataclasses.dataclass(kw_only=True)
class GaussianModelOriginFused(GaussianModelOriginBase):
    """Activations fused into the kernels (origin/model.py:435-465)."""

    @property
    def fused_quaternion_xyzw_act_op(self):
        return ("normalize", "normalize_grad_out")

    @property
    def fused_scale_act_op(self):
        return ("exponential", "exponential_grad_out")

    @property
    def fused_opacity_act_op(self):
        return ("sigmoid", "sigmoid_grad_out")


@dataclasses.dataclass(kw_only=True)
class GaussianModelOrigin(GaussianModelOriginBase):
    """Activations applied by torch ahead of the operator (origin/model.py:249-270)."""

    @property
    def quaternion_xyzw_act(self) -> torch.Tensor:
        if self.act_applied:
            return self.quaternion_xyzw
        return torch.nn.functional.normalize(self.quaternion_xyzw, p=2, dim=-1)

    @property
    def scale_act(self) -> torch.Tensor:
        if self.act_applied:
            return self.scale
        return torch.exp(self.scale)

    def inverse_scale_act(self, scale_act: torch.Tensor) -> torch.Tensor:
        return torch.log(scale_act)

    @property
    def opacity_act(self) -> torch.Tensor:
        if self.act_applied:
            return self.opacity
        return torch.sigmoid(self.opacity)
