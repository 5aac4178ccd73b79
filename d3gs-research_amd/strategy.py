"""Densification of the original 3DGS recipe: per-gaussian statistics of the screen-space gradient,
clone / split / prune, opacity reset, and the matching surgery on the optimizer state.

Restates d3sim/algos/d3gs/strategy.py:86-202 (train state, optimizer helpers) and
origin/strategy.py:19-364 (``GaussianStrategyOrigin``) with torch operations: the reference runs
these few per-gaussian formulas through its JIT kernel builder; none of them is on the render path.
"""
from __future__ import annotations

import dataclasses
from typing import Mapping

import torch
from torch.optim.optimizer import Optimizer

from . import config_def
from .model import GaussianModelOriginBase, GaussianModelOriginFused

_FIELDS = ("xyz", "quaternion_xyzw", "scale", "opacity", "color_sh", "color_sh_base")


@dataclasses.dataclass
class GaussianTrainState:
    """strategy.py:86-110.  duv_ndc_length accumulates |duv * 0.5 * (W, H)| over the views in which the
    gaussian was visible, count the number of such views, max_radii the largest screen radius / max(W, H)."""
    duv_ndc_length: torch.Tensor
    count: torch.Tensor
    max_radii: torch.Tensor
    scene_scale: float = 1.0

    @classmethod
    def create(cls, num_gaussian: int, scene_scale: float = 1.0, device=None):
        z = lambda: torch.zeros(num_gaussian, dtype=torch.float32, device=device)
        return cls(z(), z(), z(), scene_scale)

    def reset(self):
        self.duv_ndc_length.zero_()
        self.count.zero_()
        self.max_radii.zero_()

    def select(self, index: torch.Tensor) -> "GaussianTrainState":
        return GaussianTrainState(self.duv_ndc_length[index], self.count[index], self.max_radii[index], self.scene_scale)

    def concat(self, other: "GaussianTrainState") -> "GaussianTrainState":
        return GaussianTrainState(torch.cat([self.duv_ndc_length, other.duv_ndc_length]),
                                  torch.cat([self.count, other.count]), torch.cat([self.max_radii, other.max_radii]),
                                  self.scene_scale)

    def assign_inplace(self, other: "GaussianTrainState"):
        self.duv_ndc_length, self.count, self.max_radii = other.duv_ndc_length, other.count, other.max_radii


def activated(model: GaussianModelOriginBase):
    """(xyz, quaternion, scale, opacity) with the model family's activations applied
    (origin/model.py:249-270 in torch, 435-465 inside the kernels)."""
    if model.act_applied:
        return model.xyz, model.quaternion_xyzw, model.scale, model.opacity
    if isinstance(model, GaussianModelOriginFused):
        return (model.xyz, torch.nn.functional.normalize(model.quaternion_xyzw, p=2, dim=-1), torch.exp(model.scale),
                torch.sigmoid(model.opacity))
    return model.xyz_act, model.quaternion_xyzw_act, model.scale_act, model.opacity_act


def quat_xyzw_to_rotmat(q: torch.Tensor) -> torch.Tensor:
    """Rotation matrices R (``R @ v`` rotates v) of unit quaternions stored (x, y, z, w)."""
    x, y, z, w = q.unbind(-1)
    return torch.stack([
        1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y),
        2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x),
        2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], -1).reshape(q.shape[:-1] + (3, 3))


# ------------------------------------------------------------- optimizer state
def _groups(optimizers: Mapping[str, Optimizer] | Optimizer):
    if isinstance(optimizers, Optimizer):
        for group in optimizers.param_groups:
            yield optimizers, group, group["name"]
    else:
        for name, opt in optimizers.items():
            for group in opt.param_groups:
                yield opt, group, name


@torch.no_grad()
def _update_optimizer_only(param_fn, state_fn, optimizers, names):
    """strategy.py:17-66: swap the parameter of every named group and map its state tensors."""
    for opt, group, name in _groups(optimizers):
        if name not in names:
            continue
        p = group["params"][0]
        p_state = opt.state.pop(p, {})
        for key, v in list(p_state.items()):
            if key != "step" and v is not None:
                p_state[key] = state_fn(key, v)
        p_new = param_fn(name, p)
        group["params"] = [p_new]
        if p_state:
            opt.state[p_new] = p_state


def _model_names(model):
    return [k for k in _FIELDS if getattr(model, k) is not None]


def select_gs_optimizer_by_mask(model, optimizers, inds: torch.Tensor):
    """strategy.py:129-150: the optimizer state follows the gaussians gathered by ``inds``."""
    _update_optimizer_only(lambda name, p: getattr(model, name), lambda key, v: v[inds], optimizers, _model_names(model))


def zero_optimizer_by_range(model, optimizers, interval: tuple[int, int]):
    """strategy.py:153-176: fresh (zero) moments for the gaussians in ``interval``."""
    def state_fn(key, v):
        v[interval[0]:interval[1]].zero_()
        return v
    _update_optimizer_only(lambda name, p: getattr(model, name), state_fn, optimizers, _model_names(model))


def reset_param_in_optim(model, optimizers, name: str):
    """strategy.py:179-202."""
    _update_optimizer_only(lambda n, p: getattr(model, n), lambda key, v: torch.zeros_like(v), optimizers, [name])


def _index_model(model, index):
    return {k: getattr(model, k)[index] for k in _model_names(model)}


# -------------------------------------------------------------------- strategy
@dataclasses.dataclass
class GaussianStrategyOrigin(config_def.Strategy):
    """origin/strategy.py:19-364."""

    @classmethod
    def from_config(cls, cfg: config_def.Strategy):
        return cls(**dataclasses.asdict(cfg))

    @torch.no_grad()
    def update(self, state: GaussianTrainState, out, duv: torch.Tensor):
        """origin/strategy.py:75-122: duv [B, N, 2] (the gradient holder's grad), out.radii flat [B * N].
        The gradient of a mean-over-batch loss is scaled back by B."""
        width, height = out.image_shape_wh
        assert duv.ndim == 3 and out.radii is not None
        B, N = duv.shape[0], duv.shape[1]
        radii = out.radii.reshape(B, N)
        assert N == state.duv_ndc_length.shape[0]
        scale = torch.tensor([0.5 * width * B, 0.5 * height * B], dtype=duv.dtype, device=duv.device)
        length = torch.linalg.norm(duv * scale, dim=-1)
        seen = radii > 0
        state.duv_ndc_length += (length * seen).sum(0)
        state.count += seen.sum(0).to(state.count.dtype)
        if self.refine_scale2d_stop_iter > 0:
            r = torch.where(seen, radii.to(torch.float32) / float(max(width, height)), torch.zeros((), device=duv.device))
            state.max_radii.copy_(torch.maximum(state.max_radii, r.max(0).values))

    @torch.no_grad()
    def update_v1(self, state: GaussianTrainState, out, duv: torch.Tensor):
        """origin/strategy.py:45-73, the earlier form: duv [..., N, 2] and out.radii of the same leading shape; the
        gradient is scaled to NDC by (width / 2, height / 2) without the batch factor, and every (view, gaussian)
        with a positive radius adds its length and one count to the gaussian."""
        width, height = out.image_shape_wh
        n = state.duv_ndc_length.shape[0]
        scale = torch.tensor([width / 2.0, height / 2.0], dtype=duv.dtype, device=duv.device)
        length = torch.linalg.norm(duv * scale, dim=-1).reshape(-1, n)
        radii = out.radii.reshape(-1, n)
        seen = radii > 0
        state.duv_ndc_length += (length * seen).sum(0)
        state.count += seen.sum(0).to(state.count.dtype)
        if self.refine_scale2d_stop_iter > 0:
            r = torch.where(seen, radii.to(torch.float32) / float(max(width, height)), torch.zeros((), device=duv.device))
            state.max_radii.copy_(torch.maximum(state.max_radii, r.max(0).values))

    @torch.no_grad()
    def update_v2(self, state: GaussianTrainState, out, duv: torch.Tensor, batch_size: int = 1):
        """origin/strategy.py:125-157: one state row per row of duv (duv.reshape(-1, 2) and out.radii flat have the
        state's length); the gradient of a mean over ``batch_size`` views is scaled back by it."""
        width, height = out.image_shape_wh
        flat = duv.reshape(-1, 2)
        radii = out.radii.reshape(-1)
        assert flat.shape[0] == radii.shape[0] == state.duv_ndc_length.shape[0] == state.count.shape[0]
        scale = torch.tensor([0.5 * width * batch_size, 0.5 * height * batch_size], dtype=duv.dtype, device=duv.device)
        length = torch.linalg.norm(flat * scale, dim=-1)
        seen = radii > 0
        state.duv_ndc_length += length * seen
        state.count += seen.to(state.count.dtype)
        if self.refine_scale2d_stop_iter > 0:
            r = torch.where(seen, radii.to(torch.float32) / float(max(width, height)), torch.zeros((), device=duv.device))
            state.max_radii.copy_(torch.maximum(state.max_radii, r))

    @torch.no_grad()
    def refine_gs(self, model: GaussianModelOriginBase, optimizers, state: GaussianTrainState, step: int,
                  generator: torch.Generator | None = None):
        """origin/strategy.py:160-364: clone small gaussians with a high screen-space gradient, split
        large ones in two (sampled inside the parent, scale / 1.6), prune transparent (and, after the
        first opacity reset, oversized) ones; statistics restart and the new gaussians get zero moments."""
        n = len(model)
        dev = model.xyz.device
        xyz, quat, scales, opacity = activated(model)
        refine_by_radii = step < self.refine_scale2d_stop_iter
        prune_too_big = step > self.reset_opacity_every
        assert not refine_by_radii
        scene_scale = state.scene_scale
        assert n == state.duv_ndc_length.shape[0] == state.count.shape[0] == state.max_radii.shape[0]

        is_grad_high = state.duv_ndc_length / torch.clamp_min(state.count, 1.0) >= self.grow_grad2d
        scale_max = scales.max(dim=-1).values
        is_small = scale_max <= self.grow_scale3d * scene_scale
        should_dupti = is_grad_high & is_small
        prune_origin = opacity < self.prune_opacity_thresh
        if prune_too_big:
            prune_origin = prune_origin | (scale_max > self.prune_scale3d * scene_scale)
        should_split = is_grad_high & ~is_small
        origin_should_prune = prune_origin | should_split

        dupti_inds = torch.nonzero(should_dupti).view(-1)
        split_inds = torch.nonzero(should_split).view(-1)
        n_dupti, n_split = int(dupti_inds.numel()), int(split_inds.numel())
        if self.verbose:
            print("n_dupti", n_dupti, "n_split", n_split)
        new_inds = torch.cat([dupti_inds, split_inds, split_inds])
        new_fields = _index_model(model, new_inds)
        new_state = state.select(new_inds)
        new_should_prune = torch.zeros(new_inds.numel(), dtype=torch.bool, device=dev)
        new_should_prune[:n_dupti] = origin_should_prune[dupti_inds]

        # the two children of a split: a sample of the parent's own distribution, scale / (0.8 * 2)
        two = torch.cat([split_inds, split_inds])
        normals = torch.randn(n_split * 2, 3, device=dev, generator=generator)
        R = quat_xyzw_to_rotmat(quat[two])
        new_xyz = (R @ (normals * scales[two]).unsqueeze(-1)).squeeze(-1) + xyz[two]
        new_scaling = scales[two] / (0.8 * 2)
        new_fields["xyz"][n_dupti:] = new_xyz
        new_fields["scale"][n_dupti:] = torch.log(new_scaling)
        split_prune = opacity[two] < self.prune_opacity_thresh
        if prune_too_big:
            split_prune = split_prune | (new_scaling.max(dim=-1).values > self.prune_scale3d * scene_scale)
        new_should_prune[n_dupti:] = split_prune

        keep_origin = torch.nonzero(~origin_should_prune).view(-1)
        keep_new = torch.nonzero(~new_should_prune).view(-1)
        for k in _model_names(model):
            merged = torch.cat([getattr(model, k)[keep_origin], new_fields[k][keep_new]], 0).contiguous()
            setattr(model, k, merged.requires_grad_(True))
        state.assign_inplace(state.select(keep_origin).concat(new_state.select(keep_new)))
        state.reset()
        res_inds = torch.cat([keep_origin, new_inds[keep_new]])
        select_gs_optimizer_by_mask(model, optimizers, res_inds)
        zero_optimizer_by_range(model, optimizers, (int(keep_origin.numel()), int(res_inds.numel())))
        return model

    @torch.no_grad()
    def reset_opacity(self, model: GaussianModelOriginBase, optimizers):
        """train.py:319-354: activated opacity clamped from above at reset_opacity_thresh, stored as its logit."""
        _, _, _, opacity = activated(model)
        o = torch.clamp_max(opacity, self.reset_opacity_thresh)
        model.opacity = torch.log(o / (1.0 - o)).requires_grad_(True)
        reset_param_in_optim(model, optimizers, "opacity")
