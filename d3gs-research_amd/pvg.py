"""Time-dependent gaussians (periodic vibration): the ``PVGGaussianModel`` family of the reference
(d3sim/algos/d3gs/pvg/model.py:13-39, 103-126, 248-268).

The reference evaluates this family inside its JIT-compiled preprocess kernels through a code-emitting proxy.
An ahead-of-time library has no such hook, and does not need one: the family only changes where a gaussian is
and how opaque it is at the camera's time stamp,

    a         = 2 pi / cycle
    xyz(t)    = xyz + velocity * sin((t - t_g) a) / a + velocity * exp(-exp(scale_t) / cycle / 2 * decay) * time_shift
    marginal  = exp(-(t_g - t)^2 / (2 exp(scale_t)^2))
    opacity(t)= sigmoid(opacity) * marginal            gaussians with marginal <= 0.05 are not rendered

with ``t = batch_ts[camera] - time_shift``.  Here these few element-wise operations run in torch (autograd
carries the gradients back to t_g, velocity and scale_t), and the operator receives the result as a model whose
activations are already applied.  ``rasterize_gaussians_dynamic`` keeps the reference's call
(render.py:3840-3891): ``prep_input_tensors={"batch_ts": ...}``, ``prep_inputs={"time_shift": ...}``.
"""
from __future__ import annotations

import dataclasses
import math

import torch

from .model import GaussianModelOrigin, GaussianModelOriginBase, GaussianModelOriginFused
from .render import CameraBundle, GaussianSplatOp, GaussianSplatOutput, rasterize_gaussians

MARGINAL_T_MIN = 0.05      # pvg/model.py:124-126


@dataclasses.dataclass(kw_only=True)
class PVGGaussianModel(GaussianModelOriginFused):
    """pvg/model.py:248-268.  Raw fields as in ``GaussianModelOriginFused`` plus the three temporal ones."""
    velocity: torch.Tensor = None       # [N, 3]
    scaling_t: torch.Tensor = None      # [N, 1] log of the temporal standard deviation
    t: torch.Tensor = None              # [N, 1] time of the gaussian's peak
    cycle: float = 0.2
    velocity_decay: float = 1.0

    def get_proxy_field_dict(self):
        res = super().get_proxy_field_dict()
        res.update(velocity=self.velocity, scaling_t=self.scaling_t, t=self.t)
        return res

    def at_time(self, batch_t, time_shift: float = 0.0):
        """The gaussians as seen at time ``batch_t`` (a python float or a 0-d tensor; the caller has already
        subtracted ``time_shift``, pvg/model.py:107): an activated ``GaussianModelOrigin`` and the bool mask of
        the gaussians the reference rejects (marginal <= 0.05).  Differentiable in every raw field."""
        assert not self.act_applied, "at_time takes the raw model"
        a = 2.0 * math.pi / self.cycle
        t_g = self.t.reshape(-1)
        sigma_t = torch.exp(self.scaling_t.reshape(-1))
        dt = batch_t - t_g
        xyz = self.xyz + self.velocity * (torch.sin(dt * a) / a).unsqueeze(-1)
        if time_shift != 0.0:
            inst = torch.exp(-sigma_t / self.cycle / 2.0 * self.velocity_decay)
            xyz = xyz + self.velocity * (inst * time_shift).unsqueeze(-1)
        marginal = torch.exp(-0.5 * dt * dt / sigma_t / sigma_t)
        model = GaussianModelOrigin(
            xyz=xyz, quaternion_xyzw=torch.nn.functional.normalize(self.quaternion_xyzw, p=2, dim=-1),
            scale=torch.exp(self.scale), opacity=torch.sigmoid(self.opacity) * marginal, color_sh=self.color_sh,
            color_sh_base=self.color_sh_base, instance_id=self.instance_id, act_applied=True,
            cur_sh_degree=self.cur_sh_degree)
        return model, (marginal <= MARGINAL_T_MIN).detach()


def rasterize_gaussians_dynamic(model: GaussianModelOriginBase, cameras, op: GaussianSplatOp, training=False,
                                uv_grad_holder: torch.Tensor | None = None, instance2world_T=None,
                                custom_features=None, prep_input_tensors: dict | None = None,
                                prep_inputs: dict | None = None, mask=None) -> GaussianSplatOutput:
    """render.py:3840-3891.  A model without time dependence goes straight to ``rasterize_gaussians``; a
    ``PVGGaussianModel`` is evaluated at each camera's time stamp first (``batch_ts`` [B] and ``time_shift``,
    looked up in either dictionary, pvg/model.py:50-52) and rendered camera by camera."""
    inputs = {**(prep_inputs or {}), **(prep_input_tensors or {})}
    if not isinstance(model, PVGGaussianModel):
        if inputs:
            raise NotImplementedError(f"{type(model).__name__} takes no preprocess inputs (got {sorted(inputs)})")
        return rasterize_gaussians(model, cameras, op, training, uv_grad_holder, instance2world_T, custom_features, mask)
    assert "batch_ts" in inputs and "time_shift" in inputs, "PVG needs batch_ts and time_shift"   # pvg/model.py:50-52
    batch_ts, time_shift = inputs["batch_ts"], float(inputs["time_shift"])
    num_cams = len(cameras) if isinstance(cameras, CameraBundle) else 1
    assert batch_ts.numel() == num_cams, "one time stamp per camera"
    assert uv_grad_holder is None or num_cams == 1, "uv_grad_holder: one camera per call"
    n = len(model)
    outs = []
    for b in range(num_cams):
        cam = cameras.select(b) if isinstance(cameras, CameraBundle) else cameras
        model_t, too_faint = model.at_time(batch_ts.reshape(-1)[b] - time_shift, time_shift)
        reject = too_faint
        if mask is not None:
            reject = reject | mask.reshape(num_cams, n)[b].to(torch.bool)
        outs.append(rasterize_gaussians(model_t, cam, op, training, uv_grad_holder, instance2world_T,
                                        custom_features, reject.contiguous()))
    if num_cams == 1:
        return outs[0]
    cat = lambda name: None if getattr(outs[0], name) is None else torch.cat([getattr(o, name) for o in outs], 0)
    return GaussianSplatOutput(custom_features=cat("custom_features"), T=cat("T"), color=cat("color"),
                               depth=cat("depth"), n_contrib=cat("n_contrib"), radii=cat("radii"))
