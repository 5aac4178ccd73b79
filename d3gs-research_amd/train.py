"""The training step that drives the rasterizer the way the reference trainer does
(d3sim/algos/d3gs/train.py:107-284, 299-354): render with a screen-gradient holder, L1 + D-SSIM
loss, Adam step, densification statistics, and the periodic events (SH degree up, refine, opacity
reset).  Data loading, evaluation metrics and logging stay with the caller.
"""
from __future__ import annotations

import dataclasses
import math

import torch
import torch.nn.functional as F

from . import config_def
from .model import GaussianModelOriginBase
from .render import CameraBundle, GaussianSplatOp, GaussianSplatOutput, rasterize_gaussians
from .strategy import GaussianStrategyOrigin, GaussianTrainState
from .tools import create_origin_3dgs_optimizer, create_origin_3dgs_optimizers


def l1_loss(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """losses.py:19-20."""
    return (a - b).abs().mean()


def _window(size: int, sigma: float, device, dtype) -> torch.Tensor:
    x = torch.arange(size, device=device, dtype=dtype) - size // 2
    g = torch.exp(-(x * x) / (2.0 * sigma * sigma))
    return g / g.sum()


def ssim(img1: torch.Tensor, img2: torch.Tensor, window_size: int = 11, size_average: bool = True) -> torch.Tensor:
    """Structural similarity of [B, C, H, W] images in [0, 1] (Wang et al. 2004) with the reference's
    choices (losses.py:26-73): 11-tap gaussian window of sigma 1.5, zero padding, C1 = 0.01^2,
    C2 = 0.03^2.  The 2-D window is separable, so it is applied as two 1-D passes."""
    c = img1.shape[-3]
    w = _window(window_size, 1.5, img1.device, img1.dtype)
    wx = w.view(1, 1, 1, -1).expand(c, 1, 1, window_size)
    wy = w.view(1, 1, -1, 1).expand(c, 1, window_size, 1)
    pad = window_size // 2

    def blur(x):
        return F.conv2d(F.conv2d(x, wx, padding=(0, pad), groups=c), wy, padding=(pad, 0), groups=c)

    mu1, mu2 = blur(img1), blur(img2)
    mu1_sq, mu2_sq, mu12 = mu1 * mu1, mu2 * mu2, mu1 * mu2
    s1 = blur(img1 * img1) - mu1_sq
    s2 = blur(img2 * img2) - mu2_sq
    s12 = blur(img1 * img2) - mu12
    c1, c2 = 0.01 ** 2, 0.03 ** 2
    m = ((2 * mu12 + c1) * (2 * s12 + c2)) / ((mu1_sq + mu2_sq + c1) * (s1 + s2 + c2))
    return m.mean() if size_average else m.mean(dim=(1, 2, 3))


def photometric_loss(color_nchw: torch.Tensor, gt_nchw: torch.Tensor, lambda_dssim: float) -> torch.Tensor:
    """train.py:170-172: (1 - lambda) L1 + lambda (1 - SSIM)."""
    return (1.0 - lambda_dssim) * l1_loss(color_nchw, gt_nchw) + lambda_dssim * (1.0 - ssim(color_nchw, gt_nchw))


@dataclasses.dataclass
class StepResult:
    loss: float
    output: GaussianSplatOutput
    refined: bool = False
    reset_opacity: bool = False


class Trainer:
    """One model, one rasterizer op, the original recipe's optimizer and densification strategy."""

    def __init__(self, model: GaussianModelOriginBase, op: GaussianSplatOp, cfg: config_def.Train | None = None,
                 scene_scale: float = 1.0, spatial_lr_scale: float | None = None):
        self.cfg = cfg or config_def.Train()
        self.model = model
        self.op = op
        model.act_applied = False
        model.set_requires_grad(True)
        lr_scale = scene_scale if spatial_lr_scale is None else spatial_lr_scale
        if self.cfg.batch_size > 1:
            # steps over several views (train.py:46-52): the schedules shrink by the batch size, and every
            # parameter group gets its own optimizer with rates, eps and betas scaled for it (tools.py:146-173)
            self.cfg.rescale_steps_by_batch_size(self.cfg.batch_size)
            self.optim, self.xyz_schedule = create_origin_3dgs_optimizers(model, self.cfg.optim, self.cfg.batch_size,
                                                                          lr_scale)
        else:
            self.optim, self.xyz_schedule = create_origin_3dgs_optimizer(model, self.cfg.optim, lr_scale)
        self.strategy = GaussianStrategyOrigin.from_config(self.cfg.strategy)
        self.state = GaussianTrainState.create(len(model), scene_scale, device=model.xyz.device)
        self.step = 0

    def _optimizers(self):
        return list(self.optim.values()) if isinstance(self.optim, dict) else [self.optim]

    def _set_position_lr(self):
        lr = self.xyz_schedule(self.step)
        for optim in self._optimizers():
            for group in optim.param_groups:
                if group["name"] == "xyz":
                    group["lr"] = lr

    def train_step(self, cameras, gt_image: torch.Tensor, generator: torch.Generator | None = None) -> StepResult:
        """cameras: one camera or a CameraBundle; gt_image: [B, 3, H, W] in [0, 1]."""
        cfg, st = self.cfg, self.cfg.strategy
        B = len(cameras) if isinstance(cameras, CameraBundle) else 1
        n = len(self.model)
        self._set_position_lr()
        holder = torch.zeros((B, n, 2), dtype=torch.float32, device=self.model.xyz.device, requires_grad=True)
        out = rasterize_gaussians(self.model, cameras, self.op, training=True, uv_grad_holder=holder)
        color = out.color if self.op.is_nchw else out.color.permute(0, 3, 1, 2).contiguous()
        loss = photometric_loss(color[:, :3], gt_image, cfg.lambda_dssim)
        loss.backward()
        for optim in self._optimizers():
            optim.step()
            optim.zero_grad(set_to_none=True)
        done = self.step + 1
        res = StepResult(float(loss.detach()), out)
        if done < st.refine_stop_iter and holder.grad is not None:
            self.strategy.update(self.state, out, holder.grad)
        if done % max(1000 // cfg.batch_size, 1) == 0 and self.model.cur_sh_degree < min(3, self.model.color_sh_degree):
            self.model.cur_sh_degree += 1                                        # train.py:299-302
        if done < st.refine_stop_iter:
            if st.refine_every > 0 and done % st.refine_every == 0 and done > st.refine_start_iter:
                self.strategy.refine_gs(self.model, self.optim, self.state, done, generator)   # train.py:304-317
                res.refined = True
            if st.reset_opacity_every > 0 and done % st.reset_opacity_every == 0:
                self.strategy.reset_opacity(self.model, self.optim)              # train.py:319-354
                res.reset_opacity = True
        self.step = done
        return res


def psnr(a: torch.Tensor, b: torch.Tensor) -> float:
    mse = float(((a - b) ** 2).mean())
    return float("inf") if mse == 0 else -10.0 * math.log10(mse)
