"""The operator used the way the reference's trainer uses it (d3sim/algos/d3gs/train.py:162-177):
rasterize_gaussians(model, cam, op, training=True, uv_grad_holder=h) -> loss -> loss.backward()
-> optimizer step.  A perturbed copy of a scene must move back towards the image of the original."""
import numpy as np
import pytest

from helpers import gen_scene, op_config, torch_model

pytestmark = pytest.mark.gpu


def test_adam_steps_reduce_the_image_loss():
    import torch
    from d3gs_research_amd.render import GaussianSplatOp, rasterize_gaussians

    scene = gen_scene(1, n=20000, wh=(256, 256))
    cam = scene.camera()
    op = GaussianSplatOp(op_config(scene, 4))          # the reference's default filter (OBB_DFVT)
    target_model = torch_model(scene)
    with torch.no_grad():
        target = rasterize_gaussians(target_model, cam, op, training=True).color.clone()

    model = torch_model(scene)
    model.act_applied = False
    g = torch.Generator(device="cuda").manual_seed(3)
    with torch.no_grad():
        model.xyz += 0.01 * torch.randn(model.xyz.shape, generator=g, device="cuda")
        model.scale += 0.1 * torch.randn(model.scale.shape, generator=g, device="cuda")
        model.opacity += 0.3 * torch.randn(model.opacity.shape, generator=g, device="cuda")
        model.color_sh += 0.05 * torch.randn(model.color_sh.shape, generator=g, device="cuda")
    model.set_requires_grad(True)
    params = [model.xyz, model.scale, model.quaternion_xyzw, model.opacity, model.color_sh]
    opt = torch.optim.Adam([{"params": [model.xyz], "lr": 2e-4}, {"params": [model.scale], "lr": 5e-3},
                            {"params": [model.quaternion_xyzw], "lr": 1e-3}, {"params": [model.opacity], "lr": 2e-2},
                            {"params": [model.color_sh], "lr": 2.5e-3}])
    losses = []
    for step in range(40):
        holder = torch.zeros((1, scene.n, 2), device="cuda", requires_grad=True)
        out = rasterize_gaussians(model, cam, op, training=True, uv_grad_holder=holder)
        loss = (out.color - target).abs().mean()
        opt.zero_grad(set_to_none=True)
        loss.backward()
        assert all(p.grad is not None and bool(torch.isfinite(p.grad).all()) for p in params)
        assert holder.grad is not None and holder.grad.shape == (1, scene.n, 2)   # the densification signal
        opt.step()
        losses.append(float(loss.detach()))
    print("L1 loss: first %.5f  last %.5f" % (losses[0], losses[-1]), flush=True)
    assert losses[-1] < 0.6 * losses[0]
    assert np.isfinite(losses).all()


def test_trainer_with_densification_and_opacity_reset():
    """Trainer.train_step (train.py:107-284) over two cameras of a synthetic target: photometric loss
    falls, refine_gs changes the gaussian count, the opacity reset happens, the optimizer keeps
    stepping on the re-allocated tensors."""
    import torch
    from d3gs_research_amd import config_def
    from d3gs_research_amd.camera import BasicPinholeCamera
    from d3gs_research_amd.render import CameraBundle, GaussianSplatOp, rasterize_gaussians
    from d3gs_research_amd.train import Trainer

    scene = gen_scene(1, n=8000, wh=(192, 160))
    cams = []
    for dx in (-0.3, 0.3):
        tw = np.array(scene.to_world, np.float64)
        tw[0, 3] += dx
        cams.append(BasicPinholeCamera.from_params(scene.fx * 0.4, scene.fy * 0.4, 96.0, 80.0, 192, 160, tw))
    bundle = CameraBundle.from_pinhole_cams(cams)
    op = GaussianSplatOp(op_config(scene, 4))
    with torch.no_grad():
        target = rasterize_gaussians(torch_model(scene), bundle, op, training=True).color.permute(0, 3, 1, 2).clamp(0, 1).contiguous()

    model = torch_model(scene)
    g = torch.Generator(device="cuda").manual_seed(3)
    with torch.no_grad():
        model.xyz += 0.02 * torch.randn(model.xyz.shape, generator=g, device="cuda")
        model.opacity -= 1.0
        model.color_sh *= 0.5
    # steps over two views: the trainer halves the schedules (train.py:46-52) and gives every parameter group its own
    # optimizer with the rates, eps and betas of such steps (tools.py:146-173)
    cfg = config_def.Train(batch_size=2)
    cfg.strategy.refine_start_iter, cfg.strategy.refine_every, cfg.strategy.refine_stop_iter = 20, 40, 140
    cfg.strategy.reset_opacity_every = 100
    cfg.strategy.grow_grad2d = 2e-5
    trainer = Trainer(model, op, cfg, scene_scale=2.0)
    n0, losses, events = len(model), [], []
    for step in range(80):
        res = trainer.train_step(bundle, target, generator=g)
        losses.append(res.loss)
        if res.refined:
            events.append(("refine", step, len(model)))
        if res.reset_opacity:
            events.append(("reset", step, len(model)))
    print("loss first %.4f last %.4f  n %d -> %d  events %s" % (losses[0], losses[-1], n0, len(model), events), flush=True)
    assert np.isfinite(losses).all()
    assert [e[0] for e in events] == ["refine", "refine", "reset", "refine"]          # steps 20, 40, 50, 60
    assert len(model) != n0 and trainer.state.count.shape[0] == len(model)
    assert min(losses[40:49]) < 0.8 * losses[0]                                       # before the opacity reset
    assert cfg.strategy.refine_every == 20 and cfg.strategy.reset_opacity_every == 50 and isinstance(trainer.optim, dict)
    for name, optim in trainer.optim.items():
        (group,) = optim.param_groups
        assert group["name"] == name and group["params"][0] is getattr(model, name)
        assert group["betas"] == pytest.approx((0.8, 0.998))
