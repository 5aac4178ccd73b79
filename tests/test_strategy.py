"""Densification strategy, optimizer-state surgery and the photometric loss, on the CPU
(origin/strategy.py:19-364, strategy.py:86-202, train.py:299-354, losses.py:26-73): each rule is
checked on a handful of hand-made gaussians whose fate is known."""
import math

import numpy as np
import pytest
import torch
from scipy.spatial.transform import Rotation

from d3gs_research_amd import config_def
from d3gs_research_amd.model import GaussianModelOrigin, GaussianModelOriginFused
from d3gs_research_amd.render import GaussianSplatOutput
from d3gs_research_amd.strategy import GaussianStrategyOrigin, GaussianTrainState, quat_xyzw_to_rotmat
from d3gs_research_amd.tools import create_origin_3dgs_optimizer
from d3gs_research_amd.train import ssim


def test_rotation_matrix_convention():
    q = np.random.default_rng(0).standard_normal((16, 4))
    q /= np.linalg.norm(q, axis=1, keepdims=True)
    got = quat_xyzw_to_rotmat(torch.from_numpy(q)).numpy()
    assert np.allclose(got, Rotation.from_quat(q).as_matrix(), atol=1e-12)     # scipy: scalar-last


def test_update_accumulates_ndc_gradient_length():
    st = GaussianStrategyOrigin(refine_scale2d_stop_iter=10)
    state = GaussianTrainState.create(3)
    W, H, B = 200, 100, 2
    out = GaussianSplatOutput(custom_features=None, T=torch.zeros(B, H, W), color=torch.zeros(B, H, W, 3),
                              radii=torch.tensor([5, 0, 7, 0, 0, 20], dtype=torch.int32))
    duv = torch.tensor([[[3e-3, 4e-3], [1.0, 1.0], [0.0, 1e-3]], [[9.0, 9.0], [2.0, 2.0], [6e-3, 8e-3]]])
    st.update(state, out, duv)
    # visible: camera 0 sees gaussians 0 and 2, camera 1 sees gaussian 2; scale (0.5 W B, 0.5 H B) = (200, 100)
    want0 = math.hypot(3e-3 * 200, 4e-3 * 100)
    want2 = 1e-3 * 100 + math.hypot(6e-3 * 200, 8e-3 * 100)
    assert state.duv_ndc_length.tolist() == pytest.approx([want0, 0.0, want2])
    assert state.count.tolist() == [1.0, 0.0, 2.0]
    assert state.max_radii.tolist() == pytest.approx([5 / 200, 0.0, 20 / 200])


def test_the_two_other_update_forms():
    """origin/strategy.py:45-73 (no batch factor, per view and gaussian) and 125-157 (one state row per row of duv)."""
    W, H = 200, 100
    radii = torch.tensor([5, 0, 7, 0, 0, 20], dtype=torch.int32)
    duv = torch.tensor([[[3e-3, 4e-3], [1.0, 1.0], [0.0, 1e-3]], [[9.0, 9.0], [2.0, 2.0], [6e-3, 8e-3]]])
    out = GaussianSplatOutput(custom_features=None, T=torch.zeros(2, H, W), color=torch.zeros(2, H, W, 3), radii=radii)
    st = GaussianStrategyOrigin(refine_scale2d_stop_iter=10)
    state = GaussianTrainState.create(3)
    st.update_v1(state, out, duv)       # scale (W / 2, H / 2) = (100, 50)
    assert state.duv_ndc_length.tolist() == pytest.approx([math.hypot(0.3, 0.2), 0.0, 0.05 + math.hypot(0.6, 0.4)])
    assert state.count.tolist() == [1.0, 0.0, 2.0]
    assert state.max_radii.tolist() == pytest.approx([5 / 200, 0.0, 20 / 200])
    flat = GaussianTrainState.create(6)
    st.update_v2(flat, out, duv, batch_size=2)       # scale (0.5 W B, 0.5 H B) = (200, 100), one row per (view, gaussian)
    assert flat.duv_ndc_length.tolist() == pytest.approx([math.hypot(0.6, 0.4), 0.0, 0.1, 0.0, 0.0, math.hypot(1.2, 0.8)])
    assert flat.count.tolist() == [1.0, 0.0, 1.0, 0.0, 0.0, 1.0]
    assert flat.max_radii.tolist() == pytest.approx([5 / 200, 0.0, 7 / 200, 0.0, 0.0, 20 / 200])


def _toy(fused=True):
    # 0: high gradient, small  -> cloned        1: high gradient, large -> split (parent removed)
    # 2: transparent           -> pruned        3: quiet               -> kept
    # 4: high gradient, small and transparent -> clone and original both pruned
    scale = torch.log(torch.tensor([[0.004, 0.002, 0.001], [0.05, 0.02, 0.01], [0.004, 0.004, 0.004],
                                    [0.2, 0.2, 0.2], [0.001, 0.001, 0.001]]))
    opacity = torch.logit(torch.tensor([0.5, 0.6, 0.001, 0.7, 0.002]))
    g = torch.Generator().manual_seed(0)
    cls = GaussianModelOriginFused if fused else GaussianModelOrigin
    m = cls(xyz=torch.randn(5, 3, generator=g), quaternion_xyzw=torch.randn(5, 4, generator=g), scale=scale,
            opacity=opacity, color_sh=torch.randn(5, 15, 3, generator=g), color_sh_base=torch.randn(5, 3, generator=g),
            cur_sh_degree=3)
    m.set_requires_grad(True)
    state = GaussianTrainState.create(5, scene_scale=1.0)
    state.duv_ndc_length[:] = torch.tensor([0.01, 0.01, 0.0, 0.00001, 0.01])
    state.count[:] = torch.tensor([10.0, 20.0, 0.0, 1.0, 2.0])
    return m, state


@pytest.mark.parametrize("fused", [True, False])
def test_refine_clone_split_prune_and_optimizer_state(fused):
    m, state = _toy(fused)
    optim, _ = create_origin_3dgs_optimizer(m, config_def.Optimizer(), 1.0)
    (m.xyz.sum() + m.scale.sum() + m.opacity.sum() + m.quaternion_xyzw.sum() + m.color_sh.sum() + m.color_sh_base.sum()).backward()
    optim.step()
    old = {k: v.detach().clone() for k, v in m.get_proxy_field_dict().items()}
    old_avg = {g["name"]: optim.state[g["params"][0]]["exp_avg"].clone() for g in optim.param_groups}
    st = GaussianStrategyOrigin()
    st.refine_gs(m, optim, state, step=600, generator=torch.Generator().manual_seed(5))
    # kept originals 0, 3; clone of 0; two children of 1 (the clone of 4 is pruned with it)
    assert len(m) == 5
    assert torch.equal(m.opacity.detach(), old["opacity"][[0, 3, 0, 1, 1]])
    assert torch.equal(m.color_sh.detach(), old["color_sh"][[0, 3, 0, 1, 1]])
    assert torch.equal(m.xyz.detach()[:3], old["xyz"][[0, 3, 0]])
    normals = torch.randn(2, 3, generator=torch.Generator().manual_seed(5))
    s1 = torch.exp(old["scale"][1])
    q1 = old["quaternion_xyzw"][1] / old["quaternion_xyzw"][1].norm()
    R = torch.from_numpy(Rotation.from_quat(q1.numpy()).as_matrix()).float()
    for c in range(2):
        assert torch.allclose(m.xyz.detach()[3 + c], R @ (normals[c] * s1) + old["xyz"][1], atol=1e-6)
        assert torch.allclose(torch.exp(m.scale.detach()[3 + c]), s1 / 1.6, rtol=1e-6)
    assert all(t.requires_grad and t.is_leaf for t in m.get_proxy_field_dict().values())
    assert state.count.shape == (5,) and not state.count.any() and not state.duv_ndc_length.any()
    for g in optim.param_groups:
        p = g["params"][0]
        assert p is getattr(m, g["name"])
        avg = optim.state[p]["exp_avg"]
        assert torch.equal(avg[:2], old_avg[g["name"]][[0, 3]]) and not avg[2:].any()
    # the optimizer keeps working on the new tensors
    m.xyz.sum().backward()
    optim.step()


def test_prune_oversized_only_after_the_first_opacity_reset():
    for step, want in ((600, 5), (3100, 4)):
        m, state = _toy()
        optim, _ = create_origin_3dgs_optimizer(m, config_def.Optimizer(), 1.0)
        GaussianStrategyOrigin().refine_gs(m, optim, state, step=step, generator=torch.Generator().manual_seed(1))
        assert len(m) == want        # gaussian 3 (scale 0.2 > prune_scale3d * scene_scale = 0.1) goes at step > 3000


@pytest.mark.parametrize("fused", [True, False])
def test_reset_opacity(fused):
    m, state = _toy(fused)
    optim, _ = create_origin_3dgs_optimizer(m, config_def.Optimizer(), 1.0)
    m.opacity.sum().backward()
    optim.step()
    before = torch.sigmoid(m.opacity.detach())
    GaussianStrategyOrigin().reset_opacity(m, optim)
    assert torch.allclose(torch.sigmoid(m.opacity.detach()), torch.clamp_max(before, 0.01), rtol=1e-5)
    group = [g for g in optim.param_groups if g["name"] == "opacity"][0]
    assert group["params"][0] is m.opacity and not optim.state[m.opacity]["exp_avg"].any()


def test_ssim_against_the_direct_definition():
    rng = np.random.default_rng(3)
    a = rng.random((1, 2, 9, 13))
    b = np.clip(a + 0.1 * rng.standard_normal(a.shape), 0, 1)
    x = np.arange(11) - 5
    w1 = np.exp(-x * x / (2 * 1.5 ** 2))
    w1 /= w1.sum()
    w2 = np.outer(w1, w1)

    def blur(img):
        p = np.pad(img, ((0, 0), (0, 0), (5, 5), (5, 5)))
        out = np.zeros_like(img)
        for i in range(img.shape[2]):
            for j in range(img.shape[3]):
                out[:, :, i, j] = (p[:, :, i:i + 11, j:j + 11] * w2).sum((2, 3))
        return out
    mu1, mu2 = blur(a), blur(b)
    s1, s2, s12 = blur(a * a) - mu1 ** 2, blur(b * b) - mu2 ** 2, blur(a * b) - mu1 * mu2
    want = (((2 * mu1 * mu2 + 1e-4) * (2 * s12 + 9e-4)) / ((mu1 ** 2 + mu2 ** 2 + 1e-4) * (s1 + s2 + 9e-4))).mean()
    got = float(ssim(torch.from_numpy(a), torch.from_numpy(b)))
    assert got == pytest.approx(want, rel=1e-10)
    assert float(ssim(torch.from_numpy(a), torch.from_numpy(a))) == pytest.approx(1.0)
