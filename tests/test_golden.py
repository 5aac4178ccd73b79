"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py):
the oracle must still reproduce them bit for bit, and so must the HIP path."""
import hashlib
import os

import numpy as np
import pytest

from helpers import gen_scene, grad_close, op_config, oracle_forward, torch_model

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = [(0, "none"), (1, "aabb"), (3, "obb")]


def _sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


@pytest.mark.parametrize("filt,tag", CASES)
def test_oracle_reproduces_fixture(oracle, filt, tag):
    gold = np.load(os.path.join(GOLD, f"config0_{tag}.npz"))
    scene = gen_scene(0)
    assert str(gold["scene_sha256"]) == _sha(scene.xyz) + _sha(scene.color_sh), "scene generator drifted"
    P, ref = oracle_forward(oracle, scene, filt)
    assert ref["num_rendered"] == int(gold["num_rendered"])
    for k in ("radii", "tiles_touched", "workload_ranges", "gaussian_idx_sorted"):
        assert np.array_equal(ref[k], gold[k]), k
    assert _sha(ref["keys_sorted"]) == str(gold["keys_sorted_sha256"])
    assert np.array_equal(ref["n_contrib"], gold["n_contrib"])
    assert np.array_equal(ref["color"].view(np.uint32), gold["color"].view(np.uint32))
    assert np.array_equal(ref["T"].view(np.uint32), gold["T"].view(np.uint32))
    g, pb = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                            scene.drgb[0], scene.dT[0])
    for k in ("dxyz", "dscale", "dquat", "dopacity"):
        np.testing.assert_allclose(pb[k], gold[k], rtol=1e-5, atol=1e-6 * np.abs(gold[k]).max())


@pytest.mark.gpu
@pytest.mark.parametrize("filt,tag", CASES)
def test_hip_path_reproduces_fixture(filt, tag):
    import torch
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    gold = np.load(os.path.join(GOLD, f"config0_{tag}.npz"))
    scene = gen_scene(0)
    op = GaussianSplatOp(op_config(scene, filt))
    model = torch_model(scene)
    out, ctx = op.forward(model, scene.camera(), training=True)
    cpu = lambda t: t.detach().cpu().numpy()
    assert op.last_num_rendered == int(gold["num_rendered"])
    assert np.array_equal(cpu(ctx.radii), gold["radii"])
    assert np.array_equal(cpu(ctx.workload_ranges), gold["workload_ranges"])
    assert np.array_equal(cpu(ctx.gaussian_idx_sorted), gold["gaussian_idx_sorted"])
    assert _sha(cpu(op._last_keys_sorted).view(np.uint64)) == str(gold["keys_sorted_sha256"])
    assert np.array_equal(cpu(out.n_contrib)[0], gold["n_contrib"])
    assert np.abs(cpu(out.color)[0] - gold["color"]).max() <= 1e-5
    assert np.abs(cpu(out.T)[0] - gold["T"]).max() <= 1e-5
    grads = GaussianSplatGradients(drgb=torch.from_numpy(scene.drgb).cuda(), dT=torch.from_numpy(scene.dT).cuda())
    gm, duv, _ = op.backward(model, scene.camera(), ctx, out, grads, return_uv_grad=True)
    for k, t in (("dxyz", gm.xyz), ("dscale", gm.scale), ("dquat", gm.quaternion_xyzw), ("dopacity", gm.opacity)):
        a, b = cpu(t).astype(np.float64), gold[k].astype(np.float64)
        assert np.linalg.norm(a - b) <= 1e-4 * np.linalg.norm(b), k
    ok, worst, nbad = grad_close(cpu(duv)[0], gold["duv"])
    assert ok, f"duv: {nbad} bad, worst {worst:.2f}x"
