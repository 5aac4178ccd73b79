"""Pins the oracle's backward (blend backward K7 + preprocess backward K9) against
float64 torch autograd over an independent dense restatement of the forward,
and against central finite differences.  Reference semantics that the autograd
model has to share: the alpha clamp min(0.99, .) passes gradient straight
through (render.py:1769, 1995), the frustum clamp limit is not differentiated
(gs3d.py:493-494, 524-529), and the conic uses 1 / (det + eps)."""
import numpy as np
import pytest
import torch

from f64_reference import C0, C1, C2, C3
from helpers import oracle_params, gen_scene, oracle_forward

torch.set_num_threads(4)


def _sh_torch(deg, sh, d):
    x, y, z = d[:, 0:1], d[:, 1:2], d[:, 2:3]
    r = C0 * sh[:, 0]
    if deg > 0:
        r = r - C1 * y * sh[:, 1] + C1 * z * sh[:, 2] - C1 * x * sh[:, 3]
    if deg > 1:
        xx, yy, zz, xy, yz, xz = x * x, y * y, z * z, x * y, y * z, x * z
        r = (r + C2[0] * xy * sh[:, 4] + C2[1] * yz * sh[:, 5] + C2[2] * (2 * zz - xx - yy) * sh[:, 6]
             + C2[3] * xz * sh[:, 7] + C2[4] * (xx - yy) * sh[:, 8])
    if deg > 2:
        r = (r + C3[0] * y * (3 * xx - yy) * sh[:, 9] + C3[1] * xy * z * sh[:, 10]
             + C3[2] * y * (4 * zz - xx - yy) * sh[:, 11] + C3[3] * z * (2 * zz - 3 * xx - 3 * yy) * sh[:, 12]
             + C3[4] * x * (4 * zz - xx - yy) * sh[:, 13] + C3[5] * z * (xx - yy) * sh[:, 14]
             + C3[6] * x * (xx - 3 * yy) * sh[:, 15])
    return r + 0.5


def _quat_to_R(q):
    x, y, z, w = q[:, 0], q[:, 1], q[:, 2], q[:, 3]
    return torch.stack([
        torch.stack([1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y)], -1),
        torch.stack([2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x)], -1),
        torch.stack([2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], -1)], -2)


def _render_f64(scene, params, member, order, anti_aliasing=False, feat=None, inv_depth=False):
    """Dense float64 forward: `member[p, j]` says gaussian order[j] is in pixel p's tile list.
    inv_depth: the depth channel blends 1 / z.
    Returns colour, T, blended depth and blended alpha (the sum of the weights), and the blended
    custom features when `feat` [N, F] is given."""
    xyz, quat, scale, opac, sh = params
    tw = torch.tensor(scene.to_world, dtype=torch.float64)
    W, c = tw[:3, :3].T, tw[:3, 3]
    pc = (xyz - c) @ W.T
    z = pc[:, 2]
    fx, fy = scene.fx, scene.fy
    uv = torch.stack([fx * pc[:, 0] / z + scene.cx - 0.5, fy * pc[:, 1] / z + scene.cy - 0.5], -1)
    q = quat / quat.norm(dim=1, keepdim=True)
    M = _quat_to_R(q) * torch.exp(scale)[:, None, :]
    S3 = M @ M.transpose(1, 2)
    lx = (0.5 * scene.width / fx * 1.3 * z).abs().detach()
    ly = (0.5 * scene.height / fy * 1.3 * z).abs().detach()
    tx = torch.maximum(torch.minimum(pc[:, 0], lx), -lx)
    ty = torch.maximum(torch.minimum(pc[:, 1], ly), -ly)
    zero = torch.zeros_like(z)
    J = torch.stack([torch.stack([fx / z, zero, -fx * tx / z ** 2], -1),
                     torch.stack([zero, fy / z, -fy * ty / z ** 2], -1)], -2)
    T = J @ W
    S2 = T @ S3 @ T.transpose(1, 2)
    a, b, cc = S2[:, 0, 0] + 0.3, S2[:, 0, 1], S2[:, 1, 1] + 0.3
    det = a * cc - b * b
    o = torch.sigmoid(opac)
    if anti_aliasing:
        # mip-splatting style compensation: exact inverse of the low-passed covariance, opacity scaled by
        # sqrt(det(cov) / det(cov + 0.3 I)) (clamped below at 0.000025)
        ca, cb, ccn = cc / det, -b / det, a / det
        ratio = ((a - 0.3) * (cc - 0.3) - b * b) / det
        o = o * torch.sqrt(torch.clamp_min(ratio, 0.000025))
    else:
        ca, cb, ccn = cc / (det + 1e-6), -b / (det + 1e-6), a / (det + 1e-6)
    d = xyz - c
    rgb = torch.clamp_min(_sh_torch(scene.sh_degree, sh, d / d.norm(dim=1, keepdim=True)), 0.0)

    H, Wd = scene.height, scene.width
    ys, xs = torch.meshgrid(torch.arange(H, dtype=torch.float64), torch.arange(Wd, dtype=torch.float64), indexing="ij")
    px, py = xs.reshape(-1), ys.reshape(-1)
    Tcur = torch.ones(H * Wd, dtype=torch.float64)
    col = torch.zeros(H * Wd, 3, dtype=torch.float64)
    dep = torch.zeros(H * Wd, dtype=torch.float64)
    asum = torch.zeros(H * Wd, dtype=torch.float64)
    done = torch.zeros(H * Wd, dtype=torch.bool)
    fimg = None if feat is None else torch.zeros(H * Wd, feat.shape[1], dtype=torch.float64)
    for j, g in enumerate(order):
        dx, dy = uv[g, 0] - px, uv[g, 1] - py
        power = -0.5 * (ca[g] * dx * dx + ccn[g] * dy * dy) - cb[g] * dx * dy
        raw = o[g] * torch.exp(power)
        alpha = raw + (torch.clamp_max(raw, 0.99) - raw).detach()        # straight-through clamp
        live = member[:, j] & ~done & (alpha.detach() >= 1 / 255.0)
        nT = Tcur * (1 - alpha)
        stop = live & (nT.detach() < 1e-4)
        done = done | stop
        use = live & ~stop & (power.detach() <= 0)
        w = torch.where(use, alpha * Tcur, torch.zeros_like(Tcur))
        col = col + w[:, None] * rgb[g]
        dep = dep + (w / z[g] if inv_depth else w * z[g])
        asum = asum + w
        if feat is not None:
            fimg = fimg + w[:, None] * feat[g]
        Tcur = torch.where(use, nT, Tcur)
    if feat is not None:
        return col.reshape(H, Wd, 3), Tcur.reshape(H, Wd), dep.reshape(H, Wd), asum.reshape(H, Wd), \
            fimg.reshape(H, Wd, -1)
    return col.reshape(H, Wd, 3), Tcur.reshape(H, Wd), dep.reshape(H, Wd), asum.reshape(H, Wd)


def _setup(seed_cfg=0, n=96, wh=(48, 32), filt=0, sh_cfg=None):
    scene = gen_scene(seed_cfg, n=n, wh=wh)
    if sh_cfg is not None:               # degree-3 colours on the tiny geometry
        donor = gen_scene(1, n=n, wh=(64, 64))
        scene.color_sh, scene.sh_degree = donor.color_sh, 3
    # concentrate the gaussians on the small image and make them larger
    scene.xyz[:, :2] *= 0.25
    scene.scale += 1.0
    return scene


def _f64_grads(scene, ref, drgb, dT, ddepth=None, anti_aliasing=False, feat=None, feat_image=None, dfeat=None,
               far_to_near=False):
    """Float64 autograd gradients of sum(color*drgb) + sum(T*dT) (+ sum(depth*ddepth))
    (+ sum(features*dfeat)) w.r.t. the raw model tensors (and the custom features, last in the list).
    A four-channel drgb also weights the blended alpha."""
    # global depth order (stable) and per-pixel tile-list membership from the oracle's binning
    valid = np.flatnonzero(ref["radii"] > 0)
    order = valid[np.argsort(ref["depths"][valid].view(np.uint32), kind="stable")]
    if far_to_near:
        # render_inv_depth: the order is not taken from the oracle's depth buffer but from the camera-space z
        # itself, descending (what sorting by 1 / z amounts to), and the depth channel blends 1 / z
        tw = np.asarray(scene.to_world, np.float64)
        z = (scene.xyz[valid].astype(np.float64) - tw[:3, 3]) @ tw[:3, 2]
        order = valid[np.argsort(-z, kind="stable")]
    pos = {g: j for j, g in enumerate(order.tolist())}
    tiles_x = (scene.width + 15) // 16
    member = np.zeros((scene.height * scene.width, len(order)), bool)
    pix_tile = (np.arange(scene.height)[:, None] // 16) * tiles_x + np.arange(scene.width)[None, :] // 16
    for t, (r0, r1) in enumerate(ref["workload_ranges"]):
        cols = [pos[g] for g in ref["gaussian_idx_sorted"][r0:r1].tolist()]
        member[np.ix_(np.flatnonzero(pix_tile.reshape(-1) == t), cols)] = True

    params = [torch.tensor(a, dtype=torch.float64, requires_grad=True)
              for a in (scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)]
    fimg = None
    if feat is not None:
        params.append(torch.tensor(feat, dtype=torch.float64, requires_grad=True))
        col, Tfin, dep, asum, fimg = _render_f64(scene, params[:5], torch.from_numpy(member), order.tolist(),
                                                 anti_aliasing, params[5])
    else:
        col, Tfin, dep, asum = _render_f64(scene, params, torch.from_numpy(member), order.tolist(), anti_aliasing,
                                           inv_depth=far_to_near)
    # the float64 forward agrees with the oracle's float32 forward (no threshold flips on this scene)
    assert np.abs(col.detach().numpy() - ref["color"][..., :3]).max() <= 2e-5
    assert np.abs(Tfin.detach().numpy() - ref["T"]).max() <= 1e-5
    d64 = torch.from_numpy(drgb).double()
    loss = (col * d64[..., :3]).sum() + (Tfin * torch.from_numpy(dT).double()).sum()
    if drgb.shape[-1] == 4:
        assert np.abs(asum.detach().numpy() - ref["color"][..., 3]).max() <= 2e-5
        loss = loss + (asum * d64[..., 3]).sum()
    if ddepth is not None:
        assert np.abs(dep.detach().numpy() - ref["depth"]).max() <= 1e-4
        loss = loss + (dep * torch.from_numpy(ddepth).double()).sum()
    if fimg is not None:
        assert np.abs(fimg.detach().numpy() - feat_image).max() <= 2e-5 * max(1.0, np.abs(feat).max())
        loss = loss + (fimg * torch.from_numpy(dfeat).double()).sum()
    loss.backward()
    return [p.grad for p in params]


def _close(got, want, name):
    want = want.numpy()
    scale = np.abs(want).max()
    err = np.abs(np.asarray(got, np.float64) - want).max()
    assert err <= 2e-4 * scale + 1e-9, f"{name}: max err {err:.3e} vs scale {scale:.3e}"


@pytest.mark.parametrize("sh3", [False, True])
def test_backward_matches_float64_autograd(oracle, sh3):
    scene = _setup(sh_cfg=1 if sh3 else None)
    P, ref = oracle_forward(oracle, scene, 0)
    rng = np.random.default_rng(11)
    drgb = rng.standard_normal((scene.height, scene.width, 3)).astype(np.float32)
    dT = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    g_ref, pb = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                                drgb, dT)

    grads = _f64_grads(scene, ref, drgb, dT)

    _close(pb["dxyz"], grads[0], "dxyz")
    _close(pb["dquat"], grads[1], "dquat")
    _close(pb["dscale"], grads[2], "dscale")
    _close(pb["dopacity"], grads[3], "dopacity")
    _close(pb["dsh"], grads[4], "dsh")


def test_blend_backward_finite_differences(oracle):
    """Central differences in float64 of the dense forward w.r.t. the blend inputs (uv, conic, opacity,
    colour) on a handful of gaussians, against orc_blend_bwd's analytic gradients."""
    scene = _setup(n=48, wh=(32, 32))
    P, ref = oracle_forward(oracle, scene, 0)
    rng = np.random.default_rng(2)
    drgb = rng.standard_normal((scene.height, scene.width, 3)).astype(np.float32)
    dT = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    g = oracle.blend_bwd(P, ref["workload_ranges"], ref["gaussian_idx_sorted"], ref["uvs"], ref["conic_opacity"],
                         ref["rgb_gaussian"], ref["T"], ref["n_contrib"], ref["color"], drgb, dT)
    from f64_reference import blend_pixel_f64
    tiles_x = (scene.width + 15) // 16

    def loss(uvs, co, rgb):
        tot = 0.0
        for py in range(scene.height):
            for px in range(scene.width):
                t = (py // 16) * tiles_x + px // 16
                r0, r1 = ref["workload_ranges"][t]
                c, T, _, _ = blend_pixel_f64(px, py, ref["gaussian_idx_sorted"][r0:r1], uvs, co, rgb)
                tot += float((c * drgb[py, px]).sum() + T * dT[py, px])
        return tot

    uvs, co, rgb = (ref[k].astype(np.float64) for k in ("uvs", "conic_opacity", "rgb_gaussian"))
    picks = np.flatnonzero(np.abs(g["dopacity"]) > 1e-3)[:4]
    assert len(picks) >= 3
    h = 1e-5
    for gi in picks:
        for arr, idx, want in ((uvs, 0, g["duv"][gi, 0]), (uvs, 1, g["duv"][gi, 1]), (co, 0, g["dconic"][gi, 0]),
                               (co, 1, g["dconic"][gi, 1]), (co, 2, g["dconic"][gi, 2]), (co, 3, g["dopacity"][gi]),
                               (rgb, 1, g["dcolor"][gi, 1])):
            old = arr[gi, idx]
            arr[gi, idx] = old + h
            lp = loss(uvs, co, rgb)
            arr[gi, idx] = old - h
            lm = loss(uvs, co, rgb)
            arr[gi, idx] = old
            fd = (lp - lm) / (2 * h)
            assert abs(fd - want) <= 2e-3 * max(abs(want), abs(fd)) + 1e-4, (gi, idx, fd, want)


def test_sh_mask_bit_order_switch(oracle):
    """The reference writes the clamp mask r->bit2,g->bit1,b->bit0 (render.py:608) and reads it back reversed
    (render.py:3344-3350).  Default = consistent mapping; the compat switch reproduces the reversed read."""
    scene = _setup(sh_cfg=1)
    scene.color_sh[:, 0, 0] = -3.0       # red always clamped, green/blue never
    scene.color_sh[:, 0, 1:] = 1.0
    P, ref = oracle_forward(oracle, scene, 0)
    assert (ref["sh_to_rgb_ne_0"][ref["radii"] > 0] == 4).all()
    drgb = np.ones((scene.height, scene.width, 3), np.float32)
    dT = np.zeros((scene.height, scene.width), np.float32)
    _, ok = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh, drgb, dT)
    _, compat = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                                drgb, dT, sh_mask_compat=True)
    assert not ok["dsh"][:, 0, 0].any() and ok["dsh"][:, 0, 2].any()           # red masked, blue flows
    assert compat["dsh"][:, 0, 0].any() and not compat["dsh"][:, 0, 2].any()   # reversed: blue masked instead


def test_activated_inputs_chain_to_the_raw_gradients(oracle):
    """fused_activation = 0 (GaussianModelOrigin, origin/model.py:249-270): the oracle takes activated
    scale / quaternion / opacity and returns gradients w.r.t. them.  Pushed through the float64
    Jacobians of exp / normalize / sigmoid they must equal the float64 autograd gradients of the raw
    tensors, and the image must be the fused path's image."""
    scene = _setup()
    P, ref = oracle_forward(oracle, scene, 0)
    q64 = torch.tensor(scene.quaternion_xyzw, dtype=torch.float64, requires_grad=True)
    s64 = torch.tensor(scene.scale, dtype=torch.float64, requires_grad=True)
    o64 = torch.tensor(scene.opacity, dtype=torch.float64, requires_grad=True)
    q_act, s_act, o_act = q64 / q64.norm(dim=1, keepdim=True), torch.exp(s64), torch.sigmoid(o64)
    act = [t.detach().numpy().astype(np.float32) for t in (q_act, s_act, o_act)]

    P0 = oracle_params(oracle, scene, 0)
    P0.fused_activation = 0
    ref0 = oracle.forward(P0, scene.xyz, act[0], act[1], act[2], scene.color_sh)
    assert np.abs(ref0["color"] - ref["color"]).max() <= 1e-5
    assert np.abs(ref0["T"] - ref["T"]).max() <= 1e-5

    rng = np.random.default_rng(11)
    drgb = rng.standard_normal((scene.height, scene.width, 3)).astype(np.float32)
    dT = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    _, pb = oracle.backward(P0, ref0, scene.xyz, act[0], act[1], act[2], scene.color_sh, drgb, dT)
    torch.autograd.backward([q_act, s_act, o_act],
                            [torch.from_numpy(pb[k]).double() for k in ("dquat", "dscale", "dopacity")])
    grads = _f64_grads(scene, ref, drgb, dT)
    _close(pb["dxyz"], grads[0], "dxyz")
    _close(q64.grad.numpy(), grads[1], "dquat")
    _close(s64.grad.numpy(), grads[2], "dscale")
    _close(o64.grad.numpy(), grads[3], "dopacity")
    _close(pb["dsh"], grads[4], "dsh")


@pytest.mark.parametrize("aa,depth,rgba", [(True, False, False), (False, True, False), (False, False, True),
                                           (True, True, True)])
def test_channels_and_anti_aliasing_match_float64_autograd(oracle, aa, depth, rgba):
    """render_depth (render.py:1915-1919, 1948-1950, 1964-1967 and dz into the pinhole backward,
    render.py:3283-3292), render_rgba (1899-1906, 1926-1931) and enable_anti_aliasing (391-407,
    3293-3306; gs3d.py:592-679) against float64 autograd over the dense restatement."""
    scene = _setup()
    P = oracle_params(oracle, scene, 0)
    P.enable_anti_aliasing, P.render_depth, P.render_rgba = int(aa), int(depth), int(rgba)
    ref = oracle.forward(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    rng = np.random.default_rng(12)
    drgb = rng.standard_normal((scene.height, scene.width, 4 if rgba else 3)).astype(np.float32)
    dT = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    ddepth = rng.standard_normal((scene.height, scene.width)).astype(np.float32) if depth else None
    g, pb = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                            drgb, dT, ddepth=ddepth)
    assert (g["dz"] is not None) == depth
    grads = _f64_grads(scene, ref, drgb, dT, ddepth, aa)
    for i, name in enumerate(["dxyz", "dquat", "dscale", "dopacity", "dsh"]):
        _close(pb[name], grads[i], name)


def test_inverse_depth_matches_float64_autograd_over_far_to_near_lists(oracle):
    """render_inv_depth (config_def.py:95; render.py:582, 773, 1965, 3051, 3283): K1 stores 1 / z, the sort key takes
    its depth part from that buffer, so every list runs from the far end to the near one; the depth channel blends
    1 / z and K9 turns dL/d(1/z) into -dz / z^2.  Pinned by the dense float64 restatement run over the gaussians
    in descending camera-space z (computed here from the scene, not from the oracle's buffers) with 1 / z as the
    depth channel: image, T, depth image and every model gradient; and the plain render of the same scene is a
    different image (the order matters)."""
    scene = _setup()
    P = oracle_params(oracle, scene, 0)
    P.render_depth, P.render_inv_depth = 1, 1
    ref = oracle.forward(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    P0 = oracle_params(oracle, scene, 0)
    P0.render_depth = 1
    ref0 = oracle.forward(P0, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    seen = ref0["radii"] > 0
    assert np.array_equal(ref["radii"], ref0["radii"]) and np.array_equal(ref["tiles_touched"], ref0["tiles_touched"])
    assert np.array_equal(ref["depths"][seen], (np.float32(1.0) / ref0["depths"][seen]).astype(np.float32))
    assert np.abs(ref["color"] - ref0["color"]).max() > 1e-2
    # inside every tile list the camera depth never grows
    z0 = ref0["depths"]
    for r0, r1 in ref["workload_ranges"]:
        zs = z0[ref["gaussian_idx_sorted"][r0:r1]]
        assert np.all(zs[1:] <= zs[:-1])
    rng = np.random.default_rng(14)
    drgb = rng.standard_normal((scene.height, scene.width, 3)).astype(np.float32)
    dT = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    ddepth = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    g, pb = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                            drgb, dT, ddepth=ddepth)
    grads = _f64_grads(scene, ref, drgb, dT, ddepth, far_to_near=True)
    for i, name in enumerate(["dxyz", "dquat", "dscale", "dopacity", "dsh"]):
        _close(pb[name], grads[i], name)
    # the depth gradient alone (nothing but ddepth): what -dz / z^2 carries into dxyz
    zeros3, zeros1 = np.zeros_like(drgb), np.zeros_like(dT)
    _, pb_d = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                              zeros3, zeros1, ddepth=ddepth)
    grads_d = _f64_grads(scene, ref, zeros3, zeros1, ddepth, far_to_near=True)
    _close(pb_d["dxyz"], grads_d[0], "dxyz from the depth channel alone")


@pytest.mark.parametrize("F,depth", [(2, False), (3, False), (7, True)])
def test_custom_features_match_float64_autograd(oracle, F, depth):
    """Custom feature channels (render.py:1571-1573, 1892-1895, 1920-1923, 1952-1955, 1969-1972):
    the blended feature image, its share of the geometry gradients and dcustom_features against
    float64 autograd over the dense restatement.  F = 2 and 7 cover a partly filled last triple."""
    scene = _setup()
    P = oracle_params(oracle, scene, 0)
    P.render_depth = int(depth)
    ref = oracle.forward(P, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh)
    rng = np.random.default_rng(13)
    feat = rng.standard_normal((scene.n, F)).astype(np.float32)
    fimg = oracle.blend_custom_features(P, ref, feat)
    assert fimg.shape == (scene.height, scene.width, F)
    # a constant feature blends to the sum of the weights, 1 - T
    ones = oracle.blend_custom_features(P, ref, np.ones((scene.n, 1), np.float32))
    assert np.abs(ones[..., 0] + ref["T"] - 1.0).max() <= 1e-5
    drgb = rng.standard_normal((scene.height, scene.width, 3)).astype(np.float32)
    dT = rng.standard_normal((scene.height, scene.width)).astype(np.float32)
    ddepth = rng.standard_normal((scene.height, scene.width)).astype(np.float32) if depth else None
    dfeat = rng.standard_normal(fimg.shape).astype(np.float32)
    g, pb = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                            drgb, dT, ddepth=ddepth, custom_features=feat, custom_feature_image=fimg,
                            dcustom_features=dfeat)
    grads = _f64_grads(scene, ref, drgb, dT, ddepth, False, feat, fimg, dfeat)
    for i, name in enumerate(["dxyz", "dquat", "dscale", "dopacity", "dsh"]):
        _close(pb[name], grads[i], name)
    _close(g["dcustom_features"], grads[5], "dcustom_features")
    # the feature term matters: without it the geometry gradients are far from the autograd ones
    _, pb0 = oracle.backward(P, ref, scene.xyz, scene.quaternion_xyzw, scene.scale, scene.opacity, scene.color_sh,
                             drgb, dT, ddepth=ddepth)
    assert np.abs(pb0["dxyz"] - grads[0].numpy()).max() > 1e-2 * np.abs(grads[0].numpy()).max()
