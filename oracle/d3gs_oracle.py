"""numpy front end of the CPU oracle (``libd3gs_oracle.so``).

TEST INFRASTRUCTURE ONLY: tests, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module; the product
package never does.  Every function here is a thin ctypes call into
``d3gs_oracle.cpp``, whose header lists the reference lines each stage restates.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libd3gs_oracle.so")

FILTER_NONE, FILTER_AABB, FILTER_ELLIPSE, FILTER_OBB, FILTER_OBB_DFVT = 0, 1, 2, 3, 4


class OracleParams(C.Structure):
    _fields_ = [
        ("n", C.c_int32), ("width", C.c_int32), ("height", C.c_int32),
        ("tiles_x", C.c_int32), ("tiles_y", C.c_int32),
        ("sh_degree", C.c_int32), ("sh_stride", C.c_int32), ("has_sh_base", C.c_int32),
        ("filter_algo", C.c_int32), ("training", C.c_int32),
        ("fx", C.c_float), ("fy", C.c_float), ("cx", C.c_float), ("cy", C.c_float),
        ("tan_fovx", C.c_float), ("tan_fovy", C.c_float),
        ("w2c", C.c_float * 9), ("cam_center", C.c_float * 3),
        ("z_near", C.c_float), ("z_far", C.c_float), ("eps", C.c_float),
        ("radii_eigen_eps", C.c_float), ("clamp_factor", C.c_float), ("std_sigma", C.c_float),
        ("lowpass", C.c_float), ("alpha_eps", C.c_float), ("transmittance_eps", C.c_float),
        ("scale_global", C.c_float), ("bg", C.c_float * 3), ("fused_activation", C.c_int32),
        ("render_depth", C.c_int32), ("render_rgba", C.c_int32), ("use_nchw", C.c_int32),
        ("enable_anti_aliasing", C.c_int32), ("enable_32bit_sort", C.c_int32), ("depth_32bit_prec", C.c_float),
        ("render_inv_depth", C.c_int32),
    ]


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s", "libd3gs_oracle.so"], check=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_expf.restype = C.c_float
        _lib.orc_expf.argtypes = [C.c_float]
        _lib.orc_expf_blend.restype = C.c_float
        _lib.orc_expf_blend.argtypes = [C.c_float]
        _lib.orc_logf.restype = C.c_float
        _lib.orc_logf.argtypes = [C.c_float]
        _lib.orc_scan.restype = C.c_int64
        _lib.orc_higher_msb.restype = C.c_int32
        _lib.orc_higher_msb.argtypes = [C.c_uint32]
        _lib.orc_num_threads.restype = C.c_int32
    return _lib


def _p(a):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def make_params(*, n, width, height, focal_xy, principal_point, cam2world_T, sh_degree, sh_stride,
                has_sh_base=False, filter_algo=FILTER_NONE, training=True, near=0.2, far=10000.0, eps=1e-6,
                radii_eigen_eps=0.1, clamp_factor=1.3, std_sigma=3.0, lowpass=0.3, alpha_eps=1.0 / 255.0,
                transmittance_eps=1e-4, scale_global=1.0, bg=(0.0, 0.0, 0.0), fused_activation=True,
                render_depth=False, render_rgba=False, use_nchw=False, enable_anti_aliasing=False,
                enable_32bit_sort=False, depth_32bit_prec=0.001, render_inv_depth=False) -> OracleParams:
    """cam2world_T is the 4x3 matrix ``to_world[:3].T`` (render.py:205-206)."""
    P = OracleParams()
    P.n, P.width, P.height = int(n), int(width), int(height)
    P.tiles_x, P.tiles_y = (width + 15) // 16, (height + 15) // 16
    P.sh_degree, P.sh_stride, P.has_sh_base = int(sh_degree), int(sh_stride), int(bool(has_sh_base))
    P.filter_algo, P.training = int(filter_algo), int(bool(training))
    f = np.asarray(focal_xy, np.float32)
    pp = np.asarray(principal_point, np.float32)
    P.fx, P.fy, P.cx, P.cy = float(f[0]), float(f[1]), float(pp[0]), float(pp[1])
    # tan_fov = 0.5 * resolution / focal in float32 (render.py:358, 3274)
    tf = np.float32(0.5) * np.array([width, height], np.float32) / f
    P.tan_fovx, P.tan_fovy = float(tf[0]), float(tf[1])
    c2w = np.ascontiguousarray(np.asarray(cam2world_T, np.float32).reshape(4, 3))
    P.w2c[:] = [float(v) for v in c2w[:3].reshape(-1)]
    P.cam_center[:] = [float(v) for v in c2w[3]]
    P.z_near, P.z_far, P.eps = float(near), float(far), float(eps)
    P.radii_eigen_eps, P.clamp_factor, P.std_sigma = float(radii_eigen_eps), float(clamp_factor), float(std_sigma)
    P.lowpass, P.alpha_eps, P.transmittance_eps = float(lowpass), float(alpha_eps), float(transmittance_eps)
    P.scale_global = float(scale_global)
    P.bg[:] = [float(v) for v in bg]
    P.fused_activation = int(bool(fused_activation))
    P.render_depth, P.render_rgba = int(bool(render_depth)), int(bool(render_rgba))
    P.use_nchw, P.enable_anti_aliasing = int(bool(use_nchw)), int(bool(enable_anti_aliasing))
    P.enable_32bit_sort, P.depth_32bit_prec = int(bool(enable_32bit_sort)), float(depth_32bit_prec)
    P.render_inv_depth = int(bool(render_inv_depth))
    if P.enable_32bit_sort:
        assert P.tiles_x * P.tiles_y < 2 ** 14, "32bit sort only support 14 bits tile idx"   # render.py:227-228
    return P


def params_for_scene(scene, filter_algo, training=True, **over) -> OracleParams:
    """Oracle parameters for a synthetic scene object (fields n, width, height, fx, fy, cx, cy,
    cam2world_T, sh_degree, color_sh, near, far)."""
    kw = dict(n=scene.n, width=scene.width, height=scene.height, focal_xy=(scene.fx, scene.fy),
              principal_point=(scene.cx, scene.cy), cam2world_T=scene.cam2world_T, sh_degree=scene.sh_degree,
              sh_stride=scene.color_sh.shape[1], has_sh_base=False, filter_algo=int(filter_algo), training=training,
              near=scene.near, far=scene.far)
    kw.update(over)
    return make_params(**kw)


def expf(x):
    L = lib()
    return np.array([L.orc_expf(float(v)) for v in np.asarray(x, np.float32).ravel()], np.float32)


def expf_blend(x):
    """exp as the blend evaluates it (orc_expf_blend)."""
    L = lib()
    return np.array([L.orc_expf_blend(float(v)) for v in np.asarray(x, np.float32).ravel()], np.float32)


def logf(x):
    L = lib()
    return np.array([L.orc_logf(float(v)) for v in np.asarray(x, np.float32).ravel()], np.float32)


def higher_msb(n: int) -> int:
    return int(lib().orc_higher_msb(int(n)))


def set_num_threads(n: int):
    lib().orc_set_num_threads(C.c_int32(int(n)))


def num_threads() -> int:
    return int(lib().orc_num_threads())


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, np.float32)


def _instances(instances):
    """(instance_ids [N] int32, instance_cameras [I, 12] float32) or None -> the three C arguments."""
    if instances is None:
        return None, None, C.c_int32(0), ()
    ids = np.ascontiguousarray(instances[0], np.int32)
    cams = np.ascontiguousarray(instances[1], np.float32).reshape(-1, 12)
    return _p(ids), _p(cams), C.c_int32(cams.shape[0]), (ids, cams)


def instance_cameras(cam2world_T, instance2world_T):
    """Cameras in the instances' frames, [I, 12] float32 (9 of the world-to-camera rotation, row major, then
    the camera centre), from the view's cam2world_T [4, 3] (rows 0-2: columns of the camera-to-world rotation,
    row 3: centre) and instance2world_T [I, 4, 3] in the same layout: cam2instance = world2instance o cam2world
    (render.py:350-354), evaluated in float64."""
    cw = np.asarray(cam2world_T, np.float64)
    iw = np.asarray(instance2world_T, np.float64).reshape(-1, 4, 3)
    Rc_T, c = cw[:3], cw[3]                 # R_c^T (world -> camera), camera centre
    out = np.empty((iw.shape[0], 12), np.float64)
    for k, T in enumerate(iw):
        Ri, ti = T[:3].T, T[3]              # instance -> world rotation and translation
        out[k, :9] = (Rc_T @ Ri).reshape(-1)
        out[k, 9:] = Ri.T @ (c - ti)
    return out.astype(np.float32)


def preprocess_fwd(P, xyz, quat, scale, opacity, sh, sh_base=None, invalid_mask=None, instances=None):
    n = P.n
    out = dict(
        depths=np.empty(n, np.float32), radii=np.empty(n, np.int32), uvs=np.empty((n, 2), np.float32),
        conic_opacity=np.empty((n, 4), np.float32), tiles_touched=np.empty(n, np.int32),
        rgb_gaussian=np.empty((n, 3), np.float32), cov2d_vecs=np.empty((n, 3), np.float32),
        sh_to_rgb_ne_0=np.empty(n, np.uint8))
    xyz, quat, scale, opacity, sh, sh_base = map(_f32, (xyz, quat, scale, opacity, sh, sh_base))
    mask = None if invalid_mask is None else np.ascontiguousarray(invalid_mask, np.uint8)
    rc = lib().orc_preprocess_fwd(C.byref(P), _p(xyz), _p(quat), _p(scale), _p(opacity), _p(sh), _p(sh_base), _p(mask),
                                  _p(out["depths"]), _p(out["radii"]), _p(out["uvs"]), _p(out["conic_opacity"]),
                                  _p(out["tiles_touched"]), _p(out["rgb_gaussian"]), _p(out["cov2d_vecs"]),
                                  _p(out["sh_to_rgb_ne_0"]), *_instances(instances)[:3])
    if rc != 0:
        raise ValueError("oracle: unsupported early_filter_algo")
    return out


def scan(tiles_touched):
    t = np.ascontiguousarray(tiles_touched, np.int32).copy()
    total = lib().orc_scan(_p(t), C.c_int32(t.shape[0]))
    return t, int(total)


def make_keys(P, radii, uvs, conic_opacity, depths, offsets, m):
    keys = np.zeros(m, np.uint64)
    vals = np.zeros(m, np.int32)
    lib().orc_make_keys(C.byref(P), _p(radii), _p(uvs), _p(conic_opacity), _p(depths), _p(offsets), _p(keys), _p(vals))
    return keys, vals


def sort_pairs(keys, vals, begin_bit, end_bit):
    keys = np.ascontiguousarray(keys, np.uint64)
    vals = np.ascontiguousarray(vals, np.int32)
    ko, vo = np.empty_like(keys), np.empty_like(vals)
    lib().orc_sort_pairs(_p(keys), _p(vals), _p(ko), _p(vo), C.c_int64(keys.shape[0]), C.c_int32(begin_bit),
                         C.c_int32(end_bit))
    return ko, vo


def tile_ranges(keys_sorted, num_tiles, shift=32):
    """shift: where the tile index starts in the key, 32 or (32-bit sort) 18 (render.py:900)."""
    r = np.zeros((num_tiles, 2), np.int32)
    lib().orc_tile_ranges(_p(keys_sorted), C.c_int64(keys_sorted.shape[0]), _p(r), C.c_int32(num_tiles),
                          C.c_int32(shift))
    return r


def _color_shape(P):
    ch = 3 + int(bool(P.render_rgba))
    return (ch, P.height, P.width) if P.use_nchw else (P.height, P.width, ch)


def blend_fwd(P, ranges, idx_sorted, uvs, conic_opacity, rgb, depths=None):
    """Returns (color, T, n_contrib, depth); depth is None unless P.render_depth."""
    H, W = P.height, P.width
    color = np.zeros(_color_shape(P), np.float32)
    T = np.zeros((H, W), np.float32)
    nc = np.zeros((H, W), np.int32)
    depth = np.zeros((H, W), np.float32) if P.render_depth else None
    assert not P.render_depth or depths is not None
    lib().orc_blend_fwd(C.byref(P), _p(ranges), _p(idx_sorted), _p(uvs), _p(conic_opacity), _p(rgb), _p(depths),
                        _p(color), _p(T), _p(nc), _p(depth))
    return color, T, nc, depth


def blend_bwd(P, ranges, idx_sorted, uvs, conic_opacity, rgb, final_T, n_contrib, color, drgb, dT, depths=None,
              final_depth=None, ddepth=None):
    n = P.n
    duv = np.zeros((n, 2), np.float64)
    dconic = np.zeros((n, 3), np.float64)
    dop = np.zeros(n, np.float64)
    dcol = np.zeros((n, 3), np.float64)
    dz = np.zeros(n, np.float64) if P.render_depth else None
    mass = np.zeros((n, 10), np.float64)
    statemass = np.zeros((n, 6), np.float64)
    drgb, dT, ddepth = _f32(drgb), _f32(dT), _f32(ddepth)
    assert drgb.shape == _color_shape(P)
    assert not P.render_depth or (depths is not None and final_depth is not None and ddepth is not None)
    lib().orc_blend_bwd(C.byref(P), _p(ranges), _p(idx_sorted), _p(uvs), _p(conic_opacity), _p(rgb), _p(depths),
                        _p(final_T), _p(n_contrib), _p(color), _p(final_depth), _p(drgb), _p(dT), _p(ddepth),
                        _p(duv), _p(dconic), _p(dop), _p(dcol), _p(dz), _p(mass), _p(statemass))
    # absmass[:, k]: sum of |per-pixel terms| behind each of the ten gradient values (the scale that
    # bounds reordering error): columns duv(2), dconic(3), dopacity(1), dcolor(3), dz(1)
    # statemass[:, k]: for duv(2), dconic(3), dopacity(1), the sum over pixels of |d term / d dl| times
    # sum_ch |drgb| |final colour|: the scale of the error a backward makes whose per-pixel colour state is rebuilt
    # from sums rounded at the magnitude of the final colour (the per-gaussian algorithm)
    return dict(duv=duv, dconic=dconic, dopacity=dop, dcolor=dcol, dz=dz, absmass=mass, statemass=statemass)


def preprocess_bwd(P, xyz, quat, scale, opacity, sh, radii, cov2d, ne0, duv, dconic, dopacity, dcolor, dz=None,
                   sh_mask_compat=False, instances=None):
    n, K = P.n, P.sh_stride
    xyz, quat, scale, opacity, sh, cov2d, duv, dconic, dopacity, dcolor, dz = map(
        _f32, (xyz, quat, scale, opacity, sh, cov2d, duv, dconic, dopacity, dcolor, dz))
    out = dict(dxyz=np.empty((n, 3), np.float32), dquat=np.empty((n, 4), np.float32),
               dscale=np.empty((n, 3), np.float32), dopacity=np.empty(n, np.float32),
               dsh=np.empty((n, K, 3), np.float32),
               dsh_base=np.empty((n, 3), np.float32) if P.has_sh_base else None)
    lib().orc_preprocess_bwd(C.byref(P), _p(xyz), _p(quat), _p(scale), _p(opacity), _p(sh), _p(radii), _p(cov2d),
                             _p(ne0), _p(duv), _p(dconic), _p(dopacity), _p(dcolor), _p(dz),
                             C.c_int32(int(sh_mask_compat)), _p(out["dxyz"]), _p(out["dquat"]), _p(out["dscale"]),
                             _p(out["dopacity"]), _p(out["dsh"]), _p(out["dsh_base"]), *_instances(instances)[:3])
    return out


def forward(P, xyz, quat, scale, opacity, sh, sh_base=None, invalid_mask=None, instances=None):
    """Whole forward: K1 .. K6.  Returns every intermediate the op context holds."""
    pre = preprocess_fwd(P, xyz, quat, scale, opacity, sh, sh_base, invalid_mask, instances)
    offsets, m = scan(pre["tiles_touched"])
    num_tiles = P.tiles_x * P.tiles_y
    keys, vals = make_keys(P, pre["radii"], pre["uvs"], pre["conic_opacity"], pre["depths"], offsets, m)
    # render.py:850-854, 900: 64-bit keys are sorted up to the tile bits in use, 32-bit keys whole
    end_bit = 32 if P.enable_32bit_sort else 32 + higher_msb(num_tiles)
    ks, vs = sort_pairs(keys, vals, 0, end_bit)
    ranges = tile_ranges(ks, num_tiles, 18 if P.enable_32bit_sort else 32)
    color, T, nc, depth = blend_fwd(P, ranges, vs, pre["uvs"], pre["conic_opacity"], pre["rgb_gaussian"], pre["depths"])
    out = dict(pre)
    out.update(offsets=offsets, num_rendered=m, keys=keys, vals=vals, keys_sorted=ks, gaussian_idx_sorted=vs,
               workload_ranges=ranges, color=color, T=T, n_contrib=nc, depth=depth, end_bit=end_bit)
    return out


def _feature_params(P):
    Q = OracleParams.from_buffer_copy(P)
    Q.training, Q.render_depth, Q.render_rgba, Q.use_nchw = 1, 0, 0, 0
    return Q


def _feature_triples(feat):
    feat = _f32(feat)
    for k in range(0, feat.shape[1], 3):
        w = min(3, feat.shape[1] - k)
        tri = np.zeros((feat.shape[0], 3), np.float32)
        tri[:, :w] = feat[:, k:k + w]
        yield k, w, tri


def blend_custom_features(P, fwd, feat):
    """Custom feature image [H, W, F] (render.py:1571-1573, 1920-1923, 2268-2270): every channel is
    accumulated as ``acc += weight * value`` with the colour channels' weights and written without
    background or clamp, so three channels at a time go through the colour blend in training mode."""
    Q = _feature_params(P)
    out = np.zeros((P.height, P.width, feat.shape[1]), np.float32)
    for k, w, tri in _feature_triples(feat):
        img, _, _, _ = blend_fwd(Q, fwd["workload_ranges"], fwd["gaussian_idx_sorted"], fwd["uvs"],
                                 fwd["conic_opacity"], tri)
        out[:, :, k:k + w] = img[:, :, :w]
    return out


def backward(P, fwd, xyz, quat, scale, opacity, sh, drgb, dT, sh_base=None, sh_mask_compat=False, ddepth=None,
             custom_features=None, custom_feature_image=None, dcustom_features=None, instances=None):
    """Whole backward: K7 + K9 from the dict ``forward`` returned.  With custom features
    (render.py:1892-1895, 1952-1955, 1969-1972) the alpha gradient gains
    ``dot(dfeat, T * feat - rest)`` and ``dcustom_features = sum weight * dfeat``: both are linear in
    the channel values, so they are taken from colour-blend backward passes over three channels at a
    time (zero dT) and added; ``g["dcustom_features"]`` is [N, F]."""
    g = blend_bwd(P, fwd["workload_ranges"], fwd["gaussian_idx_sorted"], fwd["uvs"], fwd["conic_opacity"],
                  fwd["rgb_gaussian"], fwd["T"], fwd["n_contrib"], fwd["color"], drgb, dT, fwd["depths"],
                  fwd["depth"], ddepth)
    if custom_features is not None:
        Q = _feature_params(P)
        F = custom_features.shape[1]
        g["dcustom_features"] = np.zeros((P.n, F), np.float64)
        g["absmass_features"] = np.zeros((P.n, F), np.float64)
        zero_dT = np.zeros((P.height, P.width), np.float32)
        for k, w, tri in _feature_triples(custom_features):
            img = np.zeros((P.height, P.width, 3), np.float32)
            img[:, :, :w] = custom_feature_image[:, :, k:k + w]
            dimg = np.zeros_like(img)
            dimg[:, :, :w] = dcustom_features[:, :, k:k + w]
            gk = blend_bwd(Q, fwd["workload_ranges"], fwd["gaussian_idx_sorted"], fwd["uvs"], fwd["conic_opacity"],
                           tri, fwd["T"], fwd["n_contrib"], img, dimg, zero_dT)
            for name in ("duv", "dconic", "dopacity"):
                g[name] += gk[name]
            g["absmass"][:, 0:6] += gk["absmass"][:, 0:6]
            g["dcustom_features"][:, k:k + w] = gk["dcolor"][:, :w]
            g["absmass_features"][:, k:k + w] = gk["absmass"][:, 6:6 + w]
    sh_in = sh
    pb = preprocess_bwd(P, xyz, quat, scale, opacity, sh_in, fwd["radii"], fwd["cov2d_vecs"], fwd["sh_to_rgb_ne_0"],
                        g["duv"].astype(np.float32), g["dconic"].astype(np.float32),
                        g["dopacity"].astype(np.float32), g["dcolor"].astype(np.float32),
                        dz=None if g["dz"] is None else g["dz"].astype(np.float32), sh_mask_compat=sh_mask_compat,
                        instances=instances)
    return g, pb
