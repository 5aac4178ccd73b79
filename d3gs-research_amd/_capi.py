"""ctypes binding of ``libd3gs_hip.so`` (declared in ``include/d3gs_hip.h``).

The library is built in-tree by ``csrc/Makefile`` (``build()`` below drives it).
There is no CPU fallback: loading fails loudly when the shared object is
missing, and every entry point raises ``RuntimeError`` on a non-zero status.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "csrc")
# D3GS_HIP_LIBRARY overrides the in-tree location (a library installed elsewhere)
LIB_PATH = os.environ.get("D3GS_HIP_LIBRARY") or os.path.join(_CSRC, "libd3gs_hip.so")

ABI_VERSION = 34
GRAD_RECORD_FLOATS = 16   # D3GS_GRAD_RECORD_FLOATS
BATCH_CAMERA_FLOATS = 16  # D3GS_BATCH_CAMERA_FLOATS
BUCKET_SIZE = 64          # D3GS_BUCKET_SIZE
ERR_SORT_LOOKBACK = -5    # D3GS_ERR_SORT_LOOKBACK
COUNT_SCAN_GAVE_UP, COUNT_SORT_GAVE_UP, COUNT_PENDING = -1, -2, -3
BIN_WORKSPACES_ARE_ZERO, BIN_HOST_COUNT_AT_END, BIN_KEYS_16BIT = 1, 2, 4
MAX_PAIRS = (1 << 31) - 1024     # D3GS_MAX_PAIRS
SCAN_NOALLOC_MAX_N = 1 << 24   # D3GS_SCAN_NOALLOC_MAX_N


class Params(C.Structure):
    """Mirror of ``d3gs_params``."""
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
        ("render_inv_depth", C.c_int32), ("batch_size", C.c_int32), ("compact_items", C.c_int32), ("batch_cameras", C.c_void_p),
        ("atomic_add_count", C.c_void_p),
    ]


class Instances(C.Structure):
    """Mirror of ``d3gs_instances``: per-gaussian instance ids and one camera (12 floats) per instance."""
    _fields_ = [("instance_ids", C.c_void_p), ("instance_cameras", C.c_void_p), ("num_instances", C.c_int32)]


_VP = C.c_void_p
_SIGNATURES = {
    "d3gs_abi_version": (C.c_int, []),
    "d3gs_last_error_string": (C.c_char_p, []),
    "d3gs_higher_msb": (C.c_int, [C.c_uint32]),
    "d3gs_depth_key_bits": (C.c_int, [C.POINTER(Params)]),
    "d3gs_preprocess_fwd": (C.c_int, [C.POINTER(Params)] + [_VP] * 17 + [C.POINTER(Instances), _VP]),
    "d3gs_sh_colors": (C.c_int, [C.POINTER(Params)] + [_VP] * 6 + [C.POINTER(Instances), _VP]),
    "d3gs_scan_workspace_bytes": (C.c_int, [C.c_int32, C.POINTER(C.c_size_t)]),
    "d3gs_scan_tiles": (C.c_int, [_VP, C.c_int32, _VP, C.c_size_t, _VP, _VP]),
    "d3gs_bin_pairs": (C.c_int, [C.POINTER(Params)] + [_VP] * 10 + [_VP, C.c_size_t, _VP, _VP, C.c_size_t, _VP, _VP, C.c_int64,
                                 _VP, _VP, _VP, _VP, _VP, C.c_size_t, _VP, _VP, C.c_int32, C.POINTER(C.c_int),
                                 C.POINTER(C.c_int), _VP]),
    "d3gs_scan_gathered_workspace_bytes": (C.c_int, [C.c_int32, C.POINTER(C.c_size_t)]),
    "d3gs_scan_gathered": (C.c_int, [_VP, C.c_int32, _VP, C.c_int32, _VP, _VP, C.c_size_t, C.c_int32, _VP, _VP, _VP]),
    "d3gs_scan_gathered_noalloc": (C.c_int, [_VP, C.c_int32, _VP, C.c_int32, _VP, _VP, _VP, _VP]),
    "d3gs_make_keys": (C.c_int, [C.POINTER(Params)] + [_VP] * 11 + [C.c_int64, _VP]),
    "d3gs_depth_keys": (C.c_int, [_VP, C.c_int32, _VP, _VP, _VP]),
    "d3gs_gather_i32": (C.c_int, [_VP, C.c_int32, _VP, C.c_int32, _VP, _VP]),
    "d3gs_sort_workspace_bytes": (C.c_int, [C.c_int64, C.c_int, C.c_int, C.POINTER(C.c_size_t)]),
    "d3gs_sort_pairs": (C.c_int, [_VP, _VP, _VP, _VP, _VP, C.c_size_t, C.c_int64, C.c_int, C.c_int,
                                  C.POINTER(C.c_int), _VP]),
    "d3gs_sort_pairs_u32": (C.c_int, [_VP, _VP, _VP, _VP, _VP, C.c_size_t, C.c_int64, _VP, C.c_int, C.c_int, C.c_int, C.c_int,
                                      C.POINTER(C.c_int), _VP]),
    "d3gs_sort_error_offset": (C.c_int, [C.c_int64, C.c_int, C.c_int, C.POINTER(C.c_size_t)]),
    "d3gs_sort_status": (C.c_int, [_VP, C.c_size_t, C.c_int64, C.c_int, C.c_int, _VP, _VP, _VP]),
    "d3gs_tile_ranges": (C.c_int, [_VP, C.c_int64, _VP, C.c_int32, _VP, _VP]),
    "d3gs_tile_ranges_u32": (C.c_int, [_VP, C.c_int64, _VP, _VP, C.c_int32, _VP, _VP]),
    "d3gs_blend_fwd": (C.c_int, [C.POINTER(Params)] + [_VP] * 11 + [_VP, C.c_size_t] + [_VP]),
    "d3gs_blend_bwd": (C.c_int, [C.POINTER(Params)] + [_VP] * 16 + [_VP]),
    "d3gs_blend_features_fwd": (C.c_int, [C.POINTER(Params)] + [_VP] * 5 + [C.c_int32, _VP, _VP, _VP]),
    "d3gs_blend_features_bwd": (C.c_int, [C.POINTER(Params)] + [_VP] * 5 + [C.c_int32] + [_VP] * 7 + [_VP]),
    "d3gs_preprocess_fwd_sparse": (C.c_int, [C.POINTER(Params)] + [_VP] * 17 + [C.POINTER(Instances), _VP]),
    "d3gs_sh_colors_sparse": (C.c_int, [C.POINTER(Params), _VP, _VP, C.c_int32] + [_VP] * 6 + [C.POINTER(Instances), _VP]),
    "d3gs_preprocess_bwd_sparse": (C.c_int, [C.POINTER(Params)] + [_VP] * 11 + [C.c_int32, C.c_int32] + [_VP] * 6 +
                                   [C.POINTER(Instances), _VP, _VP]),
    "d3gs_unique_ids_workspace_bytes": (C.c_int, [C.c_int32, C.c_int32, C.POINTER(C.c_size_t)]),
    "d3gs_unique_ids": (C.c_int, [_VP, C.c_int32, C.c_int32, _VP, _VP, _VP, _VP, _VP, C.c_size_t, _VP, _VP, _VP]),
    "d3gs_merge_rows": (C.c_int, [_VP, C.c_int32, C.c_int32, _VP, _VP, C.c_int32, _VP, _VP]),
    "d3gs_bucket_offsets": (C.c_int, [_VP, C.c_int32, _VP, _VP]),
    "d3gs_snapshot_floats": (C.c_int, [C.POINTER(Params)]),
    "d3gs_blend_fwd_snapshots": (C.c_int, [C.POINTER(Params)] + [_VP] * 11 + [_VP, C.c_size_t] + [_VP] * 3),
    "d3gs_blend_bwd_per_gaussian": (C.c_int, [C.POINTER(Params)] + [_VP] * 18 + [_VP]),
    "d3gs_preprocess_bwd": (C.c_int, [C.POINTER(Params)] + [_VP] * 10 + [C.c_int32, C.c_int32] + [_VP] * 6 +
                            [C.POINTER(Instances), _VP]),
    "d3gs_preprocess_bwd_camera": (C.c_int, [C.POINTER(Params), C.c_int32, C.c_int32] + [_VP] * 10 +
                                   [C.c_int32, C.c_int32] + [_VP] * 6 + [C.POINTER(Instances), _VP]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def build(force: bool = True) -> str:
    """Compile every HIP source for gfx950 into ``csrc/libd3gs_hip.so``."""
    cmd = ["make", "-C", _CSRC, "-j8"]
    if force:
        cmd.append("-B")
    subprocess.run(cmd, check=True, stdout=subprocess.DEVNULL)
    return LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {_CSRC}` (hipcc, gfx950). "
                "There is no CPU fallback for the rasterizer.")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        if L.d3gs_abi_version() != ABI_VERSION:
            raise RuntimeError(f"libd3gs_hip.so ABI {L.d3gs_abi_version()} != expected {ABI_VERSION}")
        _lib = L
    return _lib


def check(rc: int, what: str):
    if rc != 0:
        msg = lib().d3gs_last_error_string()
        raise RuntimeError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")


def ptr(t):
    """Device pointer of a torch tensor (None -> NULL)."""
    if t is None:
        return None
    assert t.is_contiguous(), "tensor passed to the HIP library must be contiguous"
    return C.c_void_p(t.data_ptr())
