"""CPU-side checks of the C-ABI shared library: it loads, exports every symbol the
header declares, and validates arguments without touching a GPU."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "d3gs_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(d3gs_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    from d3gs_research_amd import _capi
    lib = C.CDLL(_capi.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 13
    for sym in declared:
        assert hasattr(lib, sym), f"{sym} declared in d3gs_hip.h but not exported"
    assert sorted(_capi.EXPORTED_SYMBOLS) == declared, "ctypes binding and header disagree"


def test_params_struct_matches_header_layout():
    from d3gs_research_amd import _capi
    # 10 int32 + 6 float + 9 + 3 + 10 float + 3 float + 6 int32 + 1 float + 3 int32, padding to 8, two pointers
    assert C.sizeof(_capi.Params) == 4 * (10 + 6 + 9 + 3 + 10 + 3 + 6 + 1 + 3) + 4 + 16


def test_params_fields_follow_the_header_in_name_and_order():
    """The ctypes mirror of d3gs_params lists the header's fields, in the header's order, with the header's types."""
    from d3gs_research_amd import _capi
    text = open(os.path.join(ROOT, "include", "d3gs_hip.h")).read()
    body = text[text.index("typedef struct d3gs_params {"):text.index("} d3gs_params;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    declared = []
    for ctype, names in re.findall(r"^\s*(int32_t|float|const float\*|uint32_t\*)\s+([^;]+);", body, flags=re.M):
        for name in names.split(","):
            m = re.match(r"\s*(\w+)(?:\[(\d+)\])?\s*$", name)
            declared.append((m.group(1), ctype, int(m.group(2) or 0)))
    kinds = {"int32_t": C.c_int32, "float": C.c_float, "const float*": C.c_void_p, "uint32_t*": C.c_void_p}
    want = [(n, kinds[t] * k if k else kinds[t]) for n, t, k in declared]
    got = list(_capi.Params._fields_)
    assert [n for n, _ in got] == [n for n, _ in want]
    for (n, a), (_, b) in zip(got, want):
        assert C.sizeof(a) == C.sizeof(b) and (a is b or getattr(a, "_length_", 0) == getattr(b, "_length_", 0)), n


def test_abi_version_and_msb():
    from d3gs_research_amd import _capi
    L = _capi.lib()
    assert L.d3gs_abi_version() == 34
    # devsort.py:131-149: bit length; the sort's end bit for the benchmark tile grids
    assert [L.d3gs_higher_msb(v) for v in (0, 1, 64, 1024, 8160, 32400)] == [0, 1, 7, 11, 13, 15]
    # depth-sort key width: float bits of z_far minus those of z_near, or the 18 depth-step bits
    P = _capi.Params()
    widths = []
    for near, far, sort32 in ((0.2, 1e4, 0), (0.01, 100.0, 0), (1.0, 2.0, 0), (0.2, 1e4, 1), (5.0, 1.0, 0), (0.0, 1e4, 0)):
        P.z_near, P.z_far, P.enable_32bit_sort = near, far, sort32
        widths.append(L.d3gs_depth_key_bits(C.byref(P)))
    import struct
    bits = lambda v: struct.unpack("<I", struct.pack("<f", v))[0]
    assert widths == [(bits(1e4) - bits(0.2)).bit_length(), (bits(100.0) - bits(0.01)).bit_length(), 24, 18, 1,
                      bits(1e4).bit_length()] and widths[0] == 27


def test_error_codes_without_compute():
    from d3gs_research_amd import _capi
    L = _capi.lib()
    P = _capi.Params()
    P.n, P.width, P.height, P.tiles_x, P.tiles_y, P.sh_stride = 4, 32, 32, 3, 2, 1   # wrong tile counts
    nul = [None] * 11 + [None, 0, None]     # eleven buffers, the optional clear region, the stream
    rc = L.d3gs_blend_fwd(C.byref(P), *nul)
    assert rc == -1 and b"tiles_x" in L.d3gs_last_error_string()
    P.tiles_x = 2
    P.filter_algo = 7
    assert L.d3gs_blend_fwd(C.byref(P), *nul) == -1 and b"early_filter_algo" in L.d3gs_last_error_string()
    P.filter_algo = 1
    assert L.d3gs_blend_fwd(C.byref(P), *nul) == -1 and b"NULL" in L.d3gs_last_error_string()
    odd = [None] * 11 + [C.c_void_p(24), 32, None]     # clear region not on a 16-byte boundary
    assert L.d3gs_blend_fwd(C.byref(P), *odd) == -1 and b"multiples of 16" in L.d3gs_last_error_string()
    P.sh_degree, P.sh_stride = 3, 4
    assert L.d3gs_blend_fwd(C.byref(P), *nul) == -1 and b"sh_stride" in L.d3gs_last_error_string()
    # the feature kernels: nothing to do without channels, NULL buffers refused with them
    P.sh_stride = 16
    assert L.d3gs_blend_features_fwd(C.byref(P), None, None, None, None, None, 0, None, None, None) == 0
    assert L.d3gs_blend_features_fwd(C.byref(P), None, None, None, None, None, 3, None, None, None) == -1
    assert b"NULL" in L.d3gs_last_error_string()
    assert L.d3gs_blend_features_bwd(C.byref(P), *([None] * 5), -1, *([None] * 8)) == -1
    assert b"num_features" in L.d3gs_last_error_string()
    # 16-bit tile ids are refused for a call with more than 2^16 tiles (before anything is launched)
    big = _capi.Params()
    big.n, big.width, big.height, big.tiles_x, big.tiles_y, big.sh_stride = 4, 16 * 300, 16 * 300, 300, 300, 1
    flags_out = C.c_int(0), C.c_int(0)
    total = C.c_int64(0)
    args = [None] * 10 + [None, 0, None, None, 0, C.addressof(total), None, 0] + [None] * 4 + [None, 0, None, None]
    rc = L.d3gs_bin_pairs(C.byref(big), *args, _capi.BIN_KEYS_16BIT, C.byref(flags_out[0]), C.byref(flags_out[1]), None)
    assert rc == -1 and b"2^16 tiles" in L.d3gs_last_error_string()
    n = C.c_size_t(0)
    assert L.d3gs_sort_workspace_bytes(1000, 0, 65, C.byref(n)) == -1
    assert L.d3gs_sort_workspace_bytes(1000, 0, 45, C.byref(n)) == 0 and n.value > 0
    in_b = C.c_int(7)
    assert L.d3gs_sort_pairs(None, None, None, None, None, 0, 1 << 31, 0, 45, C.byref(in_b), None) == -2   # unsupported size
    assert L.d3gs_sort_pairs(None, None, None, None, None, 0, 0, 0, 45, C.byref(in_b), None) == 0 and in_b.value == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    import pytest
    from d3gs_research_amd import _capi
    monkeypatch.setattr(_capi, "_lib", None)
    monkeypatch.setattr(_capi, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _capi.lib()


def test_operator_config_gate():
    """Options the operator carries out construct; the ones it does not raise at construction, by name."""
    from d3gs_research_amd.config_def import GaussianSplatConfig, RasterizeBackwardAlgo
    from d3gs_research_amd.render import GaussianSplatOp
    GaussianSplatOp(GaussianSplatConfig())
    GaussianSplatOp(GaussianSplatConfig(rasterize_backward_algo=RasterizeBackwardAlgo.PER_GAUSSIAN))
    GaussianSplatOp(GaussianSplatConfig(rasterize_backward_algo=RasterizeBackwardAlgo.PER_GAUSSIAN, render_depth=True,
                                        render_rgba=True, use_nchw=True))
    GaussianSplatOp(GaussianSplatConfig(disable_builtin_rgb=True, render_rgba=True, render_depth=True,
                                        enable_anti_aliasing=True))
    GaussianSplatOp(GaussianSplatConfig(move_opacity_in_grad_to_prep=True, use_int64_tile_touched=True,
                                        enable_32bit_sort=True))
    GaussianSplatOp(GaussianSplatConfig(sparse_mode=True))
    GaussianSplatOp(GaussianSplatConfig(render_inv_depth=True, render_depth=True))
    for kw, word in ((dict(sparse_mode=True, disable_builtin_rgb=True), "sparse_mode"),
                     (dict(rasterize_backward_algo=RasterizeBackwardAlgo.PER_GAUSSIAN, disable_builtin_rgb=True), "PER_GAUSSIAN"),
                     (dict(transmittance_is_double=True), "transmittance_is_double"), (dict(tile_size=(8, 8)), "tile_size"),
                     (dict(disable_builtin_rgb=True, use_nchw=True), "use_nchw")):
        with pytest.raises(NotImplementedError, match=word):
            GaussianSplatOp(GaussianSplatConfig(**kw))


def test_reference_entry_points_are_importable_from_the_render_module():
    """Callers of the reference import these names from its render module (render.py:3783, 3840)."""
    from d3gs_research_amd.render import (CameraBundle, GaussianSplatGradients, GaussianSplatOp,  # noqa: F401
                                          GaussianSplatOutput, rasterize_gaussians, rasterize_gaussians_dynamic)
    from d3gs_research_amd import pvg
    assert rasterize_gaussians_dynamic is pvg.rasterize_gaussians_dynamic
