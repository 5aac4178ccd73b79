"""A sort whose look-back gave up must be reported, never taken for a result (the reference's sort throws,
devsort.py:34-37).  The condition is forced from the host: the tests set the error word of a sort workspace
themselves; every kernel runs and exits normally."""
import ctypes as C

import numpy as np
import pytest

from helpers import gen_scene, op_config, torch_model

pytestmark = pytest.mark.gpu


def _error_word(ws, m, begin_bit, end_bit):
    """View of the uint32 error word inside a sort workspace tensor."""
    import torch
    from d3gs_research_amd import _capi
    off = C.c_size_t(0)
    _capi.check(_capi.lib().d3gs_sort_error_offset(m, begin_bit, end_bit, C.byref(off)), "d3gs_sort_error_offset")
    assert off.value % 4 == 0 and off.value + 4 <= ws.numel()
    return ws[off.value:off.value + 4].view(torch.int32)


def test_sort_status_c_abi():
    import torch
    from d3gs_research_amd import _capi
    L = _capi.lib()
    m, begin, end = 70001, 0, 27
    rng = np.random.default_rng(3)
    keys = rng.integers(0, 1 << 27, size=m).astype(np.int32)
    ka, va = torch.from_numpy(keys).cuda(), torch.arange(m, dtype=torch.int32, device="cuda")
    kb, vb = torch.empty_like(ka), torch.empty_like(va)
    nbytes = C.c_size_t(0)
    _capi.check(L.d3gs_sort_workspace_bytes(m, begin, end, C.byref(nbytes)), "ws")
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device="cuda")
    in_b = C.c_int(0)
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    _capi.check(L.d3gs_sort_pairs_u32(_capi.ptr(ka), _capi.ptr(kb), _capi.ptr(va), _capi.ptr(vb), _capi.ptr(ws),
                                      nbytes.value, m, None, 0, 0, begin, end, C.byref(in_b), s), "sort")
    st_dev = torch.full((1,), 77, dtype=torch.int32, device="cuda")
    st_host = torch.full((1,), 77, dtype=torch.int32).pin_memory()
    _capi.check(L.d3gs_sort_status(_capi.ptr(ws), nbytes.value, m, begin, end, _capi.ptr(st_dev),
                                   C.c_void_p(st_host.data_ptr()), s), "status")
    torch.cuda.synchronize()
    assert int(st_dev.item()) == 0 and int(st_host[0]) == 0
    ks = kb if in_b.value else ka
    assert np.array_equal(ks.cpu().numpy(), np.sort(keys, kind="stable"))
    # a workgroup that gives up sets this word; here the host sets it
    _error_word(ws, m, begin, end).fill_(1)
    _capi.check(L.d3gs_sort_status(_capi.ptr(ws), nbytes.value, m, begin, end, _capi.ptr(st_dev),
                                   C.c_void_p(st_host.data_ptr()), s), "status")
    torch.cuda.synchronize()
    assert int(st_dev.item()) == _capi.ERR_SORT_LOOKBACK and int(st_host[0]) == _capi.ERR_SORT_LOOKBACK
    # argument checks
    assert L.d3gs_sort_status(None, nbytes.value, m, begin, end, _capi.ptr(st_dev), None, s) == -1
    assert L.d3gs_sort_status(_capi.ptr(ws), nbytes.value, m, begin, end, None, None, s) == -1
    assert L.d3gs_sort_status(_capi.ptr(ws), 16, m, begin, end, _capi.ptr(st_dev), None, s) == -1


class _LibWithRaisedSortError:
    """The library, except that d3gs_bin_pairs finds the error word of one of its two sort workspaces already
    set, as a workgroup that gave up its look-back would have left it."""

    def __init__(self, lib, which):
        self._lib, self._which = lib, which
        self.calls = 0

    def __getattr__(self, name):
        return getattr(self._lib, name)

    def d3gs_bin_pairs(self, *a):
        import torch
        # argument positions of d3gs_bin_pairs: 0 params .. 11 depth_sort_ws, 12 its size .. 18 capacity ..
        # 23 pair_sort_ws, 24 its size
        params = a[0]._obj
        n, tiles = params.n, params.tiles_x * params.tiles_y
        ws_arg, size, m, bits = ((a[11], a[12], n, self._lib.d3gs_depth_key_bits(a[0])) if self._which == "depth"
                                 else (a[23], a[24], a[18], self._lib.d3gs_higher_msb(tiles)))
        off = C.c_size_t(0)
        assert self._lib.d3gs_sort_error_offset(m, 0, bits, C.byref(off)) == 0 and off.value + 4 <= size

        class _Word:       # the error word as a one-element device array
            __cuda_array_interface__ = {"shape": (1,), "typestr": "<i4", "data": (ws_arg.value + off.value, False),
                                        "version": 2}
        torch.as_tensor(_Word(), device="cuda").fill_(1)
        self.calls += 1
        return self._lib.d3gs_bin_pairs(*a)


@pytest.mark.parametrize("which", ["depth", "pairs"])
def test_forward_bins_again_when_a_sort_of_the_one_call_binning_gave_up(which):
    """Second view of an operator (binning as one library call): the raised error word reaches the host as a
    negative pair count; forward then bins the view once more, launch by launch into exactly sized buffers, and
    renders the right image."""
    import torch
    from d3gs_research_amd.render import GaussianSplatGradients, GaussianSplatOp
    scene = gen_scene(1, n=20000, wh=(256, 192))
    op = GaussianSplatOp(op_config(scene, 1))
    model = torch_model(scene)
    grads = GaussianSplatGradients(drgb=torch.from_numpy(scene.drgb).cuda(), dT=torch.from_numpy(scene.dT).cuda())
    out, ctx = op.forward(model, scene.camera(), training=True)       # sizes the pair buffers
    gm0, _, _ = op.backward(model, scene.camera(), ctx, out, grads)
    good, good_idx, good_dxyz = out.color.clone(), ctx.gaussian_idx_sorted.clone(), gm0.xyz.clone()
    real = op._lib
    op._lib = _LibWithRaisedSortError(real, which)
    out, ctx = op.forward(model, scene.camera(), training=True)
    gm, _, _ = op.backward(model, scene.camera(), ctx, out, grads)
    torch.cuda.synchronize()
    assert op._lib.calls == 1 and op.recovered_views == 1 and not op.last_forward_fused
    assert torch.equal(out.color, good) and torch.equal(ctx.gaussian_idx_sorted, good_idx)
    assert torch.allclose(gm.xyz, good_dxyz, rtol=1e-3, atol=1e-5 * float(good_dxyz.abs().max()))
    op._lib = real
    out, ctx = op.forward(model, scene.camera(), training=True)       # and the next view takes the one-call path again
    assert op.last_forward_fused and op.recovered_views == 1 and torch.equal(out.color, good)


def test_forward_raises_when_the_second_binning_gives_up_too():
    """... and when the launch-by-launch binning reports a look-back that gave up as well, forward raises."""
    import torch
    from d3gs_research_amd.render import GaussianSplatOp
    scene = gen_scene(1, n=20000, wh=(256, 192))
    op = GaussianSplatOp(op_config(scene, 1))
    model = torch_model(scene)
    out, ctx = op.forward(model, scene.camera(), training=True)
    good = out.color.clone()
    real = op._lib

    class _Lib(_LibWithRaisedSortError):
        def d3gs_sort_status(self, ws, nbytes, m, begin, end, st_dev, st_host, stream):
            bad = torch.ones(nbytes, dtype=torch.uint8, device="cuda")      # a workspace whose error word is set
            self.keep = bad
            return real.d3gs_sort_status(C.c_void_p(bad.data_ptr()), nbytes, m, begin, end, st_dev, st_host, stream)

    op._lib = _Lib(real, "pairs")
    with pytest.raises(RuntimeError, match="not sorted"):
        op.forward(model, scene.camera(), training=True)
    assert op.recovered_views == 1
    torch.cuda.synchronize()
    op._lib = real
    out, ctx = op.forward(model, scene.camera(), training=True)       # the operator is usable afterwards
    assert torch.equal(out.color, good)


def test_stepwise_forward_raises_when_a_sort_gave_up():
    """First view of an operator (launch by launch): each sort's status goes to a pinned host word."""
    import torch
    from d3gs_research_amd.render import GaussianSplatOp
    scene = gen_scene(1, n=20000, wh=(256, 192))
    op = GaussianSplatOp(op_config(scene, 1))
    model = torch_model(scene)
    real = op._lib

    class _Lib:
        def __getattr__(self, name):
            return getattr(real, name)

        def d3gs_sort_status(self, ws, nbytes, m, begin, end, st_dev, st_host, stream):
            # report on a workspace whose error word is set instead of the sort's own
            bad = torch.ones(nbytes, dtype=torch.uint8, device="cuda")
            self.keep = bad
            return real.d3gs_sort_status(C.c_void_p(bad.data_ptr()), nbytes, m, begin, end, st_dev, st_host, stream)

    op._lib = _Lib()
    with pytest.raises(RuntimeError, match="not sorted"):
        op.forward(model, scene.camera(), training=True)
    torch.cuda.synchronize()
