"""d3gs_scan_gathered_noalloc (status words in a file-scope device array of the library) against
d3gs_scan_gathered (status words in a caller workspace), through the C ABI: same outputs bit for bit, on two
calls in a row, the second over a smaller input, so that the second call meets the first one's status words."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _both(L, x, perm, n):
    import torch
    from d3gs_research_amd import _capi
    src = torch.from_numpy(x).cuda()
    idx = None if perm is None else torch.from_numpy(perm).cuda()
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = []
    for noalloc in (False, True):
        out = torch.full((n,), -1, dtype=torch.int32, device="cuda")
        total = torch.full((1,), -7, dtype=torch.int64, device="cuda")
        host = torch.full((1,), -9, dtype=torch.int64).pin_memory()
        if noalloc:
            _capi.check(L.d3gs_scan_gathered_noalloc(_capi.ptr(src), x.shape[0], _capi.ptr(idx), n, _capi.ptr(out),
                                                     _capi.ptr(total), C.c_void_p(host.data_ptr()), s), "noalloc")
        else:
            nbytes = C.c_size_t(0)
            _capi.check(L.d3gs_scan_gathered_workspace_bytes(n, C.byref(nbytes)), "ws")
            ws = torch.zeros(nbytes.value, dtype=torch.uint8, device="cuda")
            _capi.check(L.d3gs_scan_gathered(_capi.ptr(src), x.shape[0], _capi.ptr(idx), n, _capi.ptr(out), _capi.ptr(ws),
                                             nbytes.value, 1, _capi.ptr(total), C.c_void_p(host.data_ptr()), s), "scan")
        torch.cuda.synchronize()
        res.append((out.cpu().numpy(), int(total.item()), int(host[0])))
    return res


def test_scan_noalloc_matches_scan_with_workspace():
    import torch
    from d3gs_research_amd import _capi
    L = _capi.lib()
    rng = np.random.default_rng(5)
    for n in (3_000_001, 70_001, 1, 1_000_003):        # big, then smaller inputs that reuse the array, then bigger again
        print(f"scan noalloc n={n}", flush=True)
        x = rng.integers(0, 60, size=n, dtype=np.int32)
        perm = rng.permutation(n).astype(np.int32)
        (want, want_total, want_host), (got, got_total, got_host) = _both(L, x, perm, n)
        assert np.array_equal(want, np.cumsum(x[perm].astype(np.int64)).astype(np.int32))
        assert np.array_equal(got, want)
        assert got_total == want_total == int(x.sum()) and got_host == want_host == want_total
    # empty input, and an input beyond the built-in array's size
    total = torch.full((1,), -7, dtype=torch.int64, device="cuda")
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.d3gs_scan_gathered_noalloc(None, 0, None, 0, None, _capi.ptr(total), None, s) == 0
    torch.cuda.synchronize()
    assert int(total.item()) == 0
    rc = L.d3gs_scan_gathered_noalloc(None, 0, None, _capi.SCAN_NOALLOC_MAX_N + 1, None, _capi.ptr(total), None, s)
    assert rc == -3 and b"exceeds" in L.d3gs_last_error_string()
