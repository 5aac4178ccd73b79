"""Key expansion (render.py:745-840) handed offsets it must not trust: a view with more than 2^31 - 1 pairs has
32-bit prefix sums that wrapped negative, and on the one-call binning path the keys are expanded before the host
has seen the (64-bit) total and refused the view.  Nothing may be written outside the key / index buffers;
gaussians whose offsets are sound are still expanded.  Every kernel here runs to completion."""
import ctypes as C

import numpy as np
import pytest

from helpers import gen_scene, op_config, oracle_forward, torch_model

pytestmark = pytest.mark.gpu

GUARD = 4096
SENTINEL_KEY, SENTINEL_VAL = 0x5A5A5A5A5A5A5A5A, -77


@pytest.mark.parametrize("with_masks,key64", [(False, True), (True, True), (True, False)])
@pytest.mark.parametrize("damage", ["wrapped", "shifted"])
def test_make_keys_never_writes_outside_its_buffers(oracle, with_masks, key64, damage):
    import torch
    from d3gs_research_amd import _capi
    from d3gs_research_amd.render import GaussianSplatOp
    scene = gen_scene(1, n=20000, wh=(250, 190))
    filt = 3
    print(f"make_keys guards masks={with_masks} key64={key64} damage={damage}", flush=True)
    _, ref = oracle_forward(oracle, scene, filt)
    op = GaussianSplatOp(op_config(scene, filt))
    model = torch_model(scene)
    P = op.make_params(model, scene.camera(), True)
    L, p = _capi.lib(), _capi.ptr
    N, dev = scene.n, "cuda"
    s = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    f32, i32 = torch.float32, torch.int32
    depths, radii = torch.empty(N, dtype=f32, device=dev), torch.empty(N, dtype=i32, device=dev)
    uvs, conic = torch.empty((N, 2), dtype=f32, device=dev), torch.empty((N, 4), dtype=f32, device=dev)
    touched, rgb = torch.empty(N, dtype=i32, device=dev), torch.empty((N, 3), dtype=f32, device=dev)
    cov2d, ne0 = torch.empty((N, 3), dtype=f32, device=dev), torch.empty(N, dtype=torch.uint8, device=dev)
    masks = torch.empty((N, 2), dtype=torch.int64, device=dev) if with_masks else None
    _capi.check(L.d3gs_preprocess_fwd(C.byref(P), p(model.xyz), p(model.quaternion_xyzw), p(model.scale), p(model.opacity),
                                      p(model.color_sh), None, None, p(depths), p(radii), p(uvs), p(conic), p(touched),
                                      p(rgb), p(cov2d), p(ne0), p(masks), None, None, s), "preprocess")
    M = int(ref["num_rendered"])
    good = ref["offsets"].astype(np.int64)
    cut = N // 2
    bad = good.copy()
    if damage == "wrapped":                 # the prefix sums pass 2^31 at gaussian `cut` and wrap
        bad[cut:] -= 1 << 31
    else:                                   # everything moved in front of the buffer by a few hundred slots
        bad -= 300
    assert (bad < 0).any() and bad.min() >= -(1 << 31)
    offsets = torch.from_numpy(bad.astype(np.int32)).to(dev)

    key_dtype = torch.int64 if key64 else i32
    sent_key = SENTINEL_KEY if key64 else (SENTINEL_KEY & 0x7FFFFFFF)
    keys_full = torch.full((GUARD + M + GUARD,), sent_key, dtype=key_dtype, device=dev)
    vals_full = torch.full((GUARD + M + GUARD,), SENTINEL_VAL, dtype=i32, device=dev)
    keys, vals = keys_full[GUARD:GUARD + M], vals_full[GUARD:GUARD + M]
    _capi.check(L.d3gs_make_keys(C.byref(P), p(radii), p(uvs), p(conic), p(depths), p(offsets), None, None, p(masks),
                                 p(keys) if key64 else None, None if key64 else p(keys), p(vals), M, s), "make_keys")
    torch.cuda.synchronize()
    kf, vf = keys_full.cpu().numpy(), vals_full.cpu().numpy()
    for side in (slice(0, GUARD), slice(GUARD + M, None)):
        assert (kf[side] == sent_key).all() and (vf[side] == SENTINEL_VAL).all()

    # gaussians whose slot range [before, end) is sound still get their pairs, at the slots the offsets name
    before = np.concatenate([[0], bad[:-1]])
    sound = (before >= 0) & (bad > before) & (bad <= M)
    owner = np.repeat(np.arange(N), ref["tiles_touched"])
    ref_keys = ref["keys"] if key64 else (ref["keys"] >> np.uint64(32)).astype(np.uint32)
    ref_start = np.concatenate([[0], good[:-1]])
    written = np.zeros(M, bool)
    got_k = kf[GUARD:GUARD + M].view(np.uint64 if key64 else np.uint32)
    got_v = vf[GUARD:GUARD + M]
    checked = 0
    for g in np.flatnonzero(sound & (ref["tiles_touched"] > 0))[:3000]:
        cnt = int(min(bad[g] - before[g], ref["tiles_touched"][g]))
        dst, src = int(before[g]), int(ref_start[g])
        if damage == "shifted" and g == 0:
            continue
        assert np.array_equal(got_k[dst:dst + cnt], ref_keys[src:src + cnt]), g
        assert (got_v[dst:dst + cnt] == g).all() and (owner[src:src + cnt] == g).all()
        written[dst:dst + cnt] = True
        checked += 1
    assert checked > 500
    if damage == "wrapped":                 # and the gaussians behind the wrap wrote nothing at all
        first_unsound = int(good[cut - 1])
        assert (got_v[first_unsound:] == SENTINEL_VAL).all()
