"""Pins tile filters, scan, key expansion, sort and tile ranges of the oracle:
brute force over pixels for the filters' losslessness, numpy cumsum / stable
argsort for the integer stages, and structural invariants of the result."""
import numpy as np
import pytest

from helpers import gen_scene, oracle_forward

NONE, AABB, ELLIPSE, OBB, DFVT = 0, 1, 2, 3, 4


def _tile_sets(ref, n):
    tiles = (ref["keys"] >> np.uint64(32)).astype(np.int64)
    sets = [set() for _ in range(n)]
    for t, g in zip(tiles.tolist(), ref["vals"].tolist()):
        sets[g].add(t)
    return sets


@pytest.mark.parametrize("make", [lambda: gen_scene(0, n=1500), lambda: gen_scene(4, n=3000, wh=(480, 270))])
def test_filters_are_lossless_and_nested(oracle, make):
    """config_def.py:136-141: AABB / OBB only drop tiles in which no pixel reaches alpha >= 1/255;
    OBB tiles are a subset of AABB tiles, which are a subset of the 3-sigma rect (NONE)."""
    scene = make()
    refs = {f: oracle_forward(oracle, scene, f)[1] for f in (NONE, AABB, ELLIPSE, OBB, DFVT)}
    sets = {f: _tile_sets(refs[f], scene.n) for f in refs}
    pre = refs[NONE]
    tiles_x = (scene.width + 15) // 16
    uv = pre["uvs"].astype(np.float64)
    co = pre["conic_opacity"].astype(np.float64)
    dropped_checked = 0
    for g in range(scene.n):
        s_none, s_aabb, s_obb, s_ell = sets[NONE][g], sets[AABB][g], sets[OBB][g], sets[ELLIPSE][g]
        assert s_obb <= s_aabb <= s_none
        assert s_ell <= s_aabb                             # the ellipse lies inside its bounding boxes
        assert sets[DFVT][g] == s_obb                      # the author's invariant, render.py:1051-1072
        for t in s_none - (s_obb & s_ell):
            tx, ty = t % tiles_x, t // tiles_x
            xs = np.arange(tx * 16, min(tx * 16 + 16, scene.width), dtype=np.float64)
            ys = np.arange(ty * 16, min(ty * 16 + 16, scene.height), dtype=np.float64)
            dx = uv[g, 0] - xs[None, :]
            dy = uv[g, 1] - ys[:, None]
            power = -0.5 * (co[g, 0] * dx * dx + co[g, 2] * dy * dy) - co[g, 1] * dx * dy
            alpha = co[g, 3] * np.exp(power)
            assert alpha.max() < (1 / 255.0) * (1 + 1e-4), (g, t, alpha.max())
            dropped_checked += 1
    assert dropped_checked > 100          # the test did examine dropped tiles
    # a lossless filter cannot change the image
    for f in (AABB, ELLIPSE, OBB, DFVT):
        assert np.array_equal(refs[f]["color"], refs[NONE]["color"])
        assert np.array_equal(refs[f]["T"], refs[NONE]["T"])


def test_none_filter_is_the_three_sigma_rect(oracle):
    """render.py:472-473: rect = [int((uv - r)/16), int((uv + r + 15)/16)) clamped to the grid."""
    scene = gen_scene(0)
    ref = oracle_forward(oracle, scene, NONE)[1]
    sets = _tile_sets(ref, scene.n)
    uv, r = ref["uvs"].astype(np.float64), ref["radii"].astype(np.float64)
    tiles = 8
    for g in np.flatnonzero(ref["radii"] > 0)[:800]:
        lo = np.clip(np.trunc((uv[g] - r[g]) / 16), 0, tiles).astype(int)
        hi = np.clip(np.trunc((uv[g] + r[g] + 15) / 16), 0, tiles).astype(int)
        want = {y * tiles + x for y in range(lo[1], hi[1]) for x in range(lo[0], hi[0])}
        assert sets[g] == want
        assert len(want) == (ref["tiles_touched"][g])


@pytest.mark.parametrize("cfg_id,n,wh,filt", [(0, None, None, NONE), (1, 30000, None, AABB), (2, 50000, (640, 360), OBB)])
def test_scan_keys_sort_ranges(oracle, cfg_id, n, wh, filt):
    scene = gen_scene(cfg_id, n=n, wh=wh)
    ref = oracle_forward(oracle, scene, filt)[1]
    tt = ref["tiles_touched"]
    m = ref["num_rendered"]
    # scan == numpy cumsum
    assert np.array_equal(ref["offsets"], np.cumsum(tt, dtype=np.int64).astype(np.int32)) and m == int(tt.sum())
    # keys: emitted at [offset[i-1], offset[i]) with value i, low word = float bits of the depth,
    # high word = tile id in row-major order (render.py:773, 809, 830-833)
    owner = np.repeat(np.arange(scene.n, dtype=np.int32), tt)
    assert np.array_equal(ref["vals"], owner)
    low = (ref["keys"] & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    assert np.array_equal(low, ref["depths"].view(np.uint32)[owner])
    tile = (ref["keys"] >> np.uint64(32)).astype(np.int64)
    num_tiles = ((scene.width + 15) // 16) * ((scene.height + 15) // 16)
    assert tile.min() >= 0 and tile.max() < num_tiles
    first = np.ones(m, bool)
    first[1:] = owner[1:] != owner[:-1]
    assert (np.diff(tile)[~first[1:]] > 0).all()        # row-major ascending within one gaussian
    # sort == numpy stable argsort on the full key (bits above end_bit are zero)
    assert ref["end_bit"] == 32 + int(num_tiles).bit_length()
    order = np.argsort(ref["keys"], kind="stable")
    assert np.array_equal(ref["keys_sorted"], ref["keys"][order])
    assert np.array_equal(ref["gaussian_idx_sorted"], ref["vals"][order])
    # ranges partition [0, m); untouched tiles stay [0, 0)
    r = ref["workload_ranges"]
    lens = r[:, 1] - r[:, 0]
    assert lens.sum() == m and (lens >= 0).all()
    counts = np.bincount(tile, minlength=num_tiles)
    assert np.array_equal(lens, counts)
    assert (r[counts == 0] == 0).all()
    st = tile[order]
    for t in np.flatnonzero(counts)[:200]:
        seg = slice(r[t, 0], r[t, 1])
        assert (st[seg] == t).all()
        d = ref["depths"][ref["gaussian_idx_sorted"][seg]]
        assert (np.diff(d) >= 0).all()                    # front to back
        ties = np.diff(d) == 0
        assert (np.diff(ref["gaussian_idx_sorted"][seg])[ties] > 0).all()   # stable: ties keep index order


def test_sort_bit_range_and_stability(oracle):
    rng = np.random.default_rng(5)
    keys = rng.integers(0, 1 << 40, size=50000, dtype=np.uint64)
    vals = np.arange(keys.size, dtype=np.int32)
    for b, e in ((0, 40), (8, 24), (3, 17), (32, 40), (0, 1)):
        ko, vo = oracle.sort_pairs(keys, vals, b, e)
        masked = (keys >> np.uint64(b)) & np.uint64((1 << (e - b)) - 1)
        order = np.argsort(masked, kind="stable")
        assert np.array_equal(vo, vals[order]) and np.array_equal(ko, keys[order])


def _min_form_over_box(a, b, c, u, v, x0, y0, x1, y1):
    """Exact minimum of q(p) = a (px-u)^2 + 2 b (px-u)(py-v) + c (py-v)^2 over the closed box (float64):
    zero if the centre is inside, else the minimum over the four edges (a convex quadratic on a segment)."""
    if x0 <= u <= x1 and y0 <= v <= y1:
        return 0.0
    best = np.inf
    for y in (y0, y1):                      # horizontal edges: minimise over px
        dy = y - v
        px = np.clip(u - b * dy / a, x0, x1)
        dx = px - u
        best = min(best, a * dx * dx + 2 * b * dx * dy + c * dy * dy)
    for x in (x0, x1):                      # vertical edges: minimise over py
        dx = x - u
        py = np.clip(v - b * dx / c, y0, y1)
        dy = py - v
        best = min(best, a * dx * dx + 2 * b * dx * dy + c * dy * dy)
    return best


@pytest.mark.parametrize("make", [lambda: gen_scene(0, n=1500), lambda: gen_scene(4, n=3000, wh=(480, 270))])
def test_ellipse_filter_is_the_exact_ellipse_box_test(oracle, make):
    """render.py:1277-1297; gs3d.py:1078-1240.  Inside the AABB candidate rect and the 3-sigma rect the
    ELLIPSE filter keeps exactly the tiles whose closed box [16x, 16x+16] x [16y, 16y+16] meets the
    level set {alpha >= alpha_eps}: checked against the float64 minimum of the quadratic form over the
    box, skipping tiles within 1e-3 relative of the boundary."""
    scene = make()
    ref_a = oracle_forward(oracle, scene, AABB)[1]
    ref_e = oracle_forward(oracle, scene, ELLIPSE)[1]
    s_aabb, s_ell = _tile_sets(ref_a, scene.n), _tile_sets(ref_e, scene.n)
    tiles_x = (scene.width + 15) // 16
    uv = ref_a["uvs"].astype(np.float64)
    co = ref_a["conic_opacity"].astype(np.float64)
    decided = dropped = 0
    for g in np.flatnonzero(ref_a["radii"] > 0):
        a, b, c, o = co[g]
        level = -2.0 * np.log((1 / 255.0) / o)              # q(p) <= level  <=>  alpha >= 1/255
        for t in s_aabb[g]:
            tx, ty = t % tiles_x, t // tiles_x
            q = _min_form_over_box(a, b, c, uv[g, 0], uv[g, 1], tx * 16.0, ty * 16.0, tx * 16.0 + 16, ty * 16.0 + 16)
            if abs(q - level) <= 1e-3 * level:
                continue
            assert (t in s_ell[g]) == (q < level), (g, t, q, level)
            decided += 1
            dropped += t not in s_ell[g]
    assert decided > 1000 and dropped > 50


@pytest.mark.parametrize("prec", [0.001, 0.05])
def test_32bit_sort_keys_order_and_ties(oracle, prec):
    """enable_32bit_sort (render.py:227-228, 737, 767-770, 820, 853-854, 900): key = (tile << 18) |
    (uint32(depth / prec) & 0x3FFFF), sorted whole as 32 bits by a stable sort, so gaussians of a tile that share
    a depth step keep index order.  Pinned with numpy: float32 division, truncation, stable lexsort."""
    scene = gen_scene(1, n=20000, wh=(250, 190))
    P64, ref64 = oracle_forward(oracle, scene, AABB)
    P, ref = oracle_forward(oracle, scene, AABB, enable_32bit_sort=True, depth_32bit_prec=prec)
    m = ref["num_rendered"]
    assert m == ref64["num_rendered"] > 0 and np.array_equal(ref["vals"], ref64["vals"])
    # the unsorted keys: same tiles as the 64-bit keys, depth steps from the depths
    tiles = (ref64["keys"] >> np.uint64(32)).astype(np.uint64)
    steps = (ref["depths"] / np.float32(prec)).astype(np.uint32) & np.uint32(0x3FFFF)
    assert np.array_equal(ref["keys"], (tiles << np.uint64(18)) | steps[ref["vals"]].astype(np.uint64))
    assert int(ref["keys"].max()) < 2 ** 32
    # stable sort on the whole key == lexsort by (tile, step), ties in emission order (ascending gaussian index)
    order = np.lexsort((np.arange(m), steps[ref["vals"]], tiles))
    assert np.array_equal(ref["keys_sorted"], ref["keys"][order])
    assert np.array_equal(ref["gaussian_idx_sorted"], ref["vals"][order])
    assert np.array_equal(ref["workload_ranges"], ref64["workload_ranges"])
    # inside a tile: steps ascend, and equal steps list ascending gaussian indices
    lo, hi = max(ref["workload_ranges"], key=lambda r: r[1] - r[0])
    seg_steps, seg_idx = steps[ref["gaussian_idx_sorted"][lo:hi]], ref["gaussian_idx_sorted"][lo:hi]
    assert hi - lo > 20 and (np.diff(seg_steps.astype(np.int64)) >= 0).all()
    same = np.diff(seg_steps.astype(np.int64)) == 0
    assert (np.diff(seg_idx)[same] > 0).all()
    if prec > 0.01:
        # coarse steps: ties exist and reorder the lists against the exact depth order, so the image moves
        assert same.any() and not np.array_equal(ref["gaussian_idx_sorted"], ref64["gaussian_idx_sorted"])
        assert np.abs(ref["color"] - ref64["color"]).max() > 1e-4
    else:
        # 1 mm steps on this scene: a few ties at most, the image stays within blending-order noise
        assert np.abs(ref["color"] - ref64["color"]).max() < 0.2


def test_32bit_sort_depth_steps_wrap_at_18_bits(oracle):
    """Depth steps beyond 2^18 wrap (the mask in render.py:769): with 1e-5 steps a depth of 3 sorts as 300000 - 262144."""
    scene = gen_scene(0, n=800)
    P, ref = oracle_forward(oracle, scene, NONE, enable_32bit_sort=True, depth_32bit_prec=1e-5)
    steps = (ref["depths"] / np.float32(1e-5)).astype(np.uint32)
    assert (steps[ref["radii"] > 0] >= 2 ** 18).any()
    got = (ref["keys"] & np.uint64(0x3FFFF)).astype(np.uint32)
    assert np.array_equal(got, (steps & np.uint32(0x3FFFF))[ref["vals"]])


# ---------------------------------------------------------------------------------------------------------------
# AABB and OBB tile sets pinned from both sides: an independent float64 construction of the level set's bounding
# boxes (closed forms of the inverse conic, numpy.linalg.eigh) and a numpy separating-axis test decide every tile
# of the 3-sigma rect; the oracle must keep exactly those.  A filter that is too tight AND one that is too loose
# (a full width where the reference halves it, a wrong level) both fail here.
# ---------------------------------------------------------------------------------------------------------------
_TWO_SIDED_SCENES = [lambda: gen_scene(0, n=1500), lambda: gen_scene(2, n=4000, wh=(640, 360)),
                     lambda: gen_scene(4, n=3000, wh=(480, 270))]


def _rect_tiles(lo, hi):
    ys, xs = np.meshgrid(np.arange(lo[1], hi[1]), np.arange(lo[0], hi[0]), indexing="ij")
    return xs.ravel(), ys.ravel()


def _three_sigma_rect(u, v, r, tiles_x, tiles_y):
    """render.py:472-473."""
    lim = np.array([tiles_x, tiles_y])
    lo = np.clip(np.trunc((np.array([u, v]) - r) / 16), 0, lim).astype(int)
    hi = np.clip(np.trunc((np.array([u, v]) + r + 15) / 16), 0, lim).astype(int)
    return lo, hi


def _level_and_extents(co):
    """The level L of {q <= L} <=> {alpha >= 1/255} (render.py:1019-1028) and the half extents of the level
    set's axis-aligned bounding box, sqrt(L * Sigma_ii) with Sigma the inverse of the conic matrix."""
    a, b, c, o = co
    level = -2.0 * np.log((1 / 255.0) / o)
    sigma = np.linalg.inv(np.array([[a, b], [b, c]]))
    return level, np.sqrt(level * sigma[0, 0]), np.sqrt(level * sigma[1, 1])


def _near_integer(x, tol=1e-4):
    return abs(x - np.round(x)) < tol


def _candidate_rect(u, v, ex, ey, tiles_x, tiles_y):
    """gs3d.py:968-989 / render.py:1300-1310: tiles [trunc((c - e)/16), ceil((c + e)/16)) of the level set's
    bounding box, clamped to the grid.  None when float32 could round an end to the other side of a tile edge."""
    ends = [(u - ex) / 16, (v - ey) / 16, (u + ex) / 16, (v + ey) / 16]
    if any(_near_integer(e) for e in ends):
        return None
    lim = np.array([tiles_x, tiles_y])
    lo = np.clip(np.trunc(ends[:2]), 0, lim).astype(int)
    hi = np.clip(np.ceil(ends[2:]), 0, lim).astype(int)
    return lo, hi


@pytest.mark.parametrize("make", _TWO_SIDED_SCENES)
def test_aabb_filter_is_exactly_the_level_set_bounding_box(oracle, make):
    """gs3d.py:710-742, 968-989; render.py:1300-1310: AABB keeps a tile of the 3-sigma rect iff its closed box
    [16x, 16x+16] x [16y, 16y+16] meets [u - ex, u + ex] x [v - ey, v + ey]."""
    scene = make()
    ref = oracle_forward(oracle, scene, AABB)[1]
    sets = _tile_sets(ref, scene.n)
    tiles_x, tiles_y = (scene.width + 15) // 16, (scene.height + 15) // 16
    uv, co = ref["uvs"].astype(np.float64), ref["conic_opacity"].astype(np.float64)
    decided = dropped = 0
    for g in np.flatnonzero(ref["radii"] > 0):
        u, v = uv[g]
        level, ex, ey = _level_and_extents(co[g])
        lo, hi = _three_sigma_rect(u, v, float(ref["radii"][g]), tiles_x, tiles_y)
        xs, ys = _rect_tiles(lo, hi)
        # signed gaps between the two intervals on each axis: overlap iff both <= 0
        gx = np.maximum(16.0 * xs - (u + ex), (u - ex) - (16.0 * xs + 16))
        gy = np.maximum(16.0 * ys - (v + ey), (v - ey) - (16.0 * ys + 16))
        gap = np.maximum(gx, gy)
        sure = np.abs(gap) > 1e-3 * max(ex, ey, 1.0)
        # gaps a hair away on the OTHER axis can flip the decision too
        sure &= (np.abs(gx) > 1e-3 * max(ex, 1.0)) & (np.abs(gy) > 1e-3 * max(ey, 1.0))
        want = {int(t) for t in (ys * tiles_x + xs)[sure & (gap < 0)]}
        unsure = {int(t) for t in (ys * tiles_x + xs)[~sure]}
        got = sets[g]
        assert got - unsure == want, (g, sorted(got - unsure), sorted(want))
        decided += int(sure.sum())
        dropped += int((sure & (gap > 0)).sum())
    assert decided > 3000 and dropped > 100


def _obb_gaps(co, u, v, xs, ys):
    """Separating-axis gaps (positive = separated on that axis) between the closed tile boxes and the oriented
    bounding rectangle of {q <= L}: centre (u, v), axes = eigenvectors of the conic matrix (numpy.linalg.eigh),
    half lengths sqrt(L / eigenvalue).  Returns [tiles, 4]."""
    a, b, c, o = co
    level = -2.0 * np.log((1 / 255.0) / o)
    lam, vec = np.linalg.eigh(np.array([[a, b], [b, c]]))
    half = np.sqrt(level / lam)                            # half lengths along vec[:, 0], vec[:, 1]
    d = np.stack([16.0 * xs + 8 - u, 16.0 * ys + 8 - v], 1)   # box centres relative to the rectangle's centre
    axes = np.array([[1.0, 0.0], [0.0, 1.0], vec[:, 0], vec[:, 1]])
    box_r = 8.0 * np.abs(axes).sum(1)                      # projected half extent of a 16 x 16 box
    rect_r = np.abs(axes @ vec) @ half                     # ... of the rectangle
    return np.abs(d @ axes.T) - (box_r + rect_r)[None, :]


@pytest.mark.parametrize("make", _TWO_SIDED_SCENES)
def test_obb_filter_is_exactly_the_oriented_bounding_rectangle(oracle, make):
    """gs3d.py:745-791, 981-987, 1254-1322; render.py:1300-1310: OBB keeps a tile of (candidate rect of the
    level set's bounding box) n (3-sigma rect) iff its closed box meets the oriented bounding rectangle of the
    level set.  ELLIPSE keeps a subset of it."""
    scene = make()
    ref = oracle_forward(oracle, scene, OBB)[1]
    sets = _tile_sets(ref, scene.n)
    sets_ell = _tile_sets(oracle_forward(oracle, scene, ELLIPSE)[1], scene.n)
    sets_aabb = _tile_sets(oracle_forward(oracle, scene, AABB)[1], scene.n)
    tiles_x, tiles_y = (scene.width + 15) // 16, (scene.height + 15) // 16
    uv, co = ref["uvs"].astype(np.float64), ref["conic_opacity"].astype(np.float64)
    decided = dropped = tighter_than_aabb = 0
    for g in np.flatnonzero(ref["radii"] > 0):
        assert sets_ell[g] <= sets[g], g                    # the ellipse lies inside its oriented rectangle
        u, v = uv[g]
        a, b, c, _ = co[g]
        if abs(b) < 1e-6 * max(a, c) and abs(a - c) < 1e-6 * max(a, c):
            continue                                        # isotropic: no axis (own test below)
        level, ex, ey = _level_and_extents(co[g])
        cand = _candidate_rect(u, v, ex, ey, tiles_x, tiles_y)
        if cand is None:
            continue
        lo3, hi3 = _three_sigma_rect(u, v, float(ref["radii"][g]), tiles_x, tiles_y)
        lo, hi = np.maximum(cand[0], lo3), np.minimum(cand[1], hi3)
        assert all((t % tiles_x >= lo[0]) and (t % tiles_x < hi[0]) and (t // tiles_x >= lo[1]) and
                   (t // tiles_x < hi[1]) for t in sets[g]), g
        if (hi <= lo).any():
            assert not sets[g]
            continue
        xs, ys = _rect_tiles(lo, hi)
        gaps = _obb_gaps(co[g], u, v, xs, ys)
        scale = max(np.sqrt(level / min(np.linalg.eigvalsh(np.array([[a, b], [b, c]])))), 8.0)
        sure = (np.abs(gaps) > 1e-3 * scale).all(1)
        meets = (gaps < 0).all(1)
        ids = ys * tiles_x + xs
        want = {int(t) for t in ids[sure & meets]}
        unsure = {int(t) for t in ids[~sure]}
        assert sets[g] - unsure == want, (g, sorted(sets[g] - unsure), sorted(want))
        decided += int(sure.sum())
        dropped += int((sure & ~meets).sum())
        tighter_than_aabb += len(sets_aabb[g] - sets[g])
    assert decided > 3000 and dropped > 100 and tighter_than_aabb > 50


def test_obb_without_an_axis_keeps_every_candidate_tile(oracle):
    """An isotropic conic has no major axis: the reference normalises a zero vector (gs3d.py:761-791), sine and
    cosine are NaN, every `<=` of the separating-axis test (gs3d.py:1254-1322) is false and every tile of the
    candidate rect is kept, the corner tiles the circle does not reach included.  An on-axis isotropic gaussian
    seen by a camera with fx == fy projects to such a conic."""
    import dataclasses
    base = gen_scene(0, n=4)
    xyz = np.array([[0, 0, 3.0], [0, 0, 5.0], [0.4, -0.3, 4.0], [0, 0, 2.0]], np.float32)
    scale = np.log(np.array([[0.4] * 3, [0.72] * 3, [0.5, 0.04, 0.1], [0.2] * 3], np.float32))
    quat = np.array([[0, 0, 0, 1.0]] * 4, np.float32)
    quat[2] = [0, 0, np.sin(np.pi / 8), np.cos(np.pi / 8)]      # long axis along the image diagonal
    scene = dataclasses.replace(base, xyz=xyz, scale=scale, quaternion_xyzw=quat,
                                opacity=np.full(4, 3.0, np.float32))
    refs = {f: oracle_forward(oracle, scene, f)[1] for f in (AABB, ELLIPSE, OBB, DFVT)}
    sets = {f: _tile_sets(refs[f], 4) for f in refs}
    co = refs[OBB]["conic_opacity"]
    for g in (0, 1, 3):
        assert co[g, 0] == co[g, 2] and co[g, 1] == 0 and refs[OBB]["radii"][g] > 0
        assert sets[OBB][g] == sets[AABB][g] == sets[DFVT][g]
        assert len(sets[OBB][g] - sets[ELLIPSE][g]) >= 2, g     # corners of the box the circle leaves out
    assert sets[OBB][2] < sets[AABB][2]      # the anisotropic one is still filtered
