"""Pins the oracle's deterministic exp / log against float64 libm (they are the
functions whose operation sequence the HIP kernels repeat)."""
import numpy as np


def _ulp_err(got32, want64):
    want32 = want64.astype(np.float32)
    ulp = np.spacing(np.abs(want32)).astype(np.float64)
    return np.abs(got32.astype(np.float64) - want64) / ulp


def test_expf_within_1p5_ulp(oracle):
    rng = np.random.default_rng(0)
    x = np.concatenate([np.linspace(-85.9, 87.9, 20001), rng.uniform(-12, 1, 20000), [0.0, -0.0, 1e-8, -1e-8]]).astype(np.float32)
    got = oracle.expf(x)
    err = _ulp_err(got, np.exp(x.astype(np.float64)))
    assert err.max() <= 1.5, err.max()
    # range edges and special values
    assert oracle.expf([-86.5])[0] == 0.0 and np.isinf(oracle.expf([88.5])[0]) and np.isnan(oracle.expf([np.nan])[0])
    assert oracle.expf([0.0])[0] == 1.0


def test_blend_expf_within_1p5_ulp(oracle):
    """The blend's exp takes its k = round(x log2 e) from one fused multiply-add with 1.5 * 2^23: same accuracy
    bound as the plain function over the range it is evaluated in, the same value wherever both pick the same k."""
    rng = np.random.default_rng(2)
    x = np.concatenate([np.linspace(-79.9, 79.9, 20001), rng.uniform(-6, 0, 40000), [0.0, -0.0, -1e-8,
                        # half-integers of x log2 e, where the two range reductions may pick different k
                        *(np.float32((k + 0.5) / 1.44269504088896341) for k in range(-9, 2))]]).astype(np.float32)
    got = oracle.expf_blend(x)
    assert _ulp_err(got, np.exp(x.astype(np.float64))).max() <= 1.5
    plain = oracle.expf(x)
    assert (got == plain).mean() > 0.999 and oracle.expf_blend([0.0])[0] == 1.0
    # outside the range the kernels evaluate it in: the plain function
    assert oracle.expf_blend([-86.5])[0] == 0.0 and np.isnan(oracle.expf_blend([np.nan])[0])


def test_logf_within_1p5_ulp(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([np.exp(rng.uniform(-80, 80, 20000)), rng.uniform(1 / 300, 1.0, 20000), [1.0, 0.5, 2.0]]).astype(np.float32)
    got = oracle.logf(x)
    want = np.log(x.astype(np.float64))
    want32 = want.astype(np.float32)
    ulp = np.maximum(np.spacing(np.abs(want32)).astype(np.float64), 2.0 ** -24 * 1e-3)
    err = np.abs(got.astype(np.float64) - want) / ulp
    # near x = 1 the result is tiny and an absolute bound is the meaningful one
    assert (np.abs(got.astype(np.float64) - want) <= np.maximum(1.5 * ulp, 1.2e-7)).all(), err.max()
    assert oracle.logf([1.0])[0] == 0.0
    assert np.isneginf(oracle.logf([0.0])[0]) and np.isneginf(oracle.logf([-1.0])[0])


def test_higher_msb_is_bit_length(oracle):
    # devsort.py:131-149; sort end bit = 32 + bit length of the tile count for the benchmark grids
    for n, want in ((0, 0), (1, 1), (2, 2), (64, 7), (1024, 11), (8160, 13), (32400, 15), (2 ** 31, 32)):
        assert oracle.higher_msb(n) == want == int(n).bit_length()
