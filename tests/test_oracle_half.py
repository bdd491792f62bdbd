"""Pins the oracle's FP16 <-> FP32 conversions against numpy's IEEE binary16 (an independent
implementation): every other check of the path rests on them."""
import numpy as np


def test_h2f_all_65536_inputs(O):
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    got = O.h2f(h)
    want = h.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    assert np.isnan(got[nan]).all() and nan.sum() == 2046


def _np_f2h(x):
    with np.errstate(all="ignore"):
        return x.astype(np.float16).view(np.uint16)


def test_f2h_every_tie_and_its_neighbours(O):
    """For every pair of adjacent finite halves (and the last finite one and 65536): the exact
    midpoint and the FP32 values one ulp below and above it, both signs.  Covers round-to-even,
    the subnormal range and the overflow threshold."""
    hh = np.arange(0, 0x7C00, dtype=np.uint32).astype(np.uint16)
    lo = O.h2f(hh).astype(np.float64)
    hi = O.h2f((hh + 1).astype(np.uint16)).astype(np.float64)
    hi[-1] = 65536.0
    mid = ((lo + hi) / 2).astype(np.float32)
    assert ((lo + hi) / 2 == mid.astype(np.float64)).all()      # midpoints are exact in FP32
    for d in (-1, 0, 1):
        x = (mid.view(np.uint32).astype(np.int64) + d).astype(np.uint32).view(np.float32)
        for sgn in (1.0, -1.0):
            xs = (x * np.float32(sgn)).astype(np.float32)
            assert np.array_equal(O.f2h(xs), _np_f2h(xs)), (d, sgn)


def test_f2h_random_bit_patterns_and_specials(O):
    rng = np.random.default_rng(7)
    x = rng.integers(0, 2 ** 32, 4_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    ok = ~np.isnan(x)
    assert np.array_equal(O.f2h(x)[ok], _np_f2h(x)[ok])
    assert (O.f2h(x)[~ok] & 0x7C00 == 0x7C00).all() and (O.f2h(x)[~ok] & 0x3FF != 0).all()   # NaN stays NaN
    # values in the ranges the path lives in
    for scale in (1e-4, 1e-3, 0.02, 1.0, 3e4):
        y = (rng.standard_normal(500_000) * scale).astype(np.float32)
        assert np.array_equal(O.f2h(y), _np_f2h(y))
    spec = np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.99, 65520.0, -65520.0, 2.0 ** -24, 2.0 ** -25,
                     np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -14, 1e-45, 3.4e38], np.float32)
    assert np.array_equal(O.f2h(spec), _np_f2h(spec))
    assert O.lib.orc_f2h(-0.0) == 0x8000 and O.lib.orc_h2f(0x8000) == 0.0


def test_round_trip_is_identity_on_halves(O):
    h = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    finite = (h & 0x7C00) != 0x7C00
    assert np.array_equal(O.f2h(O.h2f(h))[finite], h[finite])
