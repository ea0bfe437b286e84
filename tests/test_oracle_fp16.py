"""Pins the oracle's software binary16 conversions against numpy's float16 (IEEE, round-to-nearest-even)."""
import ctypes as C

import numpy as np


def _h2f(olib, h):
    f = np.empty(h.shape, np.float32)
    olib.oracle_half_to_float(h.ctypes.data, f.ctypes.data, h.size)
    return f


def _f2h(olib, f):
    h = np.empty(f.shape, np.uint16)
    olib.oracle_float_to_half(f.ctypes.data, h.ctypes.data, f.size)
    return h


def test_half_to_float_all_patterns(olib):
    h = np.arange(65536, dtype=np.uint16)
    got = _h2f(olib, h)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(got[np.isnan(want)]).all()


def test_float_to_half_roundtrip_and_ties(olib):
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    ok = ~np.isnan(f)
    assert np.array_equal(_f2h(olib, f)[ok], h[ok])
    # midpoints between neighbouring halves (ties) and their float32 neighbours on either side
    pos = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = pos.view(np.float16).astype(np.float64)
    hi = (pos + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0  # the would-be next value above 65504 decides the overflow tie
    mid = ((lo + hi) / 2).astype(np.float32)
    for cand in (mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)), -mid):
        cand = np.ascontiguousarray(cand, dtype=np.float32)
        with np.errstate(over="ignore"):
            want = cand.astype(np.float16).view(np.uint16)
        assert np.array_equal(_f2h(olib, cand), want)


def test_float_to_half_random_bits(olib):
    rng = np.random.default_rng(7)
    bits = rng.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    ok = ~np.isnan(f)
    with np.errstate(over="ignore", invalid="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = _f2h(olib, np.ascontiguousarray(f))
    assert np.array_equal(got[ok], want[ok])
    assert ((got[~ok] & 0x7c00) == 0x7c00).all() and ((got[~ok] & 0x3ff) != 0).all()
    # dense sweep through the subnormal/normal boundary and the overflow boundary
    for lo, hi in ((0x33000000 - 64, 0x33000000 + 64), (0x38800000 - 4096, 0x38800000 + 4096),
                   (0x477fe000 - 64, 0x477ff000 + 64)):
        f = np.arange(lo, hi, dtype=np.uint32).view(np.float32)
        with np.errstate(over="ignore"):
            assert np.array_equal(_f2h(olib, np.ascontiguousarray(f)), f.astype(np.float16).view(np.uint16))
