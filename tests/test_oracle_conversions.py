"""Pins the oracle's scalar conversions against IEEE-754 as numpy implements it."""
import numpy as np


def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def _check_f32_to_f16(oracle, f):
    f = np.ascontiguousarray(f, dtype=np.float32)
    got = oracle.f32_to_f16(f)
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    nan = np.isnan(f)
    assert np.array_equal(got[~nan], want[~nan])
    # NaN stays NaN with its sign
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x3FF) != 0)


def test_f32_to_f16_round_trip_and_ties(oracle):
    h = np.arange(65536, dtype=np.uint16)
    exact = h.view(np.float16).astype(np.float32)
    _check_f32_to_f16(oracle, exact)
    # midpoints between neighbouring f16 values (ties) and their f32 neighbours
    fin = exact[np.isfinite(exact)]
    fin = np.unique(fin)
    mid = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)
    for cand in (mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))):
        _check_f32_to_f16(oracle, cand)
    # overflow boundary, tiny values, signed zeros, infinities, NaN
    edge = np.array([65504.0, 65519.99, 65520.0, 65536.0, 1e9, -65520.0, 2.0 ** -24, 2.0 ** -25,
                     np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -26, 0.0, -0.0,
                     np.inf, -np.inf, np.nan, 6.1e-5, 6.0e-5], dtype=np.float32)
    _check_f32_to_f16(oracle, edge)


def test_f32_to_f16_random(oracle):
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    _check_f32_to_f16(oracle, bits.view(np.float32))
    _check_f32_to_f16(oracle, rng.standard_normal(1_000_000).astype(np.float32) * 0.01)


def test_bf16_round_trip_and_rounding(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.bf16_to_f32(bits)
    assert np.array_equal(f.view(np.uint32), bits.astype(np.uint32) << 16)
    ok = ~np.isnan(f)
    assert np.array_equal(oracle.f32_to_bf16(f[ok]), bits[ok])
    # round to nearest even on the dropped 16 bits, checked in integer arithmetic
    rng = np.random.default_rng(2)
    u = rng.integers(0, 2 ** 32, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    fin = np.isfinite(x)
    u, x = u[fin], x[fin]
    got = oracle.f32_to_bf16(x).astype(np.uint32)
    lo, keep = u & 0xFFFF, u >> 16
    up = (lo > 0x8000) | ((lo == 0x8000) & ((keep & 1) == 1))
    assert np.array_equal(got, (keep + up) & 0xFFFF)
    # the package's numpy twin agrees
    from cyb_amd import formats
    assert np.array_equal(formats.f32_to_bf16_bits(x), got.astype(np.uint16))
