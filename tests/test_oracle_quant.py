"""Pins quantise / pack / dequant of the oracle against their closed forms and
against the package's independent numpy implementation (cyb_amd.formats)."""
import numpy as np
import pytest

from cyb_amd import formats, synth


@pytest.mark.parametrize("bits", [4, 8])
def test_dequant_closed_form_exhaustive(oracle, bits):
    # every f16 scale x every representable q: w = f32(d) * q, exact in f32
    scales = np.arange(65536, dtype=np.uint16)
    d = scales.view(np.float16).astype(np.float64)
    qs = np.arange(-8, 8) if bits == 4 else np.arange(-128, 128)
    reps = -(-len(qs) // 32)
    qrow = np.resize(qs, reps * 32).astype(np.int8)
    q = np.tile(qrow, (65536, 1))
    s = np.repeat(scales[:, None], reps, axis=1)
    got = oracle.dequant(q, s)
    with np.errstate(invalid="ignore", over="ignore"):
        want = (d[:, None] * qrow[None, :].astype(np.float64)).astype(np.float32)
    fin = np.isfinite(want)
    assert np.array_equal(got[fin].view(np.uint32), want[fin].view(np.uint32))
    # the float64 product is exactly representable: no rounding happened
    assert np.array_equal(want[fin].astype(np.float64), (d[:, None] * qrow[None, :].astype(np.float64))[fin])
    assert np.array_equal(formats.dequantize(q, s)[fin].view(np.uint32), got[fin].view(np.uint32))


@pytest.mark.parametrize("bits", [4, 8])
def test_quantize_invariants(oracle, bits):
    w = synth.weights(7, 96, 256)
    w[3, :32] = 0.0                       # an all-zero group
    w[4, 32:64] *= 1e-7                   # scale underflows towards f16 subnormals
    q, s = oracle.quantize(w, bits)
    qmax = 7 if bits == 4 else 127
    assert q.min() >= (-8 if bits == 4 else -127) and q.max() <= qmax
    d = s.view(np.float16).astype(np.float32)
    g = w.reshape(96, 8, 32)
    amax = np.abs(g).max(axis=2)
    # scale is the f16 rounding of absmax / qmax
    assert np.array_equal(s, (amax / np.float32(qmax)).astype(np.float16).view(np.uint16))
    # zero group -> zero scale, zero q
    assert s[3, 0] == 0 and not q[3, :32].any()
    # the absmax element maps to +-qmax (its quotient is qmax up to the f16 rounding of d)
    qg = q.reshape(96, 8, 32)
    nz = d >= np.float32(2.0 ** -14)          # normal f16 scales
    assert np.all(np.abs(qg).max(axis=2)[nz] == qmax)
    # reconstruction error is at most half a step, or the clamp distance where the
    # f16 rounding of d (subnormal scales lose bits) leaves absmax beyond qmax * d
    err = np.abs(oracle.dequant(q, s).reshape(96, 8, 32) - g)
    bound = np.maximum(0.5 * d, np.abs(amax - np.float32(qmax) * d))
    assert np.all(err <= bound[:, :, None] * (1 + 1e-5) + 1e-30)
    # idempotence: quantising the dequantised tensor reproduces (q, s) when the
    # group still contains +-qmax
    q2, s2 = oracle.quantize(oracle.dequant(q, s), bits)
    assert np.array_equal(s2, s) and np.array_equal(q2, q)


@pytest.mark.parametrize("bits", [4, 8])
def test_quantize_brute_force_tiny(oracle, bits):
    # one group, scalar restatement in float64 / Python
    rng = np.random.default_rng(5)
    for trial in range(200):
        w = (rng.standard_normal(32) * rng.choice([1e-3, 0.02, 3.0])).astype(np.float32)
        if trial % 7 == 0:
            w[rng.integers(32)] = np.float32(0.5) * np.float32(rng.integers(1, 9))  # provoke .5 quotients
        q, s = oracle.quantize(w.reshape(1, 32), bits)
        qmax = 7.0 if bits == 4 else 127.0
        d16 = np.float16(np.float32(np.abs(w).max()) / np.float32(qmax))
        d = np.float32(d16)
        exp = []
        for v in w:
            if d == 0:
                exp.append(0)
                continue
            r = float(np.float32(v) / d)               # f32 division, then exact
            r = np.sign(r) * np.floor(abs(r) + 0.5)
            exp.append(int(min(max(r, -8 if bits == 4 else -127), qmax)))
        assert s[0, 0] == d16.view(np.uint16)
        assert q[0].tolist() == exp


@pytest.mark.parametrize("bits", [4, 8])
def test_numpy_quantizer_matches_oracle(oracle, bits):
    w = synth.weights(8, 64, 512)
    w[0, :32] = 0
    w[1, 5] = 0.3
    q, s = oracle.quantize(w, bits)
    q2, s2 = formats.quantize(w, bits)
    assert np.array_equal(q, q2) and np.array_equal(s, s2)


def test_pack_planar_exhaustive_bytes(oracle):
    # every byte value: low nibble is the even k, high nibble the odd k, two's complement
    lo = np.tile(np.arange(-8, 8, dtype=np.int8), 16)
    hi = np.repeat(np.arange(-8, 8, dtype=np.int8), 16)
    q = np.empty((1, 512), np.int8)
    q[0, 0::2], q[0, 1::2] = lo, hi
    plane = oracle.pack_planar(q, 4)
    assert sorted(plane.tolist()) == list(range(256))
    assert np.array_equal(plane, ((lo.astype(np.int16) & 15) | ((hi.astype(np.int16) & 15) << 4)).astype(np.uint8))
    assert np.array_equal(oracle.unpack_planar(plane, 4, 1, 512), q)
    assert np.array_equal(formats.pack_planar(q, 4).reshape(-1), plane)
    assert np.array_equal(formats.unpack_planar(plane, 4, 1, 512), q)


def test_pack_blocks_hand_vector(oracle):
    # one Q4 block written out by hand: d = 0.5 (0x3800), w[j] = j - 8 for j < 16, w[j+16] = 7 - j
    q = np.concatenate([np.arange(16) - 8, 7 - np.arange(16)]).astype(np.int8).reshape(1, 32)
    s = np.array([[0x3800]], dtype=np.uint16)
    blk = oracle.pack_blocks(q, s, 4)
    want = [0x00, 0x38] + [(j) | ((15 - j) << 4) for j in range(16)]
    assert blk.tolist() == want
    q2, s2 = oracle.unpack_blocks(blk, 4, 1, 32)
    assert np.array_equal(q2, q) and np.array_equal(s2, s)
    assert formats.pack_blocks(q, s, 4).tolist() == want
    # Q8 block: d then the 32 int8 in order
    q8 = (np.arange(32) * 7 - 100).astype(np.int8).reshape(1, 32)
    blk8 = oracle.pack_blocks(q8, s, 8)
    assert blk8.tolist() == [0x00, 0x38] + q8.view(np.uint8).reshape(-1).tolist()
    assert formats.pack_blocks(q8, s, 8).tolist() == blk8.tolist()


@pytest.mark.parametrize("bits", [4, 8])
def test_layout_round_trips(oracle, bits):
    w = synth.weights(9, 48, 160)
    q, s = oracle.quantize(w, bits)
    assert np.array_equal(oracle.unpack_planar(oracle.pack_planar(q, bits), bits, 48, 160), q)
    qb, sb = oracle.unpack_blocks(oracle.pack_blocks(q, s, bits), bits, 48, 160)
    assert np.array_equal(qb, q) and np.array_equal(sb, s)
    qb, sb = formats.unpack_blocks(oracle.pack_blocks(q, s, bits), bits, 48, 160)
    assert np.array_equal(qb, q) and np.array_equal(sb, s)
    assert np.array_equal(formats.pack_blocks(q, s, bits), oracle.pack_blocks(q, s, bits))


def test_bad_arguments(oracle):
    import ctypes
    w = np.zeros((2, 48), np.float32)          # K % 32 != 0
    q = np.zeros((2, 48), np.int8)
    s = np.zeros((2, 2), np.uint16)
    vp = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    assert oracle.L.cybq_oracle_quantize(4, vp(w), 2, 48, vp(q), vp(s)) == -1
    assert oracle.L.cybq_oracle_quantize(5, vp(w), 2, 64, vp(q), vp(s)) == -1
    assert oracle.L.cybq_oracle_dequant(vp(q), vp(s), 2, 48, vp(w)) == -1
