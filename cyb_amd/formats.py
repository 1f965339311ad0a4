"""Host-side tensor-data formats of the import stage (numpy, integer/byte work).

Mirrors what the reference does once, at import time
("F16/F32 weights -> Q4_0 ... canonicalize + quantize + pack" -
/root/reference/decide/pipeline.md:38-40; "no format conversion at runtime" -
:59): quantise a [N,K] = [out,in] weight matrix (:30) in groups of 32 along K
with one f16 scale per group, and pack it into one of the two interchange
layouts libcybq accepts (see include/cybq.h, cybq_layout).

The quantiser definition (scale = absmax / qmax rounded to f16, round half away
from zero, clamp) is this build's; the reference's own quantiser lives in the
`import` crate outside its tree and could not be pinned.
"""
from __future__ import annotations

import numpy as np

GROUP = 32
Q4, Q8 = 4, 8
PLANAR, BLOCK_AOS = 0, 1


def _check(bits: int, K: int) -> None:
    if bits not in (Q4, Q8):
        raise ValueError("bits must be 4 or 8")
    if K % GROUP:
        raise ValueError("K must be a multiple of 32")


def quantize(w: np.ndarray, bits: int):
    """w [N,K] float32 -> (q int8 [N,K], scales uint16 [N,K/32] holding f16 bits)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    N, K = w.shape
    _check(bits, K)
    qmax = np.float32(7.0 if bits == Q4 else 127.0)
    lo = np.float32(-8.0 if bits == Q4 else -127.0)
    g = w.reshape(N, K // GROUP, GROUP)
    amax = np.max(np.abs(g), axis=2)
    with np.errstate(over="ignore"):
        d16 = (amax / qmax).astype(np.float16)
    d16 = np.where(np.isinf(d16), np.float16(65504.0), d16)
    d = d16.astype(np.float32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        r = (g / d).astype(np.float32)
    # round half away from zero, done in float64 so that |r| + 0.5 is exact
    r64 = r.astype(np.float64)
    r64 = np.sign(r64) * np.floor(np.abs(r64) + 0.5)
    r64 = np.clip(r64, float(lo), float(qmax))
    r64 = np.where(d == 0, 0.0, r64)
    q = r64.astype(np.int8).reshape(N, K)
    return q, d16.view(np.uint16).reshape(N, K // GROUP).copy()


def dequantize(q: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """(q int8 [N,K], scales u16 [N,K/32]) -> float32 [N,K]; exact in float32."""
    N, K = q.shape
    d = scales.view(np.float16).astype(np.float32)
    return (q.reshape(N, K // GROUP, GROUP).astype(np.float32) * d[:, :, None]).reshape(N, K)


def pack_planar(q: np.ndarray, bits: int) -> np.ndarray:
    N, K = q.shape
    _check(bits, K)
    if bits == Q8:
        return q.astype(np.int8).view(np.uint8).reshape(N, K).copy()
    u = q.astype(np.int16) & 15
    return (u[:, 0::2] | (u[:, 1::2] << 4)).astype(np.uint8)


def unpack_planar(qplane: np.ndarray, bits: int, N: int, K: int) -> np.ndarray:
    _check(bits, K)
    if bits == Q8:
        return qplane.reshape(N, K).view(np.int8).copy()
    b = qplane.reshape(N, K // 2).astype(np.int16)
    out = np.empty((N, K), dtype=np.int16)
    out[:, 0::2] = b & 15
    out[:, 1::2] = b >> 4
    return np.where(out >= 8, out - 16, out).astype(np.int8)


def pack_blocks(q: np.ndarray, scales: np.ndarray, bits: int) -> np.ndarray:
    """-> uint8 [N * K/32 * (18|34)]: per block f16 d, then the Q4_0 / Q8_0 payload."""
    N, K = q.shape
    _check(bits, K)
    nb = N * (K // GROUP)
    g = q.reshape(nb, GROUP).astype(np.int16)
    bs = 18 if bits == Q4 else 34
    out = np.empty((nb, bs), dtype=np.uint8)
    out[:, 0:2] = scales.reshape(nb, 1).view(np.uint8)
    if bits == Q4:
        out[:, 2:] = (((g[:, :16] + 8) & 15) | (((g[:, 16:] + 8) & 15) << 4)).astype(np.uint8)
    else:
        out[:, 2:] = g.astype(np.int8).view(np.uint8)
    return out.reshape(-1)


def unpack_blocks(blocks: np.ndarray, bits: int, N: int, K: int):
    _check(bits, K)
    nb = N * (K // GROUP)
    bs = 18 if bits == Q4 else 34
    b = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(nb, bs)
    scales = b[:, 0:2].copy().view(np.uint16).reshape(N, K // GROUP)
    if bits == Q4:
        p = b[:, 2:].astype(np.int16)
        q = np.concatenate([(p & 15) - 8, (p >> 4) - 8], axis=1).astype(np.int8)
    else:
        q = b[:, 2:].copy().view(np.int8)
    return q.reshape(N, K), scales


def weight_bytes(bits: int, N: int, K: int) -> int:
    """Algorithmic size of a quantised tensor: payload plus one f16 scale per group."""
    _check(bits, K)
    return N * K * bits // 8 + N * (K // GROUP) * 2


def matmul_bytes(bits: int, N: int, K: int, M: int, x_itemsize: int, y_itemsize: int) -> int:
    """Algorithmic HBM bytes of one op invocation: W once, x once, y once."""
    return weight_bytes(bits, N, K) + M * K * x_itemsize + M * N * y_itemsize


def f32_to_bf16_bits(a: np.ndarray) -> np.ndarray:
    """float32 -> bfloat16 bit patterns (uint16), round to nearest even."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    r = np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
