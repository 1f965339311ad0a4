"""ctypes front of the C oracle (oracle/_build/libcybq_oracle.so).

Test infrastructure: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py only.  Builds the library on first use when it is
missing (gcc only, no GPU involved)."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(_ROOT, "oracle", "_build", "libcybq_oracle.so")
_SO_CPU = os.path.join(_ROOT, "oracle", "_build", "libcybq_cpu_baseline.so")


def _arr(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a, a.ctypes.data_as(ctypes.c_void_p)


class Oracle:
    def __init__(self):
        if not os.path.exists(_SO) or not os.path.exists(_SO_CPU):
            subprocess.run(["make"], cwd=os.path.join(_ROOT, "oracle"), check=True,
                           stdout=subprocess.DEVNULL)
        L = ctypes.CDLL(_SO)
        vp, sz, ci = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
        L.cybq_oracle_f16_to_f32.restype = ctypes.c_float
        L.cybq_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.cybq_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.cybq_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        for n in ("f16_to_f32_n", "f32_to_f16_n", "bf16_to_f32_n", "f32_to_bf16_n"):
            getattr(L, "cybq_oracle_" + n).argtypes = [vp, vp, sz]
            getattr(L, "cybq_oracle_" + n).restype = None
        L.cybq_oracle_quantize.argtypes = [ci, vp, sz, sz, vp, vp]
        L.cybq_oracle_pack_planar.argtypes = [ci, vp, sz, sz, vp]
        L.cybq_oracle_unpack_planar.argtypes = [ci, vp, sz, sz, vp]
        L.cybq_oracle_pack_blocks.argtypes = [ci, vp, vp, sz, sz, vp]
        L.cybq_oracle_unpack_blocks.argtypes = [ci, vp, sz, sz, vp, vp]
        L.cybq_oracle_dequant.argtypes = [vp, vp, sz, sz, vp]
        L.cybq_oracle_matmul_f32.argtypes = [vp, vp, sz, sz, vp, sz, vp]
        L.cybq_oracle_matmul_f64.argtypes = [vp, vp, sz, sz, vp, sz, vp]
        L.cybq_oracle_matmul_blocked_mt.argtypes = [vp, vp, sz, sz, vp, sz, vp, ci]
        L.cybq_oracle_rel_l2.argtypes = [vp, vp, sz]
        L.cybq_oracle_rel_l2.restype = ctypes.c_double
        self.L = L

    # conversions -----------------------------------------------------------
    def f16_to_f32(self, h):
        h, hp = _arr(h, np.uint16)
        out = np.empty(h.shape, np.float32)
        self.L.cybq_oracle_f16_to_f32_n(hp, out.ctypes.data_as(ctypes.c_void_p), h.size)
        return out

    def f32_to_f16(self, f):
        f, fp = _arr(f, np.float32)
        out = np.empty(f.shape, np.uint16)
        self.L.cybq_oracle_f32_to_f16_n(fp, out.ctypes.data_as(ctypes.c_void_p), f.size)
        return out

    def bf16_to_f32(self, h):
        h, hp = _arr(h, np.uint16)
        out = np.empty(h.shape, np.float32)
        self.L.cybq_oracle_bf16_to_f32_n(hp, out.ctypes.data_as(ctypes.c_void_p), h.size)
        return out

    def f32_to_bf16(self, f):
        f, fp = _arr(f, np.float32)
        out = np.empty(f.shape, np.uint16)
        self.L.cybq_oracle_f32_to_bf16_n(fp, out.ctypes.data_as(ctypes.c_void_p), f.size)
        return out

    # import stage ------------------------------------------------------------
    def quantize(self, w, bits):
        w, wp = _arr(w, np.float32)
        N, K = w.shape
        q = np.empty((N, K), np.int8)
        s = np.empty((N, K // 32), np.uint16)
        rc = self.L.cybq_oracle_quantize(bits, wp, N, K, q.ctypes.data_as(ctypes.c_void_p),
                                         s.ctypes.data_as(ctypes.c_void_p))
        assert rc == 0
        return q, s

    def pack_planar(self, q, bits):
        q, qp = _arr(q, np.int8)
        N, K = q.shape
        out = np.empty(N * K * bits // 8, np.uint8)
        assert self.L.cybq_oracle_pack_planar(bits, qp, N, K, out.ctypes.data_as(ctypes.c_void_p)) == 0
        return out

    def unpack_planar(self, plane, bits, N, K):
        plane, pp = _arr(plane, np.uint8)
        q = np.empty((N, K), np.int8)
        assert self.L.cybq_oracle_unpack_planar(bits, pp, N, K, q.ctypes.data_as(ctypes.c_void_p)) == 0
        return q

    def pack_blocks(self, q, s, bits):
        q, qp = _arr(q, np.int8)
        s, sp = _arr(s, np.uint16)
        N, K = q.shape
        out = np.empty(N * (K // 32) * (18 if bits == 4 else 34), np.uint8)
        assert self.L.cybq_oracle_pack_blocks(bits, qp, sp, N, K, out.ctypes.data_as(ctypes.c_void_p)) == 0
        return out

    def unpack_blocks(self, blocks, bits, N, K):
        blocks, bp = _arr(blocks, np.uint8)
        q = np.empty((N, K), np.int8)
        s = np.empty((N, K // 32), np.uint16)
        assert self.L.cybq_oracle_unpack_blocks(bits, bp, N, K, q.ctypes.data_as(ctypes.c_void_p),
                                                s.ctypes.data_as(ctypes.c_void_p)) == 0
        return q, s

    def dequant(self, q, s):
        q, qp = _arr(q, np.int8)
        s, sp = _arr(s, np.uint16)
        N, K = q.shape
        w = np.empty((N, K), np.float32)
        assert self.L.cybq_oracle_dequant(qp, sp, N, K, w.ctypes.data_as(ctypes.c_void_p)) == 0
        return w

    # the op ------------------------------------------------------------------
    def _mm(self, fn, q, s, x, out_dtype, *extra):
        q, qp = _arr(q, np.int8)
        s, sp = _arr(s, np.uint16)
        x, xp = _arr(x, np.float32)
        if x.ndim == 1:
            x = x.reshape(1, -1)
        N, K = q.shape
        M = x.shape[0]
        assert x.shape[1] == K
        y = np.empty((M, N), out_dtype)
        assert fn(qp, sp, N, K, xp, M, y.ctypes.data_as(ctypes.c_void_p), *extra) == 0
        return y

    def matmul_f32(self, q, s, x):
        return self._mm(self.L.cybq_oracle_matmul_f32, q, s, x, np.float32)

    def matmul_f64(self, q, s, x):
        return self._mm(self.L.cybq_oracle_matmul_f64, q, s, x, np.float64)

    def matmul_mt(self, q, s, x, threads):
        return self._mm(self.L.cybq_oracle_matmul_blocked_mt, q, s, x, np.float32, threads)

    # the optimised CPU path that bench.py times beside the GPU (oracle/cybq_cpu_baseline.c) ----
    def _cpu(self):
        if getattr(self, "_C", None) is None:
            C = ctypes.CDLL(_SO_CPU)
            C.cybq_cpu_q4_0_matmul.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p,
                                               ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int]
            C.cybq_cpu_baseline_isa.restype = ctypes.c_char_p
            self._C = C
        return self._C

    def cpu_baseline_isa(self) -> str:
        return self._cpu().cybq_cpu_baseline_isa().decode()

    def cpu_baseline_q4_0(self, blocks, N, K, x, threads, out=None):
        """y [M,N] f32 = x [M,K] f32 times the Q4_0 BLOCK_AOS tensor `blocks` (uint8, N*K/32*18 bytes)."""
        assert blocks.dtype == np.uint8 and blocks.flags.c_contiguous and blocks.size == N * (K // 32) * 18
        x, xp = _arr(x, np.float32)
        M = x.shape[0]
        if out is None:
            out = np.empty((M, N), np.float32)
        used = self._cpu().cybq_cpu_q4_0_matmul(blocks.ctypes.data, N, K, xp, M, out.ctypes.data, threads)
        return out, used

    def rel_l2(self, a, b):
        a, ap = _arr(a, np.float32)
        b, bp = _arr(b, np.float64)
        assert a.size == b.size
        return float(self.L.cybq_oracle_rel_l2(ap, bp, a.size))
