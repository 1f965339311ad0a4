"""ctypes binding of libcybq.so and the host-side mirror of the runtime's
backend seam.

Reference shape being mirrored (the runtime crate itself is outside the
reference tree, so these are the in-tree facts the mirror is built from):
  * one backend object per process, created when the mind is spawned
    (/root/reference/shell/src/worlds/soma_bridge.rs:65);
  * weights are handed over once per model load and kept until the model is
    swapped (/root/reference/shell/src/worlds/models/mod.rs:7-8,386);
  * the graph IR names an op, its weight tensor (HF-style name) and its in/out
    edges (/root/reference/decide/pipeline.md:28-30); the executor calls the
    backend once per node per token (:51);
  * failures surface as values, never as panics
    (/root/reference/shell/src/worlds/soma_bridge.rs:322-333) - here CybqError.

Nothing in this module computes the op on the host.  If libcybq.so cannot be
loaded the import of this module still succeeds (so that CPU-only tooling can
use cyb_amd.formats), but constructing a Backend raises.
"""
from __future__ import annotations

import ctypes
import os
from dataclasses import dataclass, field
from typing import Dict, Optional

import numpy as np

from . import formats

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "lib", "libcybq.so")

F32, F16, BF16 = 0, 1, 2
EPILOGUES = {"none": 0, "add": 1, "swiglu": 2}      # enum cybq_epilogue
_DTYPE_CODES = {"torch.float32": F32, "torch.float16": F16, "torch.bfloat16": BF16,
                "float32": F32, "float16": F16}
_ITEMSIZE = {F32: 4, F16: 2, BF16: 2}


class CybqError(RuntimeError):
    def __init__(self, status: int, text: str, detail: str = ""):
        self.status = status
        msg = f"cybq status {status} ({text})"
        if detail:
            msg += f": {detail}"
        super().__init__(msg)


def library_path() -> str:
    return _LIB_PATH


_lib = None


def load_library() -> ctypes.CDLL:
    """Loads libcybq.so from cyb_amd/lib (built in-tree by __graft_entry__.build())."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise CybqError(-4, "library missing", f"{_LIB_PATH} not built; run __graft_entry__.build()")
    lib = ctypes.CDLL(_LIB_PATH)
    vp, i64, ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.cybq_version.restype = ctypes.c_char_p
    lib.cybq_strerror.restype = ctypes.c_char_p
    lib.cybq_strerror.argtypes = [ci]
    lib.cybq_last_error.restype = ctypes.c_char_p
    lib.cybq_last_error.argtypes = [vp]
    lib.cybq_init.argtypes = [ci, ctypes.POINTER(vp)]
    lib.cybq_destroy.argtypes = [vp]
    lib.cybq_destroy.restype = None
    lib.cybq_weight_upload.argtypes = [vp, ci, ci, i64, i64, vp, vp, ctypes.POINTER(vp)]
    lib.cybq_weight_from_device.argtypes = [vp, ci, i64, i64, vp, vp, vp, ctypes.POINTER(vp)]
    lib.cybq_weight_clone.argtypes = [vp, vp, ctypes.POINTER(vp)]
    lib.cybq_weight_free.argtypes = [vp, vp]
    lib.cybq_weight_info.argtypes = [vp, ctypes.POINTER(ci), ctypes.POINTER(i64), ctypes.POINTER(i64),
                                     ctypes.POINTER(i64)]
    lib.cybq_matmul.argtypes = [vp, vp, vp, ci, i64, vp, ci, vp]
    lib.cybq_matmul_static.argtypes = [vp, vp, vp, ci, i64, vp, ci, vp]
    lib.cybq_matmul_ex.argtypes = [vp, vp, vp, ci, i64, vp, ci, ci, vp, vp]
    lib.cybq_matmul_norm.argtypes = [vp, vp, vp, ci, i64, vp, ci, ctypes.c_float, vp, ci, ci, vp, vp]
    lib.cybq_weight_fuse_pairs.argtypes = [vp, vp, vp, ctypes.POINTER(vp)]
    lib.cybq_matmul_many_ex.argtypes = [vp, i64, vp, vp, vp, vp, vp, ci, i64, ci, vp]
    lib.cybq_matmul_many_norm.argtypes = [vp, i64, vp, vp, vp, ci, ctypes.c_float, vp, vp, vp, ci, i64, ci, vp]
    lib.cybq_set_prefill_mode.argtypes = [vp, ci]
    lib.cybq_set_decode_mode.argtypes = [vp, ci]
    lib.cybq_matmul_many.argtypes = [vp, i64, vp, vp, vp, ci, i64, ci, vp]
    lib.cybq_dequant.argtypes = [vp, vp, vp, vp]
    lib.cybq_quantize.argtypes = [vp, ci, vp, i64, i64, vp, vp, vp]
    # diagnostics (cyb_amd/csrc/cybq_debug.h), not part of the operator interface
    lib.cybq_debug_set_gemm_tuning.argtypes = [ci]
    lib.cybq_debug_set_gemv_tuning.argtypes = [ci, ci, ci]
    lib.cybq_debug_read_weight.argtypes = [vp, i64, vp, ci, vp, vp, vp]
    lib.cybq_debug_read_pattern.argtypes = [vp, i64, vp, ci, vp]
    lib.cybq_debug_mfma_loop.argtypes = [vp, ci, ci, vp, vp]
    lib.cybq_debug_cache_read.argtypes = [vp, vp, i64, ci, ci, ci, vp]
    _lib = lib
    return lib


def _ptr(t) -> int:
    if t is None:
        return 0
    if isinstance(t, int):
        return t
    return int(t.data_ptr())


def _dtype_code(t, explicit: Optional[int]) -> int:
    if explicit is not None:
        return explicit
    key = str(getattr(t, "dtype", ""))
    if key not in _DTYPE_CODES:
        raise CybqError(-1, "invalid argument", f"unsupported dtype {key!r}")
    return _DTYPE_CODES[key]


@dataclass
class QMatMul:
    """Stand-in for the graph-IR node of the op: y = x @ dequant(w)^T.

    `w` is the HF-style tensor name, `x` / `y` are edge names.  The field list of
    the reference's node is not available in its tree; these are the facts any
    such node has to carry."""
    w: str
    x: str
    y: str
    quant: int = formats.Q4
    group: int = formats.GROUP
    M: int = 1
    N: int = 0
    K: int = 0
    op: str = "qmatmul"


class QWeight:
    """One uploaded quantised tensor (device-native layout), immutable."""

    def __init__(self, backend: "Backend", handle: int):
        self._backend = backend
        self._h = ctypes.c_void_p(handle)
        q, n, k, b = ctypes.c_int(), ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        backend._check(backend._lib.cybq_weight_info(self._h, q, n, k, b))
        self.quant, self.N, self.K, self.device_bytes = q.value, n.value, k.value, b.value

    @property
    def handle(self) -> ctypes.c_void_p:
        if not self._h:
            raise CybqError(-1, "invalid argument", "weight already freed")
        return self._h

    @property
    def algorithmic_bytes(self) -> int:
        return formats.weight_bytes(self.quant, self.N, self.K)

    def clone(self) -> "QWeight":
        out = ctypes.c_void_p()
        b = self._backend
        b._check(b._lib.cybq_weight_clone(b._ctx, self.handle, ctypes.byref(out)))
        return QWeight(b, out.value)

    def free(self) -> None:
        if self._h and self._backend._ctx:
            self._backend._lib.cybq_weight_free(self._backend._ctx, self._h)
        self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class MatmulPlan:
    """Pointer arrays of a fixed node list (one decode step's linears)."""

    def __init__(self, backend: "Backend", weights, xs, ys, epilogues=None, residuals=None, gammas=None, eps: float = 1e-5):
        n = len(weights)
        if not (n == len(xs) == len(ys)):
            raise CybqError(-1, "invalid argument", "weights / xs / ys differ in length")
        self.count = n
        self.checked = set()                            # batch sizes whose buffers were validated
        self.keep = (list(weights), list(xs), list(ys), list(residuals or []))      # keeps tensors and handles alive
        arr = ctypes.c_void_p * n
        self.w = arr(*[w.handle.value for w in weights])
        self.x = arr(*[_ptr(t) for t in xs])
        self.y = arr(*[_ptr(t) for t in ys])
        self.xdt = _dtype_code(xs[0], None) if n else F16
        self.ydt = _dtype_code(ys[0], None) if n else F32
        self.epi = self.res = None
        if epilogues is not None:
            if len(epilogues) != n or (residuals is not None and len(residuals) != n):
                raise CybqError(-1, "invalid argument", "epilogues / residuals differ in length from the node list")
            self.epi = (ctypes.c_int * n)(*[EPILOGUES[e] for e in epilogues])
            self.res = arr(*[_ptr(r) for r in (residuals or [None] * n)])
        # folded RMSNorm per node (None = no norm in front of that node): cybq_matmul_many_norm
        self.gamma = None
        self.eps = float(eps)
        self.gdt = F32
        if gammas is not None:
            if len(gammas) != n:
                raise CybqError(-1, "invalid argument", "gammas differ in length from the node list")
            given = [g for g in gammas if g is not None]
            if given:
                self.gdt = _dtype_code(given[0], None)
                if any(_dtype_code(g, None) != self.gdt for g in given):
                    raise CybqError(-1, "invalid argument", "all gammas of a plan share one type")
                self.gamma = arr(*[_ptr(g) for g in gammas])
                self.keep = self.keep + (list(gammas),)


class Backend:
    """A device context plus the tensors of the loaded model, keyed by name."""

    def __init__(self, device: int = 0):
        self._lib = load_library()
        self._ctx = ctypes.c_void_p()
        rc = self._lib.cybq_init(device, ctypes.byref(self._ctx))
        if rc != 0:
            self._ctx = ctypes.c_void_p()
            raise CybqError(rc, self._lib.cybq_strerror(rc).decode())
        self.device = device
        self.weights: Dict[str, QWeight] = {}

    # ---- plumbing
    def _check(self, rc: int) -> None:
        if rc != 0:
            detail = self._lib.cybq_last_error(self._ctx).decode() if self._ctx else ""
            raise CybqError(rc, self._lib.cybq_strerror(rc).decode(), detail)

    def close(self) -> None:
        for w in list(self.weights.values()):
            w.free()
        self.weights.clear()
        if self._ctx:
            self._lib.cybq_destroy(self._ctx)
            self._ctx = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def version(self) -> str:
        return self._lib.cybq_version().decode()

    # ---- weights
    def upload(self, quant: int, layout: int, N: int, K: int, q: np.ndarray,
               scales: Optional[np.ndarray] = None, name: Optional[str] = None) -> QWeight:
        """Host interchange buffers -> device-native weight (repacked once, here)."""
        q = np.ascontiguousarray(q)
        qp = q.ctypes.data_as(ctypes.c_void_p)
        sp = None
        if N >= 1 and K >= 32 and K % 32 == 0 and quant in (formats.Q4, formats.Q8):
            groups = N * (K // 32)
            if layout == formats.PLANAR:
                need_q, need_s = N * K * quant // 8, groups * 2
            else:
                need_q, need_s = groups * (18 if quant == formats.Q4 else 34), 0
            if q.nbytes < need_q or (need_s and scales is not None and np.asarray(scales).nbytes < need_s):
                raise CybqError(-2, "bad shape", f"host buffers are smaller than a [{N},{K}] Q{quant} tensor in this layout")
        if scales is not None:
            scales = np.ascontiguousarray(scales)
            sp = scales.ctypes.data_as(ctypes.c_void_p)
        out = ctypes.c_void_p()
        self._check(self._lib.cybq_weight_upload(self._ctx, quant, layout, N, K, qp, sp, ctypes.byref(out)))
        w = QWeight(self, out.value)
        if name is not None:
            self.weights[name] = w
        return w

    def upload_quantized(self, q: np.ndarray, scales: np.ndarray, quant: int, layout: int = formats.PLANAR,
                         name: Optional[str] = None) -> QWeight:
        """Canonical (q int8 [N,K], scales u16 [N,K/32]) -> pack -> upload."""
        N, K = q.shape
        if layout == formats.PLANAR:
            return self.upload(quant, layout, N, K, formats.pack_planar(q, quant), scales, name)
        return self.upload(quant, layout, N, K, formats.pack_blocks(q, scales, quant), None, name)

    def weight_from_device(self, quant: int, N: int, K: int, q_dev, scales_dev, stream: int = 0,
                           name: Optional[str] = None) -> QWeight:
        out = ctypes.c_void_p()
        self._check(self._lib.cybq_weight_from_device(self._ctx, quant, N, K, _ptr(q_dev), _ptr(scales_dev),
                                                      stream, ctypes.byref(out)))
        w = QWeight(self, out.value)
        if name is not None:
            self.weights[name] = w
        return w

    # ---- ops (x / y / out: torch tensors on this device, or raw device addresses)
    def _check_tensor(self, t, what: str, elems: int) -> None:
        """A tensor handed to the C ABI must be contiguous, on this context's device and large enough:
        the library only sees a raw pointer.  (Raw integer addresses are the caller's responsibility.)"""
        if t is None or isinstance(t, int):
            return
        if not t.is_contiguous():
            raise CybqError(-2, "bad shape", f"{what} must be contiguous")
        if not t.is_cuda or (t.device.index or 0) != self.device:
            raise CybqError(-1, "invalid argument", f"{what} must live on cuda:{self.device}")
        if t.numel() < elems:
            raise CybqError(-2, "bad shape", f"{what} holds {t.numel()} elements, the call needs {elems}")

    def _check_call(self, w: QWeight, x, y, M: int, epilogue: str = "none", residual=None, gamma=None) -> None:
        n_out = w.N // 2 if epilogue == "swiglu" else w.N
        self._check_tensor(x, "x", M * w.K)
        self._check_tensor(y, "y", M * n_out)
        self._check_tensor(residual, "residual", M * n_out)
        self._check_tensor(gamma, "gamma", w.K)

    def matmul(self, w: QWeight, x, y, M: Optional[int] = None, xdt: Optional[int] = None,
               ydt: Optional[int] = None, stream: int = 0) -> None:
        if M is None:
            M = int(x.shape[0]) if x.dim() == 2 else 1
        self._check_call(w, x, y, M)
        self._check(self._lib.cybq_matmul(self._ctx, w.handle, _ptr(x), _dtype_code(x, xdt), M, _ptr(y),
                                          _dtype_code(y, ydt), stream))

    def matmul_static(self, w: QWeight, x, y, M: Optional[int] = None, stream: int = 0) -> None:
        """cybq_matmul_static: the same op with its scratch in a static device array (allocates nothing)."""
        if M is None:
            M = int(x.shape[0]) if x.dim() == 2 else 1
        self._check_call(w, x, y, M)
        self._check(self._lib.cybq_matmul_static(self._ctx, w.handle, _ptr(x), _dtype_code(x, None), M, _ptr(y),
                                                 _dtype_code(y, None), stream))

    def matmul_ex(self, w: QWeight, x, y, epilogue: str = "none", residual=None, M: Optional[int] = None,
                  stream: int = 0) -> None:
        """cybq_matmul_ex: epilogue "none", "add" (y = residual + x W^T) or "swiglu" (w from
        fuse_pairs; y has half as many columns as w has rows)."""
        if epilogue not in EPILOGUES:
            raise CybqError(-1, "invalid argument", f"unknown epilogue {epilogue!r}")
        if M is None:
            M = int(x.shape[0]) if x.dim() == 2 else 1
        self._check_call(w, x, y, M, epilogue, residual)
        self._check(self._lib.cybq_matmul_ex(self._ctx, w.handle, _ptr(x), _dtype_code(x, None), M, _ptr(y),
                                             _dtype_code(y, None), EPILOGUES[epilogue], _ptr(residual), stream))

    def matmul_norm(self, w: QWeight, x, gamma, eps: float, y, epilogue: str = "none", residual=None,
                    M: Optional[int] = None, stream: int = 0) -> None:
        """cybq_matmul_norm: RMSNorm (gamma [K], eps) folded into the activation load, then the epilogue."""
        if epilogue not in EPILOGUES:
            raise CybqError(-1, "invalid argument", f"unknown epilogue {epilogue!r}")
        if M is None:
            M = int(x.shape[0]) if x.dim() == 2 else 1
        self._check_call(w, x, y, M, epilogue, residual, gamma)
        self._check(self._lib.cybq_matmul_norm(self._ctx, w.handle, _ptr(x), _dtype_code(x, None), M, _ptr(gamma),
                                               _dtype_code(gamma, None), ctypes.c_float(eps), _ptr(y),
                                               _dtype_code(y, None), EPILOGUES[epilogue], _ptr(residual), stream))

    def fuse_pairs(self, gate: QWeight, up: QWeight, name: Optional[str] = None) -> QWeight:
        """One weight holding gate and up projections interleaved by 16-row strip (device to device)."""
        out = ctypes.c_void_p()
        self._check(self._lib.cybq_weight_fuse_pairs(self._ctx, gate.handle, up.handle, ctypes.byref(out)))
        w = QWeight(self, out.value)
        if name is not None:
            self.weights[name] = w
        return w

    def plan_many(self, weights, xs, ys, epilogues=None, residuals=None, gammas=None, eps: float = 1e-5) -> "MatmulPlan":
        """Freezes a list of (weight, x, y[, epilogue, residual, gamma]) nodes into pointer arrays for matmul_many."""
        return MatmulPlan(self, weights, xs, ys, epilogues, residuals, gammas, eps)

    def matmul_many(self, plan: "MatmulPlan", M: int, stream: int = 0) -> None:
        if M not in plan.checked:                      # once per plan and batch size, not per step
            ws, xs, ys, rs = plan.keep[:4]
            gs = plan.keep[4] if len(plan.keep) > 4 else None
            for i, w in enumerate(ws):
                epi = "none"
                if plan.epi is not None:
                    epi = next(k for k, v in EPILOGUES.items() if v == plan.epi[i])
                self._check_call(w, xs[i], ys[i], M, epi, rs[i] if rs else None, gs[i] if gs else None)
            plan.checked.add(M)
        if plan.gamma is not None:
            self._check(self._lib.cybq_matmul_many_norm(self._ctx, plan.count, plan.w, plan.x, plan.gamma, plan.gdt,
                                                        ctypes.c_float(plan.eps), plan.y, plan.epi, plan.res, plan.xdt, M,
                                                        plan.ydt, stream))
            return
        if plan.epi is not None:
            self._check(self._lib.cybq_matmul_many_ex(self._ctx, plan.count, plan.w, plan.x, plan.y, plan.epi, plan.res,
                                                      plan.xdt, M, plan.ydt, stream))
            return
        self._check(self._lib.cybq_matmul_many(self._ctx, plan.count, plan.w, plan.x, plan.y, plan.xdt, M,
                                               plan.ydt, stream))

    def dequant(self, w: QWeight, out, stream: int = 0) -> None:
        self._check(self._lib.cybq_dequant(self._ctx, w.handle, _ptr(out), stream))

    def quantize(self, quant: int, src, N: int, K: int, q_out, scales_out, stream: int = 0) -> None:
        self._check(self._lib.cybq_quantize(self._ctx, quant, _ptr(src), N, K, _ptr(q_out), _ptr(scales_out),
                                            stream))

    def run(self, node: QMatMul, edges: dict, stream: int = 0) -> None:
        """Executes one graph node: edges[node.y] = edges[node.x] @ W[node.w]^T."""
        if node.op != "qmatmul":
            raise CybqError(-7, "unsupported", f"op {node.op!r}")
        if node.group != formats.GROUP:
            raise CybqError(-2, "bad shape", "group must be 32")
        w = self.weights.get(node.w)
        if w is None:
            raise CybqError(-1, "invalid argument", f"weight {node.w!r} not loaded")
        if (node.N and node.N != w.N) or (node.K and node.K != w.K) or node.quant != w.quant:
            raise CybqError(-2, "bad shape", f"node {node.w!r} does not match the loaded tensor")
        self.matmul(w, edges[node.x], edges[node.y], M=node.M, stream=stream)

    def set_prefill_mode(self, mode: str) -> None:
        """'fast' (default): one f16 MFMA per group, weights rounded once to f16;
        'exact': lossless hi/lo split, two MFMAs per group."""
        codes = {"fast": 0, "exact": 1}
        if mode not in codes:
            raise CybqError(-1, "invalid argument", f"prefill mode {mode!r}")
        self._check(self._lib.cybq_set_prefill_mode(self._ctx, codes[mode]))

    def set_decode_mode(self, mode: str) -> None:
        """'stream' (default): one f16 row multiplies subnormal weight operands straight from memory;
        'exact': exact integer weight operands."""
        codes = {"stream": 0, "exact": 1}
        if mode not in codes:
            raise CybqError(-1, "invalid argument", f"decode mode {mode!r}")
        self._check(self._lib.cybq_set_decode_mode(self._ctx, codes[mode]))

    def debug_read_weights(self, plan: "MatmulPlan", with_io: bool, x=None, y=None, stream: int = 0) -> None:
        """Diagnostics: the one-row decode kernel's memory requests without its arithmetic, one launch per
        weight of `plan` (with_io: also the activation read and a 16-float store per strip)."""
        self._check(self._lib.cybq_debug_read_weight(self._ctx, plan.count, plan.w, 1 if with_io else 0, _ptr(x), _ptr(y),
                                                     stream))

    def debug_read_pattern(self, plan: "MatmulPlan", pattern: int, stream: int = 0) -> None:
        """Diagnostics: the weights of `plan` read by another pure-read pattern (1 .. 6, cybq_debug.h), one
        launch per weight."""
        self._check(self._lib.cybq_debug_read_pattern(self._ctx, plan.count, plan.w, pattern, stream))

    def debug_mfma_loop(self, waves_per_simd: int, iters: int, sink, stream: int = 0) -> None:
        """Diagnostics: `iters` x 16 independent v_mfma_f32_16x16x32_f16 per wave on every SIMD
        (waves_per_simd = 0: one wave per SIMD, `iters` x 8 v_mfma_f32_32x32x16_f16)."""
        self._check(self._lib.cybq_debug_mfma_loop(self._ctx, waves_per_simd, iters, _ptr(sink), stream))

    def debug_cache_read(self, buf, nbytes: int, waves: int, in_flight: int, iters: int, stream: int = 0) -> None:
        """Diagnostics: one workgroup of `waves` waves per CU, each reads the same `nbytes` at `buf` `iters`
        times, 1 KiB per wave instruction, `in_flight` instructions outstanding per wave."""
        self._check(self._lib.cybq_debug_cache_read(self._ctx, _ptr(buf), nbytes, waves, in_flight, iters, stream))

    def set_gemm_tuning(self, rows_kernel: int = 0) -> None:
        """Experiments only: 2 keeps prefill calls of up to 512 rows away from the K-splitting kernel, 1 sends
        calls of up to 64 rows there whatever the output width, 0 restores the automatic choice."""
        self._lib.cybq_debug_set_gemm_tuning(rows_kernel)

    def set_gemv_tuning(self, waves: int = 0, rows_kernel: int = 0, unroll: int = 0) -> None:
        """Diagnostics: waves per workgroup; decode kernel choice (0 auto, 1 always the
        x-in-registers kernel, 2 never); streaming batch size.  0 = automatic."""
        self._lib.cybq_debug_set_gemv_tuning(waves, rows_kernel, unroll)
