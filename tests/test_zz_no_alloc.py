"""cybq_matmul_static - the entry point that allocates nothing - against cybq_matmul, through the C ABI.

Two calls in a row on the same device, the second with a smaller input: the static scratch keeps the
first call's contents and the second must not see them."""
import numpy as np
import pytest

from cyb_amd import formats, synth

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _case(backend, oracle, N, K, M, xdt, mode):
    backend.set_prefill_mode(mode)
    q, s = oracle.quantize(synth.weights(77, N, K), 4)
    qw = backend.upload_quantized(q, s, 4)
    x = torch.from_numpy(synth.activations(77, M, K)).cuda().to(xdt)
    want = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    got = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    backend.matmul(qw, x, want)
    backend.matmul_static(qw, x, got)
    torch.cuda.synchronize()
    # same kernels, same operands; the K split may differ (the scratch sizes differ), i.e. summation order
    err = ((got.double() - want.double()).norm() / want.double().norm()).item()
    assert err < 2e-6, (N, K, M, mode, err)
    rows = [0, M // 2, M - 1]
    ref = oracle.matmul_f64(q, s, x[rows].float().cpu().numpy())
    prefill = M > (16 if xdt == torch.float32 else 32)          # FAST prefill rounds weights (and fp32 rows) once to f16
    bar = 5e-4 if prefill and mode == "fast" else 2e-5
    assert oracle.rel_l2(got[rows].cpu().numpy(), ref) < bar, (N, K, M, mode)
    qw.free()


def test_static_scratch_matches_allocated_workspace(backend, oracle):
    try:
        for mode in ("fast", "exact"):
            # a K split with several slabs and a full stage, then a smaller call that must not see leftovers
            _case(backend, oracle, 4096, 14336, 512, torch.bfloat16, mode)
            _case(backend, oracle, 1024, 2048, 100, torch.bfloat16, mode)
        _case(backend, oracle, 14336, 4096, 300, torch.float16, "fast")
        _case(backend, oracle, 320, 4096, 1, torch.float16, "fast")         # decode rows use no scratch at all
        _case(backend, oracle, 320, 4096, 24, torch.float32, "fast")
    finally:
        backend.set_prefill_mode("fast")


def test_static_scratch_limits(backend, oracle):
    from cyb_amd.backend import CybqError
    N, K = 16, 32768 + 128
    q, s = oracle.quantize(synth.weights(78, N, K), 4)
    qw = backend.upload_quantized(q, s, 4)
    x = torch.zeros((64, K), dtype=torch.float16, device="cuda")
    y = torch.zeros((64, N), dtype=torch.float32, device="cuda")
    with pytest.raises(CybqError) as e:
        backend.matmul_static(qw, x, y)
    assert e.value.status == -7 and "32768" in str(e.value)
    backend.matmul_static(qw, x[:4].contiguous(), y[:4])                     # decode rows: no limit
    torch.cuda.synchronize()
    qw.free()
