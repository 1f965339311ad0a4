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
        _case(backend, oracle, 14336, 4096, 48, torch.bfloat16, "fast")     # few rows on a wide output: the waves split K
        _case(backend, oracle, 4096, 14336, 16, torch.float16, "fast")      # decode rows on few strips and a long K: tickets and slabs
        _case(backend, oracle, 320, 4096, 1, torch.float16, "fast")         # (other decode rows use no scratch at all)
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


def test_static_entry_point_allocates_nothing(oracle):
    """The property the entry point exists for: a call makes no device allocation.  On a fresh context a
    512-row call on a long K (staging pass, multiply split four ways over K, slab adding: every user of
    the scratch) is recorded into a HIP graph - an allocation during capture fails - and replayed against the
    eager result; and the free device memory is the same before and after a run of eager calls."""
    from cyb_amd import Backend
    be = Backend(0)
    try:
        N, K, M = 4096, 14336, 512
        q, s = oracle.quantize(synth.weights(79, N, K), 4)
        qw = be.upload_quantized(q, s, 4)
        x = torch.from_numpy(synth.activations(79, M, K)).cuda().to(torch.bfloat16)
        x1 = x[:1].to(torch.float16).contiguous()
        y = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        y1 = torch.zeros((1, N), dtype=torch.float32, device="cuda")
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):           # first launches of these kernels on this context
            st = torch.cuda.current_stream().cuda_stream
            be.matmul_static(qw, x, y, stream=st)
            be.matmul_static(qw, x1, y1, stream=st)
        want, want1 = torch.empty_like(y), torch.empty_like(y1)
        be.matmul(qw, x, want)
        be.matmul(qw, x1, want1)
        torch.cuda.synchronize()
        for _ in range(3):
            y.zero_()
            y1.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            err = ((y.double() - want.double()).norm() / want.double().norm()).item()
            assert err < 2e-6, err
            assert torch.equal(y1, want1)
        rows = [0, 255, 511]
        assert oracle.rel_l2(y[rows].cpu().numpy(), oracle.matmul_f64(q, s, x[rows].float().cpu().numpy())) < 5e-4
        # eager calls: free device memory does not move
        be.matmul_static(qw, x, y)
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        for _ in range(5):
            be.matmul_static(qw, x, y)
            be.matmul_static(qw, x1, y1)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0
        qw.free()
    finally:
        be.close()
