"""Parity of the HIP path (through the C ABI) against the oracle, on an MI355X.

Bars: dequantised weights bit-exact; matmul outputs within 1e-3 relative L2 of
the float64 oracle (the fp32-accumulating kernels land near 1e-6, asserted at
2e-5 for fp32 outputs so that a dropped group or a wrong scale cannot hide)."""
import numpy as np
import pytest

from cyb_amd import QMatMul, formats, synth
from cyb_amd.backend import CybqError

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

TOL = 1e-3          # the operator's stated tolerance
TIGHT = 2e-5        # what fp32 accumulation actually delivers
FAST = 5e-4         # prefill FAST mode: weights rounded once to f16 (expected ~2e-4)


@pytest.fixture(params=["exact", "fast"])
def prefill_mode(request, backend):
    backend.set_prefill_mode(request.param)
    yield request.param
    backend.set_prefill_mode("fast")


def _bar(mode):
    return TIGHT if mode == "exact" else FAST

TDT = {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}


def _quant(oracle, bits, N, K, cfg=21):
    w = synth.weights(cfg, N, K)
    return oracle.quantize(w, bits)


def _x(M, K, dt, cfg=21, outliers=0.0):
    x = torch.from_numpy(synth.activations(cfg, M, K, outliers=outliers)).cuda().to(TDT[dt])
    return x


def _run(backend, qw, x, ydt="f32"):
    M = x.shape[0]
    y = torch.full((M, qw.N), float("nan"), dtype=TDT[ydt], device="cuda")
    backend.matmul(qw, x, y)
    torch.cuda.synchronize()
    return y


# ------------------------------------------------------------------ dequant

@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("layout", [formats.PLANAR, formats.BLOCK_AOS])
@pytest.mark.parametrize("shape", [(1, 32), (17, 160), (16, 128), (100, 4096), (1024, 4096)])
def test_dequant_bit_exact(backend, oracle, bits, layout, shape):
    N, K = shape
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits, layout)
    out = torch.empty((N, K), dtype=torch.float32, device="cuda")
    backend.dequant(qw, out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), oracle.dequant(q, s).view(np.uint32))
    assert qw.algorithmic_bytes == formats.weight_bytes(bits, N, K)
    qw.free()


@pytest.mark.parametrize("bits", [4, 8])
def test_dequant_exhaustive_scales_and_values(backend, oracle, bits):
    # every finite f16 scale against every representable q (extremes included)
    scales = np.arange(65536, dtype=np.uint16)
    fin = np.isfinite(scales.view(np.float16))
    scales = scales[fin]
    qs = np.arange(-8, 8) if bits == 4 else np.arange(-128, 128)
    reps = -(-len(qs) // 32)
    qrow = np.resize(qs, reps * 32).astype(np.int8)
    q = np.tile(qrow, (len(scales), 1))
    s = np.repeat(scales[:, None], reps, axis=1)
    qw = backend.upload_quantized(q, s, bits)
    out = torch.empty(q.shape, dtype=torch.float32, device="cuda")
    backend.dequant(qw, out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), oracle.dequant(q, s).view(np.uint32))


# ------------------------------------------------------------ decode (M <= 16)

@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("xdt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("M", [1, 2, 3, 4, 7, 8, 16])
def test_decode_matches_oracle(backend, oracle, bits, xdt, M):
    N, K = 272, 1024
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits)
    x = _x(M, K, xdt, outliers=0.001)
    y = _run(backend, qw, x).cpu().numpy()
    ref = oracle.matmul_f64(q, s, x.float().cpu().numpy())
    err = oracle.rel_l2(y, ref)
    assert err < TIGHT, err
    # and against the fp32-accumulating CPU path itself
    y32 = oracle.matmul_f32(q, s, x.float().cpu().numpy())
    assert oracle.rel_l2(y, y32.astype(np.float64)) < TIGHT


@pytest.mark.parametrize("shape", [(1, 32), (5, 64), (16, 128), (33, 160), (1000, 2080), (48, 32768)])
def test_decode_ragged_shapes(backend, oracle, shape):
    N, K = shape
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4, formats.BLOCK_AOS)
    for M in (1, 5, 16):
        x = _x(M, K, "f16")
        y = _run(backend, qw, x).cpu().numpy()
        assert not np.isnan(y).any()
        assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.float().cpu().numpy())) < TIGHT


def test_decode_seven_strips_per_workgroup(backend, oracle):
    # N = 7 * 16 * 256: on a 256-CU part the batched-rows kernel gives every workgroup seven strips
    N, K = 28672, 256
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    for M in (4, 16):
        x = _x(M, K, "f16")
        y = _run(backend, qw, x).cpu().numpy()
        assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.float().cpu().numpy())) < TIGHT
    r = torch.from_numpy(synth.activations(34, 16, N)).cuda()
    y2 = torch.empty((16, N), dtype=torch.float32, device="cuda")
    backend.matmul_ex(qw, x, y2, "add", r)
    torch.cuda.synchronize()
    assert torch.equal(y2, torch.from_numpy(y).cuda() + r)
    # gate / up pairs of that width: eight strips (four pairs) per workgroup
    h = N // 2
    pair = backend.fuse_pairs(backend.upload_quantized(q[:h], s[:h], 4), backend.upload_quantized(q[h:], s[h:], 4))
    for M in (3, 8, 16):
        y3 = torch.empty((M, h), dtype=torch.float32, device="cuda")
        backend.matmul_ex(pair, x[:M].contiguous(), y3, "swiglu")
        torch.cuda.synchronize()
        yd = torch.from_numpy(y[:M]).cuda().double()
        ref = torch.nn.functional.silu(yd[:, :h]) * yd[:, h:]
        assert ((y3.double() - ref).norm() / ref.norm()).item() < TIGHT, M


@pytest.mark.parametrize("bits,xdt", [(4, "f16"), (4, "bf16"), (8, "f16"), (8, "bf16")])
@pytest.mark.parametrize("N", [14336, 28672, 8192])
def test_decode_batched_rows_wide_shapes(backend, oracle, bits, xdt, N):
    """Wide outputs give a workgroup of the batched-rows kernel 4, 7 or 2 strips; which shape runs
    depends on block type and activation type (register budget), and the x load pattern on the
    batch (up to 4 / 8 / 16 rows per load).  K = 384 is three K tiles: a partly filled slab."""
    K = 384
    q, s = _quant(oracle, bits, N, K, cfg=23)
    qw = backend.upload_quantized(q, s, bits)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    y1 = None
    try:
        for M in (16, 8, 5, 4):
            x = _x(16, K, xdt, cfg=24)[:M].contiguous()
            ref = x.double() @ wd.T
            backend.set_gemv_tuning(0, 0, 0)              # whichever kernel the library picks for this batch
            y = _run(backend, qw, x)
            err = ((y.double() - ref).norm() / ref.norm()).item()
            assert err < TIGHT, (M, err)
            # within the batched-rows kernel a row's bits do not depend on the batch it travels in
            # (nor on the x load pattern that follows from it)
            backend.set_gemv_tuning(0, 1, 0)
            y = _run(backend, qw, x)
            if y1 is None:
                y1 = y
            else:
                assert torch.equal(y, y1[:M]), M
    finally:
        backend.set_gemv_tuning(0, 0, 0)


@pytest.mark.parametrize("bits,xdt", [(4, "f16"), (4, "bf16"), (8, "f16"), (8, "bf16")])
@pytest.mark.parametrize("shape", [(14336, 384), (28672, 384), (8192, 384), (512, 4096 + 128), (80, 14336), (33, 160)])
def test_decode_17_to_32_rows_in_one_pass(backend, oracle, bits, xdt, shape):
    """17 .. 32 rows of 16-bit activations run the batched-rows kernel with two row blocks: the
    weights stream once.  A row's bits are those of the same kernel at 16 rows or fewer."""
    N, K = shape
    q, s = _quant(oracle, bits, N, K, cfg=27)
    qw = backend.upload_quantized(q, s, bits)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    x = _x(32, K, xdt, cfg=28)
    try:
        backend.set_gemv_tuning(0, 1, 0)                 # the batched-rows kernel for the 16-row halves too
        lo, hi = _run(backend, qw, x[:16].contiguous()), _run(backend, qw, x[16:].contiguous())
        backend.set_gemv_tuning(0, 0, 0)
        for M in (32, 17, 24):
            y = _run(backend, qw, x[:M].contiguous())
            ref = x[:M].double() @ wd.T
            err = ((y.double() - ref).norm() / ref.norm()).item()
            assert err < TIGHT, (M, err)
            assert torch.equal(y[:16], lo), M
            assert torch.equal(y[16:], hi[:M - 16]), M
    finally:
        backend.set_gemv_tuning(0, 0, 0)
    if N % 32 == 0 and K == 384:
        # epilogues in the same kernel: residual add, and SwiGLU over a gate / up pair
        M = 21
        r = torch.from_numpy(synth.activations(35, M, N)).cuda()
        y = _run(backend, qw, x[:M].contiguous())
        y2 = torch.empty((M, N), dtype=torch.float32, device="cuda")
        backend.matmul_ex(qw, x[:M].contiguous(), y2, "add", r)
        torch.cuda.synchronize()
        assert torch.equal(y2, y + r)
        h = N // 2
        g = backend.upload_quantized(q[:h], s[:h], bits)
        u = backend.upload_quantized(q[h:], s[h:], bits)
        pair = backend.fuse_pairs(g, u)
        y3 = torch.empty((M, h), dtype=torch.float32, device="cuda")
        backend.matmul_ex(pair, x[:M].contiguous(), y3, "swiglu")
        torch.cuda.synchronize()
        yd = y.double()
        ref = torch.nn.functional.silu(yd[:, :h]) * yd[:, h:]
        assert ((y3.double() - ref).norm() / ref.norm()).item() < TIGHT


@pytest.mark.parametrize("N", [8192, 12288])
def test_decode_modes_in_the_batched_rows_kernel(backend, oracle, N):
    """3 .. 32 f16 rows on outputs wide enough for two / four strips per workgroup: STREAM feeds the Q4
    weights as f16 subnormals there too (bias off through the MFMA's C operand, one bias product per K
    tile for all strips), EXACT the integer operands; both inside the tight bar, and not the same bits."""
    K = 640
    q, s = _quant(oracle, 4, N, K, cfg=29)
    qw = backend.upload_quantized(q, s, 4)
    qz = backend.upload_quantized(np.zeros((N, K), np.int8), s, 4)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    x = _x(32, K, "f16", cfg=30)
    try:
        for M in (3, 8, 16, 24, 32):
            xm = x[:M].contiguous()
            ref = xm.double() @ wd.T
            outs = {}
            for mode in ("stream", "exact"):
                backend.set_decode_mode(mode)
                y = _run(backend, qw, xm)
                err = ((y.double() - ref).norm() / ref.norm()).item()
                assert err < (TIGHT if mode == "stream" else 1e-6), (M, mode, err)
                outs[mode] = y
                z = _run(backend, qz, xm)
                if mode == "exact":
                    assert not z.any()
                else:
                    assert z.abs().max().item() < 1e-4 * ref.abs().mean().item()
            assert not torch.equal(outs["stream"], outs["exact"]), M
            # bf16 rows on the same strips: biased operands, the bias product shared by a tile's strips
            xb = _x(M, K, "bf16", cfg=31)
            yb = _run(backend, qw, xb)
            refb = xb.double() @ wd.T
            assert ((yb.double() - refb).norm() / refb.norm()).item() < TIGHT, M
            assert _run(backend, qz, xb).abs().max().item() < 1e-4 * refb.abs().mean().item()      # (the bias cancels to rounding)
    finally:
        backend.set_decode_mode("stream")


@pytest.mark.parametrize("xdt", ["f16", "bf16"])
def test_decode_long_k_split_over_workgroups(backend, oracle, xdt):
    """About one strip per CU and a long K: from twelve rows on the batched-rows kernel splits K four ways over
    workgroups, partial sums meet in slabs and the workgroup that arrives last adds them in split order.
    Ragged N (a last strip of 8 rows, a strip group of one strip) and a K whose tiles do not divide by four;
    against float64, run to run (the ticket is back at zero), across batch sizes, with the residual epilogue,
    with exact operands, and against the kernel without the split."""
    N, K = 193 * 16 - 8, 97 * 128
    q, s = _quant(oracle, 4, N, K, cfg=45)
    qw = backend.upload_quantized(q, s, 4)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    x = _x(32, K, xdt, cfg=46)
    ref = x.double() @ wd.T
    try:
        y32 = _run(backend, qw, x)
        assert ((y32.double() - ref).norm() / ref.norm()).item() < TIGHT
        for _ in range(3):
            assert torch.equal(_run(backend, qw, x), y32)
        for M in (12, 16, 17, 24):                       # one and two row blocks: a row keeps its bits
            assert torch.equal(_run(backend, qw, x[:M].contiguous()), y32[:M]), M
        backend.set_gemv_tuning(0, 4, 0)                 # the split from three rows on (the narrower x load patterns)
        for M in (3, 5, 8):
            assert torch.equal(_run(backend, qw, x[:M].contiguous()), y32[:M]), M
        backend.set_gemv_tuning(0, 3, 0)                 # never split: another order of summation, the same sums
        y_plain = _run(backend, qw, x)
        assert not torch.equal(y_plain, y32)
        assert ((y_plain.double() - y32.double()).norm() / ref.norm()).item() < 2e-6
        backend.set_gemv_tuning(0, 0, 0)
        r = torch.from_numpy(synth.activations(47, 32, N)).cuda()
        ya = torch.empty((32, N), dtype=torch.float32, device="cuda")
        backend.matmul_ex(qw, x, ya, "add", r)
        torch.cuda.synchronize()
        assert torch.equal(ya, y32 + r)
        for ydt in ("f16", "bf16"):
            assert torch.equal(_run(backend, qw, x, ydt), y32.to(TDT[ydt]))
        backend.set_decode_mode("exact")
        ye = _run(backend, qw, x[:16].contiguous())
        assert ((ye.double() - ref[:16]).norm() / ref[:16].norm()).item() < (1e-6 if xdt == "f16" else TIGHT)
        # recorded into a graph (no allocation, no memset: the ticket resets itself) and replayed
        backend.set_decode_mode("stream")
        yg = torch.zeros((32, N), dtype=torch.float32, device="cuda")
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            backend.matmul(qw, x, yg, stream=torch.cuda.current_stream().cuda_stream)
        for _ in range(3):
            yg.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(yg, y32)
            assert torch.equal(_run(backend, qw, x), y32)            # eager calls between the replays
    finally:
        backend.set_gemv_tuning(0, 0, 0)
        backend.set_decode_mode("stream")
    qw.free()


def test_decode_long_k_uses_several_slabs(backend, oracle):
    # M * K * 2 B exceeds the kernel's LDS budget: x is staged slab by slab
    N, K = 64, 14336
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    for M, xdt in ((16, "f16"), (8, "f32"), (3, "bf16")):
        x = _x(M, K, xdt)
        y = _run(backend, qw, x).cpu().numpy()
        assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.float().cpu().numpy())) < TIGHT


@pytest.mark.parametrize("bits", [4, 8])
def test_decode_every_kernel_variant(backend, oracle, bits):
    # the launch heuristics pick among one-shot (4 / 8 / 16 tiles in flight) and
    # streaming (2 / 4 tiles per batch) variants; force each of them
    N, K = 80, 4096
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits)
    try:
        for M in (1, 2, 4, 9):
            x = _x(M, K, "f16")
            ref = oracle.matmul_f64(q, s, x.float().cpu().numpy())
            for waves in (1, 2, 4, 8, 16):
                for unroll in (0, 2, 4):
                    backend.set_gemv_tuning(waves, 2, unroll)       # the LDS kernel, every variant
                    y = _run(backend, qw, x).cpu().numpy()
                    err = oracle.rel_l2(y, ref)
                    assert err < TIGHT, (M, waves, unroll, err)
                backend.set_gemv_tuning(waves, 1, 0)                # the x-in-registers kernel
                y2 = _run(backend, qw, x).cpu().numpy()
                assert oracle.rel_l2(y2, ref) < TIGHT, (M, waves)
                assert np.array_equal(y2, _run(backend, qw, x).cpu().numpy()), (M, waves)   # reproducible
    finally:
        backend.set_gemv_tuning(0, 0, 0)


def test_decode_batched_rows_equal_single_rows_bitwise(backend, oracle):
    """Within one kernel a row's bits do not depend on the batch it travels in."""
    N, K = 512, 4096
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(16, K, "f16")
    try:
        for kernel, batch in ((2, 4), (2, 16), (1, 16), (1, 7)):      # LDS kernel, x-in-registers kernel
            backend.set_gemv_tuning(0, kernel, 0)
            yb = _run(backend, qw, x[:batch].contiguous())
            for m in (0, batch // 2, batch - 1):
                y1 = _run(backend, qw, x[m:m + 1].contiguous())
                assert torch.equal(y1[0], yb[m]), (kernel, batch, m)
            assert torch.equal(_run(backend, qw, x[:batch].contiguous()), yb)     # and run to run
    finally:
        backend.set_gemv_tuning(0, 0, 0)
    # the automatic choice (LDS kernel for one or two rows, registers beyond) is deterministic too
    y16 = _run(backend, qw, x)
    assert torch.equal(_run(backend, qw, x), y16)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(64, 128), (48, 160), (100, 4096 + 96), (4096, 4096), (256, 14336), (64, 11008),
                                   (32, 16384), (16, 24576), (16, 32768)])
@pytest.mark.parametrize("xdt", ["f16", "bf16"])
def test_one_row_kernel_shapes(backend, oracle, bits, shape, xdt):
    """One and two f16 / bf16 rows (subnormal weight operands - bf16: 128 + u -, bias removed inside the accumulation; the 16
    rows of an activation operand are 1 / 2 batch rows x 16 / 8 scale groups): whole and ragged
    sets of K tiles, one to three sets per wave, and K beyond what the kernel serves (3 and 4 rows
    take the batched-rows kernel)."""
    N, K = shape
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits, formats.BLOCK_AOS if N % 32 else formats.PLANAR)
    x4 = _x(4, K, xdt, outliers=0.001)
    ref = oracle.matmul_f64(q, s, x4.float().cpu().numpy())
    for M in (1, 2, 3, 4):
        x = x4[:M].contiguous()
        y = _run(backend, qw, x)
        assert oracle.rel_l2(y.cpu().numpy(), ref[:M]) < TIGHT, M
        assert torch.equal(_run(backend, qw, x), y)                 # reproducible
        for ydt in ("f16", "bf16"):
            assert torch.equal(_run(backend, qw, x, ydt), y.to(TDT[ydt]))
        # fused epilogues of the same kernel: residual add, and SwiGLU where the rows pair up
        r = torch.from_numpy(synth.activations(36, M, N)).cuda()
        y2 = torch.empty((M, N), dtype=torch.float32, device="cuda")
        backend.matmul_ex(qw, x, y2, "add", r)
        torch.cuda.synchronize()
        assert torch.equal(y2, y + r), M
    if N % 32 == 0 and N >= 64:
        h = N // 2
        pair = backend.fuse_pairs(backend.upload_quantized(q[:h], s[:h], bits), backend.upload_quantized(q[h:], s[h:], bits))
        for M in (1, 2, 4):
            y3 = torch.empty((M, h), dtype=torch.float32, device="cuda")
            backend.matmul_ex(pair, x4[:M].contiguous(), y3, "swiglu")
            torch.cuda.synchronize()
            rd = torch.from_numpy(ref[:M]).cuda()
            want = torch.nn.functional.silu(rd[:, :h]) * rd[:, h:]
            assert ((y3.double() - want).norm() / want.norm()).item() < TIGHT, M


@pytest.mark.parametrize("bits", [4, 8])
def test_decode_modes(backend, oracle, bits):
    """STREAM (default) and EXACT weight operands for one f16 row: both inside the tight bar;
    EXACT returns exact zeros for a tensor of zeros."""
    N, K = 320, 4096
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits)
    qz = backend.upload_quantized(np.zeros((N, K), np.int8), s, bits)
    x = _x(1, K, "f16")
    ref = oracle.matmul_f64(q, s, x.float().cpu().numpy())
    scale = float(np.abs(ref).mean())
    try:
        errs = {}
        for mode in ("stream", "exact"):
            backend.set_decode_mode(mode)
            errs[mode] = oracle.rel_l2(_run(backend, qw, x).cpu().numpy(), ref)
            assert errs[mode] < TIGHT, (mode, errs)
            z = _run(backend, qz, x).cpu().numpy()
            if mode == "exact":
                assert not z.any()
            else:
                assert np.abs(z).max() < 1e-4 * scale       # the bias cancels to rounding, not to the bit
        assert errs["exact"] < 1e-6
    finally:
        backend.set_decode_mode("stream")
    with pytest.raises(CybqError):
        backend.set_decode_mode("loose")


def test_decode_lds_kernel_largest_request(backend, oracle):
    """fp32 activations, 10..16 rows, K long enough for 16 waves: the slab of x is one tile per
    wave whatever the budget says (up to 146 KB of LDS); and exact-mode fp32 prefill walks it."""
    K = 14336
    for N in (64, 4096):
        q, s = _quant(oracle, 4, N, K)
        qw = backend.upload_quantized(q, s, 4)
        for M in (12, 16):
            x = _x(M, K, "f32")
            y = _run(backend, qw, x).cpu().numpy()
            assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.cpu().numpy())) < TIGHT, (N, M)
    backend.set_prefill_mode("exact")
    try:
        x = _x(40, K, "f32")
        y = _run(backend, qw, x).cpu().numpy()
        assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.cpu().numpy())) < TIGHT
    finally:
        backend.set_prefill_mode("fast")


def test_known_answers_from_the_committed_fixture(backend):
    """tests/golden/matmul_small.json through the C ABI: both interchange layouts, f16 activations."""
    from tests.test_oracle_matmul import _golden_cases
    for name, bits, q, s, x, want in _golden_cases():
        for layout in (formats.PLANAR, formats.BLOCK_AOS):
            qw = backend.upload_quantized(q, s, bits, layout)
            xt = torch.from_numpy(x).cuda().to(torch.float16)
            y = _run(backend, qw, xt).double().cpu().numpy()
            assert np.linalg.norm(y - want) <= TIGHT * np.linalg.norm(want), (name, layout)
            if name == "by_hand_q4":
                assert np.allclose(y, [[16.0, 32.0, 48.0, 64.0]], rtol=1e-6)


def test_decode_special_cases(backend, oracle):
    N, K = 64, 256
    ones = np.full((N, K // 32), 0x3C00, np.uint16)
    # q = 0 -> 0 ; q = 1, d = 1 -> row sums of x
    qw0 = backend.upload_quantized(np.zeros((N, K), np.int8), ones, 4)
    x = _x(4, K, "f16")
    assert not _run(backend, qw0, x).any()
    qw1 = backend.upload_quantized(np.ones((N, K), np.int8), ones, 4)
    y = _run(backend, qw1, x).cpu().numpy()
    want = x.double().sum(dim=1).cpu().numpy()
    assert np.allclose(y, np.repeat(want[:, None], N, axis=1), rtol=1e-5, atol=1e-4)
    # one-hot x picks a dequantised column exactly
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    wd = oracle.dequant(q, s)
    for k in (0, 7, 8, 31, 32, 255):
        e = torch.zeros((1, K), dtype=torch.float16, device="cuda")
        e[0, k] = 1.0
        assert np.array_equal(_run(backend, qw, e).cpu().numpy()[0], wd[:, k])
    # extreme weights: every nibble value in every slot position
    qe = np.resize(np.arange(-8, 8), (N, K)).astype(np.int8)
    qe[1::2] = qe[1::2, ::-1]
    qwe = backend.upload_quantized(qe, s, 4)
    xe = _x(2, K, "f16")
    assert oracle.rel_l2(_run(backend, qwe, xe).cpu().numpy(),
                         oracle.matmul_f64(qe, s, xe.float().cpu().numpy())) < TIGHT


@pytest.mark.parametrize("ydt", ["f16", "bf16"])
def test_output_dtypes_round_once(backend, oracle, ydt):
    N, K = 128, 512
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    for M in (2, 40):
        x = _x(M, K, "bf16" if M > 16 else "f16")
        y32 = _run(backend, qw, x)
        y16 = _run(backend, qw, x, ydt)
        assert torch.equal(y16, y32.to(TDT[ydt]))


def test_config1_q8_fp32_activations(backend, oracle):
    q, s = _quant(oracle, 8, 2048, 2048, cfg=1)
    qw = backend.upload_quantized(q, s, 8, formats.BLOCK_AOS)
    x = _x(1, 2048, "f32", cfg=1)
    y = _run(backend, qw, x).cpu().numpy()
    assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.cpu().numpy())) < TIGHT


@pytest.mark.parametrize("shape", [(4096, 4096), (4096, 1024), (4096, 14336), (14336, 4096)])
def test_config2_and_3_full_size(backend, oracle, shape):
    K, N = shape
    q, s = _quant(oracle, 4, N, K, cfg=2)
    qw = backend.upload_quantized(q, s, 4)
    assert qw.algorithmic_bytes == formats.weight_bytes(4, N, K)
    for M in (1, 4, 8, 16):
        x = _x(M, K, "f16", cfg=3, outliers=0.001)
        y = _run(backend, qw, x).cpu().numpy()
        ref = oracle.matmul_f64(q, s, x[: min(M, 2)].float().cpu().numpy())
        assert oracle.rel_l2(y[: min(M, 2)], ref) < TIGHT
        # remaining rows: float64 library matmul on the dequantised weights
        full = x.double().cpu().numpy() @ oracle.dequant(q, s).astype(np.float64).T
        assert oracle.rel_l2(y, full) < TIGHT


# ------------------------------------------------------------ prefill (M > 16)

@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("xdt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("M", [17, 64, 300])
def test_prefill_matches_oracle(backend, oracle, prefill_mode, bits, xdt, M):
    N, K = 240, 512
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits)
    x = _x(M, K, xdt)
    y = _run(backend, qw, x).cpu().numpy()
    assert not np.isnan(y).any()
    err = oracle.rel_l2(y, oracle.matmul_f64(q, s, x.float().cpu().numpy()))
    # fp32 activations: exact through the decode kernel's hi/lo split up to 32 rows and in EXACT mode;
    # FAST prefill rounds them to f16 in the staging pass like any other
    exact_path = M <= (16 if xdt == "f32" else 32) or prefill_mode == "exact"
    assert err < (TIGHT if (xdt == "f32" and exact_path) else _bar(prefill_mode)), err
    if prefill_mode == "fast" and M > (16 if xdt == "f32" else 64):
        # the rounded-weight kernel really ran (up to 32 rows of 16-bit activations take the exact decode
        # kernel, and up to 64 on a weight as small as this one)
        assert err > 1e-6


@pytest.mark.parametrize("shape", [(17, 32), (112, 160), (113, 96), (130, 2080)])
def test_prefill_ragged_shapes(backend, oracle, prefill_mode, shape):
    N, K = shape
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    for M in (17, 257):
        x = _x(M, K, "bf16")
        y = _run(backend, qw, x).cpu().numpy()
        assert not np.isnan(y).any()
        assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.float().cpu().numpy())) < _bar(prefill_mode)


@pytest.mark.parametrize("xdt", ["bf16", "f32"])
def test_prefill_fast_mode_activation_range(backend, oracle, xdt):
    # FAST turns bf16 / fp32 activations into f16 operands behind a power-of-two scale per row:
    # rows of any magnitude keep the mode's accuracy, outliers far beyond f16's range survive
    N, K = 128, 1024
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(40, K, xdt)
    x[0, 5] = 3.0e5
    x[1, 77] = -9.0e5
    x[2] *= 1e-3
    x[3] *= 300.0
    x[4] *= 1e-4
    x[5] *= 1e-5
    x[6] *= 1e-6
    x[7] *= 1e-12
    x[8] *= 1e12
    x[9] = 0.0
    x[10, 1:] = 0.0
    x[11] *= 1e-36                 # largest magnitude below 2^-113: the row's power of two stops at 2^126
    if xdt == "f32":               # a row of fp32 subnormals (made on the host: bit patterns, not device arithmetic)
        x[12] = torch.from_numpy(synth.activations(21, 40, K)[12] * np.float32(1e-40)).cuda()
    backend.set_prefill_mode("fast")
    y = _run(backend, qw, x).cpu().numpy()
    assert np.isfinite(y).all()
    assert not y[9].any()
    ref = oracle.matmul_f64(q, s, x.float().cpu().numpy())
    for rows in ([0], [1], [2], [3], [4], [5], [6], [7], [8], [10], [11], list(range(13, 40))):
        assert oracle.rel_l2(y[rows], ref[rows]) < FAST, rows
    # (the subnormal row: its operands keep what f16 holds below 2^126 times the row, and the result is itself
    # an fp32 subnormal - finite, and as close as those two allow; with bf16 it is an ordinary row)
    assert oracle.rel_l2(y[[12]], ref[[12]]) < (2e-2 if xdt == "f32" else FAST)
    # a folded norm sees the same rows (gamma of mixed magnitudes)
    gamma = torch.from_numpy(np.abs(synth.activations(22, 1, K))[0] * 10.0 + 1e-3).cuda()
    yn = torch.empty((40, N), dtype=torch.float32, device="cuda")
    backend.matmul_norm(qw, x, gamma, 1e-30, yn)           # 40 rows: the prefill kernel
    torch.cuda.synchronize()
    xf = x[:9].double().cpu().numpy()
    rstd = 1.0 / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-30)
    refn = oracle.matmul_f64(q, s, (xf * gamma.double().cpu().numpy()).astype(np.float32)) * rstd
    for r in range(9):
        assert oracle.rel_l2(yn[r:r + 1].cpu().numpy(), refn[r:r + 1]) < 2 * FAST, r


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("xdt", ["f16", "bf16", "f32"])
def test_scales_beyond_f16_products(backend, oracle, bits, xdt):
    """scale * q would leave f16's range: such tensors take the decode kernels (scale in fp32) on both
    sides of the prefill boundary - whether the handle was built from host buffers (scanned on the host)
    or from device buffers (scanned by the repack kernel)."""
    N, K = 64, 256
    q, s = _quant(oracle, bits, N, K)
    s = s.copy()
    s[::3, ::2] = np.float16(30000.0).view(np.uint16)
    qd = torch.from_numpy(formats.pack_planar(q, bits)).cuda()
    sd = torch.from_numpy(s.view(np.int16)).cuda()
    handles = [backend.upload_quantized(q, s, bits, formats.BLOCK_AOS), backend.weight_from_device(bits, N, K, qd, sd)]
    for qw in handles:
        for M in (4, 32, 33, 100):
            x = _x(M, K, xdt)
            y = _run(backend, qw, x).cpu().numpy()
            assert np.isfinite(y).all(), M
            assert oracle.rel_l2(y, oracle.matmul_f64(q, s, x.float().cpu().numpy())) < TIGHT, M
    # pairs built from a wide tensor stay wide
    if bits == 4:
        pair = backend.fuse_pairs(handles[1], handles[1])
        x = _x(40, K, "f16")
        y = torch.empty((40, N), dtype=torch.float32, device="cuda")
        backend.matmul_ex(pair, x, y, "swiglu")
        torch.cuda.synchronize()
        assert torch.isfinite(y).all()
        pair.free()
    for qw in handles:
        qw.free()


def test_prefill_rows_agree_with_decode_rows(backend, oracle, prefill_mode):
    N, K = 448, 1024
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(64, K, "bf16")
    yp = _run(backend, qw, x)
    yd = _run(backend, qw, x[:16].contiguous())
    num = (yp[:16] - yd).double().norm() / yd.double().norm()
    assert num.item() < _bar(prefill_mode)
    assert torch.equal(_run(backend, qw, x), yp)            # deterministic


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(200, 4352), (37, 8192 + 96), (500, 2048)])
def test_prefill_few_tiles_split_k(backend, oracle, prefill_mode, bits, shape):
    # fewer output tiles than CUs and a long K: the K range is split over workgroups
    # (K tiles not divisible by the split, ragged N and M) and the partial sums are
    # added by a second kernel, which also does the output conversion
    N, K = shape
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits)
    for M in (17, 130, 300):
        x = _x(M, K, "bf16")
        y = _run(backend, qw, x)
        assert not torch.isnan(y).any()
        err = oracle.rel_l2(y.cpu().numpy(), oracle.matmul_f64(q, s, x.float().cpu().numpy()))
        assert err < _bar(prefill_mode), (M, err)
        assert torch.equal(_run(backend, qw, x), y)                       # fixed summation order
        for ydt in ("f16", "bf16"):
            assert torch.equal(_run(backend, qw, x, ydt), y.to(TDT[ydt]))   # rounded once


def test_prefill_more_rows_than_the_stage_holds(backend, oracle, prefill_mode):
    # 4200 x 16384 activations are 131 MiB: they pass through the 128 MiB staging area
    # in two row chunks
    N, K, M = 48, 16384, 4200
    q, s = _quant(oracle, 4, N, K)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(M, K, "bf16")
    y = _run(backend, qw, x)
    assert not torch.isnan(y).any()
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    full = x.double() @ wd.T
    for lo, hi in ((0, 1000), (3900, 4096), (4096, M)):                     # rows of both chunks
        err = ((y[lo:hi].double() - full[lo:hi]).norm() / full[lo:hi].norm()).item()
        assert err < _bar(prefill_mode), (lo, err)
    rows = [0, 4095, 4096, M - 1]
    ref = oracle.matmul_f64(q, s, x[rows].float().cpu().numpy())
    assert oracle.rel_l2(y[rows].cpu().numpy(), ref) < _bar(prefill_mode)


@pytest.mark.parametrize("M", [128, 512, 2048])
@pytest.mark.parametrize("shape", [(4096, 14336), (14336, 4096)])
def test_config4_full_size(backend, oracle, prefill_mode, M, shape):
    K, N = shape
    q, s = _quant(oracle, 4, N, K, cfg=4)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(M, K, "bf16", cfg=4)
    y = _run(backend, qw, x)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    full = (x.double() @ wd.T)
    err = ((y.double() - full).norm() / full.norm()).item()
    assert err < _bar(prefill_mode), err
    # the oracle itself on a few rows
    rows = [0, M // 2, M - 1]
    ref = oracle.matmul_f64(q, s, x[rows].float().cpu().numpy())
    assert oracle.rel_l2(y[rows].cpu().numpy(), ref) < _bar(prefill_mode)
    # linearity in x: f(2x) == 2 f(x) exactly (powers of two commute with every rounding)
    if prefill_mode == "exact":
        y2 = _run(backend, qw, (x * 2).contiguous())
        assert torch.equal(y2, y * 2)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("xdt", ["f16", "bf16"])
def test_prefill_512_row_workgroups(backend, oracle, bits, xdt):
    """FAST mode, N a multiple of 112 and enough rows for 512-row workgroups to fill the chip: a wave
    multiplies four row blocks per weight operand.  Row counts that are whole tiles, leave a last
    tile more than half full, or fall back to 256-row tiles; residual add and folded RMSNorm ride along."""
    N, K = 14336, 384
    q, s = _quant(oracle, bits, N, K, cfg=41)
    qw = backend.upload_quantized(q, s, bits)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    for M in (1024, 1300, 1100):
        x = _x(M, K, xdt, cfg=42)
        y = _run(backend, qw, x)
        ref = x.double() @ wd.T
        assert ((y.double() - ref).norm() / ref.norm()).item() < FAST, M
        assert torch.equal(_run(backend, qw, x), y)                 # reproducible
        # a row's bits depend neither on its place in a workgroup's tile nor on the tile shape
        # (600 rows run as 256-row tiles)
        assert torch.equal(_run(backend, qw, x[M - 600:].contiguous()), y[M - 600:]), M
    M = 1024
    x = _x(M, K, xdt, cfg=42)
    r = torch.from_numpy(synth.activations(43, M, N)).cuda()
    y2 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    backend.matmul_ex(qw, x, y2, "add", r)
    torch.cuda.synchronize()
    assert torch.equal(y2, _run(backend, qw, x) + r)
    gamma = (1.0 + 0.1 * torch.from_numpy(synth.activations(44, 1, K))[0]).cuda()
    y3 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    backend.matmul_norm(qw, x, gamma, 1e-5, y3)
    torch.cuda.synchronize()
    xd = x.double()
    xn = xd * torch.rsqrt((xd * xd).mean(dim=1, keepdim=True) + 1e-5) * gamma.double()
    ref = xn @ wd.T
    assert ((y3.double() - ref).norm() / ref.norm()).item() < 2 * FAST


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(14336, 384, 512), (4096, 384, 2048), (6144, 160, 1100), (14336, 384, 100), (28672, 160, 128),
                                   (14344, 160, 520), (14342, 96, 515),
                                   (4096, 416, 512), (6144, 160, 500), (8000, 96, 512), (4096, 160, 200), (6150, 96, 250),
                                   (8000, 96, 230), (8704, 96, 192), (3840, 96, 320), (4096, 160, 64), (14336, 288, 50)])
def test_prefill_role_split_kernel(backend, oracle, bits, shape):
    """FAST mode with enough 256-row tiles to fill the chip: some waves of a workgroup only multiply,
    the others only fetch and dequantise weights.  Seven and eight column blocks per tile, a ragged
    last row tile, every activation and output type, residual add and folded RMSNorm.  The last two
    shapes: up to 128 rows on a wide output run 128 x 64 tiles without a K split (role-split for one
    round of tiles, the plain kernel for more); then N that ends inside a column block, with rows of y
    that are 16-byte aligned and rows that are not (element-wise stores).  From (4096, 416, 512) on:
    narrow outputs with a short K in one round of 128-row or 64-row tiles that are 4, 6 and 8 column
    blocks wide (K of 3.25 and 2.25 tiles: a remainder behind the whole rounds of the K loops), then
    two decode passes over 64 rows of a small weight and the 64-row tiles of a wide output."""
    N, K, M = shape
    q, s = _quant(oracle, bits, N, K, cfg=45)
    qw = backend.upload_quantized(q, s, bits)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    r = torch.from_numpy(synth.activations(47, M, N)).cuda()
    for xdt, ydt in (("bf16", "f32"), ("f16", "bf16"), ("f32", "f16")):
        x = _x(M, K, xdt, cfg=46)
        ref = x.double() @ wd.T
        y = _run(backend, qw, x, ydt)
        bar = FAST if ydt == "f32" else 4e-3            # (a 16-bit output rounds every element once more)
        assert ((y.double() - ref).norm() / ref.norm()).item() < bar, (xdt, ydt)
        assert torch.equal(_run(backend, qw, x, ydt), y)             # reproducible
        y2 = torch.empty((M, N), dtype=TDT[ydt], device="cuda")
        backend.matmul_ex(qw, x, y2, "add", r.to(TDT[ydt]))
        torch.cuda.synchronize()
        want = ref + r.to(TDT[ydt]).double()
        assert ((y2.double() - want).norm() / want.norm()).item() < bar, (xdt, ydt)
    x = _x(M, K, "bf16", cfg=46)
    gamma = (1.0 + 0.1 * torch.from_numpy(synth.activations(48, 1, K))[0]).cuda()
    y3 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    backend.matmul_norm(qw, x, gamma, 1e-5, y3)
    torch.cuda.synchronize()
    xd = x.double()
    ref = (xd * torch.rsqrt((xd * xd).mean(dim=1, keepdim=True) + 1e-5) * gamma.double()) @ wd.T
    assert ((y3.double() - ref).norm() / ref.norm()).item() < 2 * FAST


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(14336, 2048, 64), (8200, 4096 + 128, 33), (8198, 4096 + 256, 47), (14336, 4096, 48),
                                   (28672, 2048, 40), (8192, 8192, 64),
                                   (4096, 4096, 128), (6144 - 16, 4096 + 128, 100), (1024, 4096, 512), (2048, 4096, 300),
                                   (4102, 8192, 70), (8192, 2048, 65),
                                   (1024, 4096 + 128, 60), (4096, 4096, 64), (1030, 2048, 130)])
def test_prefill_few_rows_waves_split_k(backend, oracle, bits, shape):
    """FAST mode, K of 16 .. 64 tiles, one round of workgroups that is at least a quarter full: the kernel whose
    four waves split K and share nothing until the end (no LDS on the way, one partial-sum exchange).  33 .. 64
    rows on outputs from 8192 columns (more than a round of workgroups on the widest); from (4096, 4096, 128)
    on, narrow outputs with up to 512 rows: one to eight workgroups of 64 rows per column group, one, two or
    four column blocks wide (the last three shapes: one), a ragged last row part.  K tile counts that do not
    divide by four (waves with unequal shares), N that ends inside a column block with rows of y aligned and
    not, every activation and output type, residual add, folded RMSNorm; the other kernels (the same call with
    this kernel switched off: the tiled ones, or two decode passes on a small weight at up to 64 rows) agree
    within the mode's tolerance; a row's bits do not depend on the rows it travels with; reproducible."""
    N, K, M = shape
    q, s = _quant(oracle, bits, N, K, cfg=61)
    qw = backend.upload_quantized(q, s, bits)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    r = torch.from_numpy(synth.activations(63, M, N)).cuda()
    try:
        for xdt, ydt in (("bf16", "f32"), ("f16", "bf16"), ("f32", "f16"), ("f16", "f32")):
            x = _x(M, K, xdt, cfg=62)
            ref = x.double() @ wd.T
            y = _run(backend, qw, x, ydt)
            bar = FAST if ydt == "f32" else 4e-3            # (a 16-bit output rounds every element once more)
            assert ((y.double() - ref).norm() / ref.norm()).item() < bar, (xdt, ydt)
            assert torch.equal(_run(backend, qw, x, ydt), y)             # reproducible
            backend.set_gemm_tuning(2)                                     # the tiled kernels on the same call
            y_tiled = _run(backend, qw, x, ydt)
            backend.set_gemm_tuning(0)
            assert ((y.double() - y_tiled.double()).norm() / ref.norm()).item() < 2 * bar, (xdt, ydt)
            if ydt == "f32":
                assert not torch.equal(y, y_tiled)                         # (another order of summation: it did run)
            y2 = torch.empty((M, N), dtype=TDT[ydt], device="cuda")
            backend.matmul_ex(qw, x, y2, "add", r.to(TDT[ydt]))
            torch.cuda.synchronize()
            want = ref + r.to(TDT[ydt]).double()
            assert ((y2.double() - want).norm() / want.norm()).item() < bar, (xdt, ydt)
        parts = (M + 63) // 64                      # fewer rows, the same number of 64-row parts: the same kernel shape
        fewer = 64 * (parts - 1) + 37
        x = _x(64 * parts, K, "f16", cfg=62)
        y_all = _run(backend, qw, x)
        y_fewer = _run(backend, qw, x[:fewer].contiguous())
        assert torch.equal(y_all[:fewer], y_fewer)
        x = _x(M, K, "bf16", cfg=62)
        gamma = (1.0 + 0.1 * torch.from_numpy(synth.activations(64, 1, K))[0]).cuda()
        y3 = torch.empty((M, N), dtype=torch.float32, device="cuda")
        backend.matmul_norm(qw, x, gamma, 1e-5, y3)
        torch.cuda.synchronize()
        xd = x.double()
        ref = (xd * torch.rsqrt((xd * xd).mean(dim=1, keepdim=True) + 1e-5) * gamma.double()) @ wd.T
        assert ((y3.double() - ref).norm() / ref.norm()).item() < 2 * FAST
    finally:
        backend.set_gemm_tuning(0)
    qw.free()


@pytest.mark.parametrize("shape", [(14336, 4096, 17), (4096, 4096, 32), (8200, 2048 + 128, 24)])
def test_prefill_fp32_rows_17_to_32_fast_mode(backend, oracle, shape):
    """fp32 activations leave the decode kernels at 17 rows; in FAST mode they are rounded to f16 by the staging
    pass and, where the shape fits, multiplied by the kernel whose waves split K (a 64-row workgroup mostly
    empty).  Against float64, against the tiled kernels, residual add, reproducible."""
    N, K, M = shape
    q, s = _quant(oracle, 4, N, K, cfg=65)
    qw = backend.upload_quantized(q, s, 4)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    x = _x(M, K, "f32", cfg=66)
    ref = x.double() @ wd.T
    try:
        y = _run(backend, qw, x)
        assert ((y.double() - ref).norm() / ref.norm()).item() < FAST
        assert torch.equal(_run(backend, qw, x), y)
        backend.set_gemm_tuning(2)
        y_tiled = _run(backend, qw, x)
        backend.set_gemm_tuning(0)
        assert ((y.double() - y_tiled.double()).norm() / ref.norm()).item() < 2 * FAST
        assert not torch.equal(y, y_tiled)                                 # (another order of summation: it did run)
        r = torch.from_numpy(synth.activations(67, M, N)).cuda()
        y2 = torch.empty((M, N), dtype=torch.float32, device="cuda")
        backend.matmul_ex(qw, x, y2, "add", r)
        torch.cuda.synchronize()
        assert ((y2.double() - (ref + r.double())).norm() / (ref + r.double()).norm()).item() < FAST
    finally:
        backend.set_gemm_tuning(0)
    qw.free()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(7168, 4096, 48, "bf16"), (2048, 4096 + 128, 100, "f16"), (14336, 2048, 33, "bf16"),
                                   (1040, 4096, 24, "f32"), (4096, 2048, 64, "bf16")])
def test_prefill_few_rows_swiglu(backend, oracle, bits, shape):
    """The SwiGLU epilogue of the kernel whose waves split K (FAST mode): a workgroup holds gate / up column blocks
    in pairs and the wave that finishes a row block writes silu(gate) * up.  One workgroup per 64 rows, two row
    parts, more than one round of workgroups, fp32 rows below 33, with a folded RMSNorm; against float64 and
    against the tiled kernels on the same call."""
    N, K, M, xdt = shape
    qg, sg = _quant(oracle, bits, N, K, cfg=81)
    qu, su = _quant(oracle, bits, N, K, cfg=82)
    wg, wu = backend.upload_quantized(qg, sg, bits), backend.upload_quantized(qu, su, bits)
    wf = backend.fuse_pairs(wg, wu)
    dg = torch.from_numpy(oracle.dequant(qg, sg)).cuda().double()
    du = torch.from_numpy(oracle.dequant(qu, su)).cuda().double()
    try:
        for ydt in ("f32", "bf16"):
            x = _x(M, K, xdt, cfg=83)
            g, u = x.double() @ dg.T, x.double() @ du.T
            ref = g / (1.0 + torch.exp(-g)) * u
            bar = 2 * FAST if ydt == "f32" else 6e-3
            y = torch.full((M, N), float("nan"), dtype=TDT[ydt], device="cuda")
            backend.matmul_ex(wf, x, y, "swiglu")
            y_again = torch.empty_like(y)
            backend.matmul_ex(wf, x, y_again, "swiglu")
            backend.set_gemm_tuning(2)
            y_tiled = torch.empty_like(y)
            backend.matmul_ex(wf, x, y_tiled, "swiglu")
            backend.set_gemm_tuning(0)
            torch.cuda.synchronize()
            assert not torch.isnan(y.float()).any()
            assert ((y.double() - ref).norm() / ref.norm()).item() < bar, ydt
            assert torch.equal(y, y_again)
            assert ((y.double() - y_tiled.double()).norm() / ref.norm()).item() < 2 * bar, ydt
            if ydt == "f32":
                assert not torch.equal(y, y_tiled)                         # (another kernel: it did run)
        x = _x(M, K, "bf16", cfg=84)
        gamma = (1.0 + 0.1 * torch.from_numpy(synth.activations(85, 1, K))[0]).cuda()
        xd = x.double()
        xn = xd * torch.rsqrt((xd * xd).mean(dim=1, keepdim=True) + 1e-5) * gamma.double()
        g, u = xn @ dg.T, xn @ du.T
        ref = g / (1.0 + torch.exp(-g)) * u
        y = torch.empty((M, N), dtype=torch.float32, device="cuda")
        backend.matmul_norm(wf, x, gamma, 1e-5, y, "swiglu")
        torch.cuda.synchronize()
        assert ((y.double() - ref).norm() / ref.norm()).item() < 4 * FAST
    finally:
        backend.set_gemm_tuning(0)
    for t in (wf, wg, wu):
        t.free()


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("shape", [(14336, 4096, 32), (2064, 2048 + 128, 17), (4096, 8192, 25)])
def test_folded_norm_17_to_32_rows_fast_mode(backend, oracle, bits, shape):
    """17 .. 32 rows of 16-bit activations with a folded RMSNorm leave the one-pass decode kernel; in FAST mode,
    where the shape fits, the staging pass folds gamma in and the kernel whose waves split K multiplies (two row
    blocks per workgroup).  Against float64, against the two decode passes that take the call otherwise, with a
    residual add, 16-bit outputs; reproducible; a row's bits do not depend on the rows it travels with."""
    N, K, M = shape
    q, s = _quant(oracle, bits, N, K, cfg=71)
    qw = backend.upload_quantized(q, s, bits)
    wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
    r = torch.from_numpy(synth.activations(73, M, N)).cuda()
    try:
        for xdt, gdt, ydt in (("bf16", torch.float16, "f32"), ("f16", torch.float32, "bf16"), ("bf16", torch.bfloat16, "f16")):
            x = _x(M, K, xdt, cfg=72)
            gamma = (1.0 + 0.1 * torch.from_numpy(synth.activations(74, 1, K))[0]).cuda().to(gdt)
            xd = x.double()
            ref = (xd * torch.rsqrt((xd * xd).mean(dim=1, keepdim=True) + 1e-5) * gamma.double()) @ wd.T
            bar = 2 * FAST if ydt == "f32" else 4e-3
            y = torch.empty((M, N), dtype=TDT[ydt], device="cuda")
            backend.matmul_norm(qw, x, gamma, 1e-5, y)
            torch.cuda.synchronize()
            assert ((y.double() - ref).norm() / ref.norm()).item() < bar, (xdt, ydt)
            y_again = torch.empty_like(y)
            backend.matmul_norm(qw, x, gamma, 1e-5, y_again)
            backend.set_gemm_tuning(2)                                     # two passes of the batched-rows decode kernel
            y_two = torch.empty_like(y)
            backend.matmul_norm(qw, x, gamma, 1e-5, y_two)
            backend.set_gemm_tuning(0)
            fewer = torch.empty((17, N), dtype=TDT[ydt], device="cuda")
            backend.matmul_norm(qw, x[:17].contiguous(), gamma, 1e-5, fewer)
            y_add = torch.empty_like(y)
            backend.matmul_norm(qw, x, gamma, 1e-5, y_add, epilogue="add", residual=r.to(TDT[ydt]))
            torch.cuda.synchronize()
            assert torch.equal(y, y_again)
            assert ((y.double() - y_two.double()).norm() / ref.norm()).item() < 2 * bar, (xdt, ydt)
            if ydt == "f32":
                assert not torch.equal(y, y_two)                           # (rounded operands, another order: it did run)
            assert torch.equal(y[:17], fewer)
            want = ref + r.to(TDT[ydt]).double()
            assert ((y_add.double() - want).norm() / want.norm()).item() < bar, (xdt, ydt)
    finally:
        backend.set_gemm_tuning(0)
    qw.free()


def test_lm_head_shape(backend, oracle):
    """The LM head of a Llama-3-sized vocabulary (decide/pipeline.md:51): 128256 rows, K = 4096, Q4 -
    8016 strips, several rounds of workgroups per CU.  Weights are made and quantised on the device;
    every output is checked against a float64 product over the exactly dequantised tensor (chunks of
    rows), a sample of rows against the oracle from the packed bytes."""
    N, K, bits = 128256, 4096, 4
    gen = torch.Generator(device="cuda")
    gen.manual_seed(1234)
    w = torch.empty((N, K), dtype=torch.float32, device="cuda").normal_(0.0, 0.02, generator=gen)
    qd = torch.empty(N * K // 2, dtype=torch.uint8, device="cuda")
    sd = torch.empty(N * (K // 32), dtype=torch.int16, device="cuda")
    backend.quantize(bits, w, N, K, qd, sd)
    qw = backend.weight_from_device(bits, N, K, qd, sd)
    torch.cuda.synchronize()
    backend.dequant(qw, w)                       # w now holds scale * q, bit-exact (tested elsewhere)
    torch.cuda.synchronize()
    rows = torch.arange(0, N, 997, device="cuda")
    qrows = formats.unpack_planar(qd.view(N, K // 2)[rows].cpu().numpy().reshape(-1), bits, len(rows), K)
    srows = sd.view(N, K // 32)[rows].cpu().numpy().view(np.uint16)
    assert np.array_equal(oracle.dequant(qrows, srows), w[rows].cpu().numpy())
    for M, xdt in ((1, "f16"), (2, "f16"), (8, "f16"), (8, "bf16"), (20, "f16")):
        x = _x(M, K, xdt, cfg=51)
        y = _run(backend, qw, x)
        xd = x.double()
        num = den = 0.0
        for r0 in range(0, N, 16032):
            ref = xd @ w[r0:r0 + 16032].double().T
            num += ((y[:, r0:r0 + 16032].double() - ref) ** 2).sum().item()
            den += (ref ** 2).sum().item()
        assert (num / den) ** 0.5 < TIGHT, (M, xdt)
        ref = oracle.matmul_f64(qrows, srows, x.float().cpu().numpy())
        assert oracle.rel_l2(y[:, rows].cpu().numpy(), ref) < TIGHT, (M, xdt)


# ------------------------------------------------------- fused epilogues
# The reference's definitions of the ops around a linear are not in its tree (parity
# unpinned); the checks below pin the library's stated formulas: y = r + x W^T, and
# y = silu(x Wg^T) * (x Wu^T) with silu(t) = t / (1 + exp(-t)), against float64.

def _silu_mul(g, u):
    return g / (1.0 + np.exp(-g)) * u


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,xdt", [(1, "f16"), (2, "bf16"), (3, "f32"), (4, "f16"), (16, "bf16"), (40, "bf16"), (300, "f16")])
def test_epilogue_residual_add(backend, oracle, prefill_mode, bits, M, xdt):
    N, K = 272, 1024
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits)
    x = _x(M, K, xdt)
    r = torch.from_numpy(synth.activations(33, M, N)).cuda()
    ref = oracle.matmul_f64(q, s, x.float().cpu().numpy()) + r.double().cpu().numpy()
    y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    backend.matmul_ex(qw, x, y, "add", r)
    torch.cuda.synchronize()
    bar = TIGHT if (M <= 16 or xdt == "f32") else _bar(prefill_mode)
    assert oracle.rel_l2(y.cpu().numpy(), ref) < bar
    # in place (residual aliases y) and with a 16-bit residual stream: added in fp32, rounded once
    y2 = r.clone()
    backend.matmul_ex(qw, x, y2, "add", y2)
    torch.cuda.synchronize()
    assert torch.equal(y2, y)
    rb = r.to(torch.bfloat16)
    yb = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    backend.matmul_ex(qw, x, yb, "add", rb)
    y32 = torch.empty((M, N), dtype=torch.float32, device="cuda")
    backend.matmul(qw, x, y32)
    torch.cuda.synchronize()
    assert torch.equal(yb, (y32 + rb.float()).to(torch.bfloat16))


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,xdt", [(1, "f16"), (2, "bf16"), (3, "f32"), (4, "f16"), (9, "f16"), (16, "bf16"), (40, "bf16"), (300, "f16")])
def test_epilogue_swiglu(backend, oracle, prefill_mode, bits, M, xdt):
    N, K = 336, 1024                      # 21 strips per projection
    qg, sg = _quant(oracle, bits, N, K, cfg=41)
    qu, su = _quant(oracle, bits, N, K, cfg=42)
    wg = backend.upload_quantized(qg, sg, bits)
    wu = backend.upload_quantized(qu, su, bits)
    wf = backend.fuse_pairs(wg, wu)
    assert (wf.N, wf.K) == (2 * N, K)
    x = _x(M, K, xdt)
    xf = x.float().cpu().numpy()
    g, u = oracle.matmul_f64(qg, sg, xf), oracle.matmul_f64(qu, su, xf)
    y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    backend.matmul_ex(wf, x, y, "swiglu")
    torch.cuda.synchronize()
    assert not torch.isnan(y).any()
    bar = TIGHT if (M <= 16 or xdt == "f32") else 2 * _bar(prefill_mode)
    assert oracle.rel_l2(y.cpu().numpy(), _silu_mul(g, u)) < bar
    # the fused weight as a plain matmul: gate and up columns interleaved in blocks of 16
    if True:
        yi = _run(backend, wf, x)
        yg, yu = _run(backend, wg, x), _run(backend, wu, x)
        inter = torch.stack([yg.view(M, N // 16, 16), yu.view(M, N // 16, 16)], dim=2).reshape(M, 2 * N)
        if M <= 16:
            assert torch.equal(yi, inter)
            # and the epilogue is exactly silu * mul of those sums, in fp32
            want = (yg / (1.0 + torch.exp(-yg)) * yu)
            assert (y - want).abs().max().item() <= 2e-6 * want.abs().max().item()
        else:
            assert ((yi - inter).double().norm() / inter.double().norm()).item() < 1e-6


def test_epilogue_swiglu_full_size_and_split_k(backend, oracle):
    # Llama-3-8B FFN width at decode (M = 1, 8) and prefill (M = 128: 14 column tiles per row block,
    # so K is split over workgroups and the activation runs in the slab-adding kernel)
    K, N = 4096, 14336
    qg, sg = _quant(oracle, 4, N, K, cfg=43)
    qu, su = _quant(oracle, 4, N, K, cfg=44)
    wg, wu = backend.upload_quantized(qg, sg, 4), backend.upload_quantized(qu, su, 4)
    wf = backend.fuse_pairs(wg, wu)
    dg = torch.from_numpy(oracle.dequant(qg, sg)).cuda().double()
    du = torch.from_numpy(oracle.dequant(qu, su)).cuda().double()
    for M, xdt, bar in ((1, "f16", TIGHT), (8, "f16", TIGHT), (128, "bf16", 2 * FAST), (512, "bf16", 2 * FAST)):
        x = _x(M, K, xdt)
        g, u = x.double() @ dg.T, x.double() @ du.T
        ref = g / (1.0 + torch.exp(-g)) * u
        y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
        backend.matmul_ex(wf, x, y, "swiglu")
        torch.cuda.synchronize()
        err = ((y.double() - ref).norm() / ref.norm()).item()
        assert err < bar, (M, err)


def _norm_ref(oracle, q, s, x, gamma, eps, op_dt):
    """float64 restatement of the stated formula: x * gamma rounded once to the operand type,
    exact matmul, rows scaled by rstd of the unrounded input."""
    xf = x.float()
    xg = xf * gamma.float()[None, :]
    if op_dt == "f32":                                # two f16 halves keep ~22 bits: compare against unrounded
        xr = xg.double().cpu().numpy()
    else:
        xr = xg.to(TDT[op_dt]).double().cpu().numpy()
    rstd = 1.0 / np.sqrt((xf.double().cpu().numpy() ** 2).mean(axis=1) + eps)
    return oracle.matmul_f64(q, s, xr) * rstd[:, None]


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("M,xdt,gdt", [(1, "f16", "f16"), (2, "bf16", "f32"), (3, "f32", "f32"), (4, "f16", "bf16"), (9, "bf16", "bf16"),
                                       (16, "f16", "f32"), (16, "f32", "f16"), (40, "bf16", "f32"), (300, "f16", "f16"),
                                       (70, "f32", "f32")])
def test_folded_rmsnorm(backend, oracle, prefill_mode, bits, M, xdt, gdt):
    N, K = 272, 1184                                   # K = 9 tiles + 1 group: a padded last tile
    eps = 1e-5
    q, s = _quant(oracle, bits, N, K)
    qw = backend.upload_quantized(q, s, bits)
    x = _x(M, K, xdt)
    x[0] *= 7.0                                        # rows of different scale: rstd must be per row
    gamma = (1.0 + 0.25 * torch.from_numpy(synth.activations(51, 1, K)[0])).cuda().to(TDT[gdt])
    y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    backend.matmul_norm(qw, x, gamma, eps, y)
    torch.cuda.synchronize()
    assert not torch.isnan(y).any()
    fast_prefill = M > (16 if xdt == "f32" else 32) and prefill_mode == "fast"
    op_dt = "f16" if (fast_prefill and xdt != "f16") else xdt       # FAST multiplies in f16
    ref = _norm_ref(oracle, q, s, x, gamma, eps, op_dt)
    bar = FAST if fast_prefill else TIGHT
    assert oracle.rel_l2(y.cpu().numpy(), ref) < bar
    # reproducible, and composes with the epilogues
    y2 = torch.empty_like(y)
    backend.matmul_norm(qw, x, gamma, eps, y2)
    r = torch.from_numpy(synth.activations(52, M, N)).cuda()
    y3 = torch.empty_like(y)
    backend.matmul_norm(qw, x, gamma, eps, y3, "add", r)
    torch.cuda.synchronize()
    assert torch.equal(y2, y)
    assert torch.equal(y3, y + r)


@pytest.mark.parametrize("M,xdt", [(1, "f16"), (8, "f16"), (64, "bf16")])
def test_folded_rmsnorm_with_swiglu_and_long_k(backend, oracle, M, xdt):
    # FFN entry as the decode loop has it: norm -> gate/up -> SwiGLU; K long enough for several x slabs
    N, K = 192, 14336
    eps = 1e-6
    qg, sg = _quant(oracle, 4, N, K, cfg=45)
    qu, su = _quant(oracle, 4, N, K, cfg=46)
    wf = backend.fuse_pairs(backend.upload_quantized(qg, sg, 4), backend.upload_quantized(qu, su, 4))
    x = _x(M, K, xdt)
    gamma = (1.0 + 0.25 * torch.from_numpy(synth.activations(53, 1, K)[0])).cuda().to(torch.float32)
    y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    backend.matmul_norm(wf, x, gamma, eps, y, "swiglu")
    torch.cuda.synchronize()
    op_dt = "f16" if M > 16 else xdt
    g = _norm_ref(oracle, qg, sg, x, gamma, eps, op_dt)
    u = _norm_ref(oracle, qu, su, x, gamma, eps, op_dt)
    assert oracle.rel_l2(y.cpu().numpy(), _silu_mul(g, u)) < (2 * FAST if M > 16 else TIGHT)


@pytest.mark.parametrize("M,xdt,gdt", [(1, "f16", "f16"), (3, "f16", "f32"), (8, "bf16", "bf16"), (16, "f16", "f16"), (16, "bf16", "f32")])
def test_folded_rmsnorm_very_long_k(backend, oracle, M, xdt, gdt):
    # K far past anything a workgroup could keep of gamma in LDS at once
    N, K = 48, 32768
    q, s = _quant(oracle, 4, N, K, cfg=47)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(M, K, xdt)
    gamma = (1.0 + 0.25 * torch.from_numpy(synth.activations(54, 1, K)[0])).cuda().to(TDT[gdt])
    y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    backend.matmul_norm(qw, x, gamma, 1e-6, y)
    torch.cuda.synchronize()
    assert oracle.rel_l2(y.cpu().numpy(), _norm_ref(oracle, q, s, x, gamma, 1e-6, xdt)) < TIGHT


@pytest.mark.parametrize("M", [1, 2, 4, 16])
def test_folded_rmsnorm_counts_subnormal_inputs(backend, oracle, M):
    # a row of f16 subnormals (|x| < 6.1e-5) with an eps far below its mean square: its squares must
    # not be flushed on the way into the sum
    N, K = 64, 1024
    eps = 1e-14
    q, s = _quant(oracle, 4, N, K, cfg=48)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(M, K, "f16")
    x[M - 1] = (x[M - 1].float() * 1e-5).to(torch.float16)
    assert x[M - 1].float().abs().max().item() < 6.1e-5
    gamma = torch.ones(K, dtype=torch.float16, device="cuda")
    y = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    backend.matmul_norm(qw, x, gamma, eps, y)
    torch.cuda.synchronize()
    ref = _norm_ref(oracle, q, s, x, gamma, eps, "f16")
    assert oracle.rel_l2(y[M - 1:].cpu().numpy(), ref[M - 1:]) < TIGHT
    assert oracle.rel_l2(y.cpu().numpy(), ref) < TIGHT


def _random_cases(seed, count):
    """Seeded draws over everything a call can vary in: block type, interchange layout, ragged N / K,
    batch rows on both sides of every kernel boundary, the three activation types, output type,
    epilogue, folded norm, prefill mode.  CYBQ_FUZZ_SEED / CYBQ_FUZZ_COUNT widen the sweep by hand."""
    rng = np.random.default_rng(seed)
    rows = [1, 2, 3, 4, 5, 8, 13, 16, 17, 24, 31, 32, 33, 48, 100, 129, 257, 300]
    cases = []
    for i in range(count):
        epi = ["none", "add", "swiglu"][int(rng.integers(0, 3))]
        N = int(rng.integers(1, 30)) * 16 if epi == "swiglu" else int(rng.integers(1, 500))
        K = 32 * int(rng.integers(1, 150)) if rng.random() < 0.8 else 32 * int(rng.integers(150, 600))
        cases.append(dict(i=i, bits=int(rng.choice([4, 8])), layout=int(rng.choice([formats.PLANAR, formats.BLOCK_AOS])),
                          N=N, K=K, M=int(rng.choice(rows)), xdt=str(rng.choice(["f16", "bf16", "f32"])),
                          ydt=str(rng.choice(["f32", "f32", "f16", "bf16"])), epi=epi, norm=bool(rng.random() < 0.4),
                          gdt=str(rng.choice(["f32", "f16", "bf16"])), mode=str(rng.choice(["fast", "exact"]))))
    return cases


@pytest.mark.parametrize("case", _random_cases(int(__import__("os").environ.get("CYBQ_FUZZ_SEED", "20240607")), int(__import__("os").environ.get("CYBQ_FUZZ_COUNT", "72"))), ids=lambda c: "-".join(str(v) for v in c.values()))
def test_random_calls_match_float64(backend, oracle, case):
    _check_random_case(backend, oracle, case)


def _random_wide_cases(seed, count):
    """The same draws over outputs wide enough for workgroups of two, four, seven or eight strips, several
    rounds of workgroups, one round of narrow prefill tiles: the variants the model shapes run, on a short K."""
    rng = np.random.default_rng(seed)
    rows = [1, 2, 3, 4, 7, 8, 12, 16, 17, 24, 32, 33, 48, 64, 100, 128, 200, 256, 300, 512]
    cases = []
    for i in range(count):
        epi = ["none", "add", "swiglu"][int(rng.integers(0, 3))]
        N = int(rng.choice([4096, 7168, 14336])) if epi == "swiglu" else int(rng.choice([6144, 8192, 9008, 12288, 14336, 16400, 28672]))
        cases.append(dict(i=1000 + i, bits=int(rng.choice([4, 4, 8])), layout=int(rng.choice([formats.PLANAR, formats.BLOCK_AOS])),
                          N=N, K=32 * int(rng.integers(1, 25)), M=int(rng.choice(rows)), xdt=str(rng.choice(["f16", "bf16", "f32"])),
                          ydt=str(rng.choice(["f32", "f32", "f16", "bf16"])), epi=epi, norm=bool(rng.random() < 0.3),
                          gdt=str(rng.choice(["f32", "f16", "bf16"])), mode=str(rng.choice(["fast", "fast", "exact"]))))
    return cases


@pytest.mark.parametrize("case", _random_wide_cases(20240608, int(__import__("os").environ.get("CYBQ_FUZZ_WIDE_COUNT", "48"))), ids=lambda c: "-".join(str(v) for v in c.values()))
def test_random_wide_calls_match_float64(backend, oracle, case):
    _check_random_case(backend, oracle, case)


def _random_mid_k_cases(seed, count):
    """Draws over K of 16 .. 34 tiles with few rows on a wide output or up to 512 rows on a narrow one: the calls
    whose 64-row pieces fill one round of workgroups (the prefill kernel whose waves split K), their neighbours
    that do not, and the modes and epilogues around them."""
    rng = np.random.default_rng(seed)
    cases = []
    for i in range(count):
        wide = bool(rng.random() < 0.4)
        N = int(rng.choice([8192, 8200, 12288, 14336])) if wide else int(rng.choice([1024, 1040, 2048, 3072, 4096, 6144]))
        M = int(rng.choice([17, 24, 33, 48, 64])) if wide else int(rng.choice([17, 40, 65, 100, 128, 129, 200, 256, 300, 384, 512]))
        cases.append(dict(i=2000 + i, bits=int(rng.choice([4, 4, 8])), layout=int(rng.choice([formats.PLANAR, formats.BLOCK_AOS])),
                          N=N, K=128 * int(rng.integers(16, 35)), M=M, xdt=str(rng.choice(["f16", "bf16", "f32"])),
                          ydt=str(rng.choice(["f32", "f32", "f16", "bf16"])), epi=str(rng.choice(["none", "add"])),
                          norm=bool(rng.random() < 0.3), gdt=str(rng.choice(["f32", "f16", "bf16"])),
                          mode=str(rng.choice(["fast", "fast", "fast", "exact"]))))
    return cases


@pytest.mark.parametrize("case", _random_mid_k_cases(20240609, int(__import__("os").environ.get("CYBQ_FUZZ_MID_COUNT", "24"))), ids=lambda c: "-".join(str(v) for v in c.values()))
def test_random_mid_k_calls_match_float64(backend, oracle, case):
    _check_random_case(backend, oracle, case)


def _check_random_case(backend, oracle, c):
    bits, N, K, M = c["bits"], c["N"], c["K"], c["M"]
    backend.set_prefill_mode(c["mode"])
    try:
        x = _x(M, K, c["xdt"], cfg=60 + c["i"])
        if M > 1:
            x[M // 2] *= 5.0
        gamma = (1.0 + 0.25 * torch.from_numpy(synth.activations(61, 1, K)[0])).cuda().to(TDT[c["gdt"]])
        eps = 1e-5
        prefill = (M > 32 and c["xdt"] != "f32") or (M > 16 and c["xdt"] == "f32" and c["mode"] == "fast")
        fast = prefill and c["mode"] == "fast"
        op_dt = "f16" if (fast and c["xdt"] != "f16") else c["xdt"]

        def product(q, s):
            if c["norm"]:
                return _norm_ref(oracle, q, s, x, gamma, eps, op_dt)
            return oracle.matmul_f64(q, s, x.float().cpu().numpy())

        if c["epi"] == "swiglu":
            qg, sg = _quant(oracle, bits, N, K, cfg=70 + c["i"])
            qu, su = _quant(oracle, bits, N, K, cfg=170 + c["i"])
            w = backend.fuse_pairs(backend.upload_quantized(qg, sg, bits, c["layout"]),
                                   backend.upload_quantized(qu, su, bits, c["layout"]))
            ref = _silu_mul(product(qg, sg), product(qu, su))
        else:
            q, s = _quant(oracle, bits, N, K, cfg=70 + c["i"])
            w = backend.upload_quantized(q, s, bits, c["layout"])
            ref = product(q, s)
        r = None
        if c["epi"] == "add":
            r = torch.from_numpy(synth.activations(62, M, N)).cuda().to(TDT[c["ydt"]])
            ref = ref + r.double().cpu().numpy()
        y = torch.full((M, N), float("nan"), dtype=TDT[c["ydt"]], device="cuda")
        if c["norm"]:
            backend.matmul_norm(w, x, gamma, eps, y, c["epi"], r)
        else:
            backend.matmul_ex(w, x, y, c["epi"], r)
        torch.cuda.synchronize()
        assert not torch.isnan(y).any(), c
        bar = FAST if fast else TIGHT
        if c["epi"] == "swiglu":
            bar *= 2
        if c["ydt"] == "f16":
            bar = max(bar, 6e-4)                          # one rounding to 11 bits
        if c["ydt"] == "bf16":
            bar = max(bar, 4e-3)                          # one rounding to 8 bits
        err = oracle.rel_l2(y.float().cpu().numpy(), ref)
        assert err < bar, (c, err)
        w.free()
    finally:
        backend.set_prefill_mode("fast")


def test_epilogue_errors(backend, oracle):
    q, s = _quant(oracle, 4, 64, 256)
    qw = backend.upload_quantized(q, s, 4)
    x = _x(2, 256, "f16")
    y = torch.empty((2, 64), dtype=torch.float32, device="cuda")
    with pytest.raises(CybqError):
        backend.matmul_ex(qw, x, y, "swiglu")                 # not a fused pair
    with pytest.raises(CybqError):
        backend.matmul_ex(qw, x, y, "add", None)              # no residual
    q2, s2 = _quant(oracle, 4, 40, 256)
    with pytest.raises(CybqError):
        backend.fuse_pairs(backend.upload_quantized(q2, s2, 4), backend.upload_quantized(q2, s2, 4))   # N % 16
    with pytest.raises(CybqError):
        backend.fuse_pairs(qw, backend.upload_quantized(q2, s2, 4))                                    # shapes differ


# ------------------------------------------------------------------ quantise

@pytest.mark.parametrize("bits", [4, 8])
def test_device_quantizer_bit_exact(backend, oracle, bits):
    N, K = 300, 1024
    w = synth.weights(31, N, K)
    w[0, :32] = 0
    w[1, 32:64] *= 1e-6
    w[2, 5] = 0.35
    src = torch.from_numpy(w).cuda()
    qd = torch.empty(N * K * bits // 8, dtype=torch.uint8, device="cuda")
    sd = torch.empty(N * K // 32, dtype=torch.int16, device="cuda")
    backend.quantize(bits, src, N, K, qd, sd)
    torch.cuda.synchronize()
    q, s = oracle.quantize(w, bits)
    assert np.array_equal(sd.cpu().numpy().view(np.uint16).reshape(N, -1), s)
    assert np.array_equal(qd.cpu().numpy(), oracle.pack_planar(q, bits))
    # device buffers -> weight handle -> the op, without touching the host
    qw = backend.weight_from_device(bits, N, K, qd, sd)
    out = torch.empty((N, K), dtype=torch.float32, device="cuda")
    backend.dequant(qw, out)
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy().view(np.uint32), oracle.dequant(q, s).view(np.uint32))


# ------------------------------------------------------------ interface / errors

def test_graph_node_execution(backend, oracle):
    N, K = 64, 128
    q, s = _quant(oracle, 4, N, K)
    backend.upload_quantized(q, s, 4, name="model.layers.0.self_attn.q_proj.weight")
    node = QMatMul(w="model.layers.0.self_attn.q_proj.weight", x="h0", y="q0", quant=4, M=2, N=N, K=K)
    edges = {"h0": _x(2, K, "f16"), "q0": torch.empty((2, N), dtype=torch.float32, device="cuda")}
    backend.run(node, edges)
    torch.cuda.synchronize()
    assert oracle.rel_l2(edges["q0"].cpu().numpy(),
                         oracle.matmul_f64(q, s, edges["h0"].float().cpu().numpy())) < TIGHT
    with pytest.raises(CybqError):
        backend.run(QMatMul(w="missing", x="h0", y="q0"), edges)
    with pytest.raises(CybqError):
        backend.run(QMatMul(w=node.w, x="h0", y="q0", quant=4, N=N + 16, K=K), edges)


def test_error_codes(backend, oracle):
    q, s = _quant(oracle, 4, 16, 64)
    with pytest.raises(CybqError) as e:
        backend.upload(4, formats.PLANAR, 16, 48, formats.pack_planar(q, 4), s)       # K % 32
    assert e.value.status == -2
    with pytest.raises(CybqError) as e:
        backend.upload(4, formats.PLANAR, 16, 64, formats.pack_planar(q, 4), None)    # no scales
    assert e.value.status == -1
    with pytest.raises(CybqError) as e:
        backend.upload(5, formats.PLANAR, 16, 64, formats.pack_planar(q, 4), s)       # bad quant
    assert e.value.status == -1
    with pytest.raises(CybqError) as e:
        backend.upload(4, formats.PLANAR, 32, 64, formats.pack_planar(q, 4), s)       # buffers of a 16-row tensor
    assert e.value.status == -2
    qw = backend.upload_quantized(q, s, 4)
    x = _x(2, 64, "f16")
    y = torch.empty((2, 16), dtype=torch.float32, device="cuda")
    with pytest.raises(CybqError) as e:
        backend.matmul(qw, x, y, M=0)
    assert e.value.status == -2
    # the host wrapper refuses tensors the library could only see as raw pointers of the wrong size
    for bad_x, bad_y in ((x[:1], y), (x, y[:1]), (x.t().contiguous().t(), y), (x.cpu(), y)):
        with pytest.raises(CybqError) as e:
            backend.matmul(qw, bad_x, bad_y, M=2)
        assert e.value.status in (-1, -2)
    buf = torch.empty(2 * 64 + 8, dtype=torch.float16, device="cuda")
    with pytest.raises(CybqError) as e:
        backend.matmul(qw, buf.data_ptr() + 2, y, M=2, xdt=1)                         # misaligned x
    assert e.value.status == -3
    # the context stays usable after errors
    backend.matmul(qw, x, y)
    torch.cuda.synchronize()
    assert oracle.rel_l2(y.cpu().numpy(), oracle.matmul_f64(q, s, x.float().cpu().numpy())) < TIGHT


# ------------------------------------------------------------ decode-step stack

def test_decode_stack_small(backend, oracle):
    """Config 5 in miniature: 2 layers x 7 linears of a scaled-down LlamaStyle model,
    weights generated and quantised on the device, every linear checked on its own."""
    from cyb_amd import stack
    shapes = {"q_proj": (512, 512), "k_proj": (512, 128), "v_proj": (512, 128), "o_proj": (512, 512),
              "gate_proj": (512, 1792), "up_proj": (512, 1792), "down_proj": (1792, 512)}
    st = stack.build(backend, layers=2, seed=5, keep_planar=2, shapes=shapes)
    assert len(st.nodes) == 14
    for M in (1, 8):
        edges = stack.edges_for(st, M, shapes=shapes)
        pl = stack.plan(st, edges)
        # run linear by linear so that every output can be read before it is overwritten
        for i, node in enumerate(st.nodes):
            node.M = M
            backend.run(node, edges)
            torch.cuda.synchronize()
            qd, sd = st.planar[node.w]
            q = formats.unpack_planar(qd.cpu().numpy(), 4, node.N, node.K)
            s = sd.cpu().numpy().view(np.uint16).reshape(node.N, node.K // 32)
            ref = oracle.matmul_f64(q, s, edges[node.x].float().cpu().numpy())
            assert oracle.rel_l2(edges[node.y].cpu().numpy(), ref) < TIGHT, node.w
        # and the whole step through the native node walk gives the last layer's outputs
        backend.matmul_many(pl, M)
        torch.cuda.synchronize()
        last = st.nodes[-1]
        qd, sd = st.planar[last.w]
        q = formats.unpack_planar(qd.cpu().numpy(), 4, last.N, last.K)
        s = sd.cpu().numpy().view(np.uint16).reshape(last.N, last.K // 32)
        ref = oracle.matmul_f64(q, s, edges[last.x].float().cpu().numpy())
        assert oracle.rel_l2(edges[last.y].cpu().numpy(), ref) < TIGHT
    assert st.step_bytes(1) == sum(formats.matmul_bytes(4, n.N, n.K, 1, 2, 4) for n in st.nodes)
    for w in st.weights:
        w.free()


def test_decode_stack_with_epilogues(backend, oracle):
    """The fused node list (qkv, o + residual, gate/up with SwiGLU, down + residual) through
    cybq_matmul_many_ex; every node's output recomputed from the weights the stack kept."""
    from cyb_amd import stack
    base = {"q_proj": (512, 512), "k_proj": (512, 128), "v_proj": (512, 128), "o_proj": (512, 512),
            "gate_proj": (512, 1792), "up_proj": (512, 1792), "down_proj": (1792, 512)}
    shapes = stack.fused_shapes(base)
    st = stack.build(backend, layers=2, seed=6, keep_planar=2, shapes=shapes, order=list(shapes), epilogues=True)
    assert st.epilogues == ["none", "add", "swiglu", "add"] * 2
    for M in (1, 8, 40):
        edges = stack.edges_for(st, M, shapes=shapes, xdtype=torch.bfloat16 if M > 16 else None)
        pl = stack.plan(st, edges)
        backend.matmul_many(pl, M)
        torch.cuda.synchronize()
        bar = TIGHT if M <= 16 else 2 * FAST
        for node, epi in list(zip(st.nodes, st.epilogues))[-4:]:          # the last layer's outputs are still in place
            qd, sd = st.planar[node.w]
            q = formats.unpack_planar(qd.cpu().numpy(), 4, node.N, node.K)
            s = sd.cpu().numpy().view(np.uint16).reshape(node.N, node.K // 32)
            ref = oracle.matmul_f64(q, s, edges[node.x].float().cpu().numpy())
            if epi == "add":
                ref = ref + edges[f"res.{node.N}"].double().cpu().numpy()
            elif epi == "swiglu":
                h = node.N // 2
                ref = _silu_mul(ref[:, :h], ref[:, h:])
            got = edges[node.y].cpu().numpy()
            assert got.shape == ref.shape
            assert oracle.rel_l2(got, ref) < bar, (M, node.w, epi)
    for w in st.weights:
        w.free()


def test_decode_stack_with_norms(backend, oracle):
    """A whole layer's linear path in one native walk (cybq_matmul_many_norm): RMSNorm folded in front
    of qkv and gate/up, SwiGLU and the two residual adds in the epilogues.  Every node of the last
    layer against the float64 restatement, and against the one-node entry point bit for bit."""
    from cyb_amd import stack
    base = {"q_proj": (512, 512), "k_proj": (512, 128), "v_proj": (512, 128), "o_proj": (512, 512),
            "gate_proj": (512, 1792), "up_proj": (512, 1792), "down_proj": (1792, 512)}
    shapes = stack.fused_shapes(base)
    st = stack.build(backend, layers=2, seed=8, keep_planar=2, shapes=shapes, order=list(shapes), epilogues=True, norms=True)
    assert [g is not None for g in st.gammas] == [True, False, True, False] * 2
    assert st.gammas[0] is not st.gammas[2] and st.gammas[0] is not st.gammas[4]
    for M in (1, 2, 8, 40):
        xdt = "bf16" if M > 16 else "f16"
        edges = stack.edges_for(st, M, shapes=shapes, xdtype=torch.bfloat16 if M > 16 else None)
        pl = stack.plan(st, edges)
        backend.matmul_many(pl, M)
        torch.cuda.synchronize()
        bar = TIGHT if M <= 16 else 2 * FAST
        for i in range(len(st.nodes) - 4, len(st.nodes)):                 # the last layer's outputs are still in place
            node, epi, gamma = st.nodes[i], st.epilogues[i], st.gammas[i]
            if gamma is None:
                ref = _node_reference(oracle, st, node, epi, edges)
            else:
                qd, sd = st.planar[node.w]
                q = formats.unpack_planar(qd.cpu().numpy(), 4, node.N, node.K)
                s = sd.cpu().numpy().view(np.uint16).reshape(node.N, node.K // 32)
                ref = _norm_ref(oracle, q, s, edges[node.x], gamma, st.eps, "f16" if M > 16 else xdt)
                if epi == "swiglu":
                    ref = _silu_mul(ref[:, :node.N // 2], ref[:, node.N // 2:])
            got = edges[node.y]
            assert oracle.rel_l2(got.cpu().numpy(), ref) < bar, (M, node.w, epi)
            one = torch.empty_like(got)
            res = edges[f"res.{node.N}"] if epi == "add" else None
            if gamma is None:
                backend.matmul_ex(st.weights[i], edges[node.x], one, epi, res)
            else:
                backend.matmul_norm(st.weights[i], edges[node.x], gamma, st.eps, one, epi, res)
            torch.cuda.synchronize()
            assert torch.equal(one, got), (M, node.w)
    for w in st.weights:
        w.free()


def test_many_norm_without_gammas_is_many_ex_and_rejects_bad_arguments(backend, oracle):
    """cybq_matmul_many_norm with no gamma anywhere is cybq_matmul_many_ex bit for bit; a node whose gamma is
    NULL runs without a norm; errors come back as values."""
    N, K, M = 96, 512, 5
    q, s = _quant(oracle, 4, N, K, cfg=95)
    w = backend.upload_quantized(q, s, 4)
    x = _x(M, K, "f16", cfg=96)
    gamma = (1.0 + 0.25 * torch.from_numpy(synth.activations(97, 1, K)[0])).cuda().to(torch.float16)
    y_plain = torch.empty((M, N), dtype=torch.float32, device="cuda")
    y_norm = torch.empty_like(y_plain)
    backend.matmul(w, x, y_plain)
    backend.matmul_norm(w, x, gamma, 1e-5, y_norm)
    ya, yb = torch.zeros_like(y_plain), torch.zeros_like(y_plain)
    backend.matmul_many(backend.plan_many([w, w], [x, x], [ya, yb], gammas=[None, gamma], eps=1e-5), M)
    torch.cuda.synchronize()
    assert torch.equal(ya, y_plain) and torch.equal(yb, y_norm)
    lib, ctx = backend._lib, backend._ctx
    import ctypes
    arr = lambda vals: (ctypes.c_void_p * len(vals))(*vals)
    ws, xs, ys = arr([w.handle]), arr([x.data_ptr()]), arr([ya.data_ptr()])
    ya.zero_()
    rc = lib.cybq_matmul_many_norm(ctx, 1, ws, xs, None, 1, ctypes.c_float(1e-5), ys, None, None, 1, M, 0, None)
    torch.cuda.synchronize()
    assert rc == 0 and torch.equal(ya, y_plain)                         # no gamma array at all
    gs = arr([gamma.data_ptr()])
    assert lib.cybq_matmul_many_norm(ctx, 1, ws, xs, gs, 77, ctypes.c_float(1e-5), ys, None, None, 1, M, 0, None) != 0     # unknown gamma type
    assert lib.cybq_matmul_many_norm(ctx, 1, ws, xs, gs, 1, ctypes.c_float(-1.0), ys, None, None, 1, M, 0, None) != 0    # negative eps
    assert lib.cybq_matmul_many_norm(ctx, 1, None, xs, gs, 1, ctypes.c_float(1e-5), ys, None, None, 1, M, 0, None) != 0   # no weights
    assert lib.cybq_matmul_many_norm(ctx, 0, ws, xs, gs, 1, ctypes.c_float(1e-5), ys, None, None, 1, M, 0, None) == 0     # nothing to do


@pytest.mark.parametrize("M", [33, 40, 64])
@pytest.mark.parametrize("xdt", ["f16", "bf16"])
def test_rows_33_to_64_on_a_small_weight_are_two_decode_passes(backend, oracle, M, xdt):
    """33..64 rows of 16-bit activations on a small weight: rows 0..31 carry the bits of a 32-row call,
    the rest those of a call with the remaining rows (a row's bits do not depend on the batch it is in),
    in both prefill modes (prefill EXACT asks the decode kernels for their exact operands), and the
    float64 result within the decode kernels' bar."""
    N, K = 272, 1184
    q, s = _quant(oracle, 4, N, K, cfg=98)
    w = backend.upload_quantized(q, s, 4)
    x = _x(M, K, xdt, cfg=99)
    r = torch.from_numpy(synth.activations(100, M, N)).cuda()
    for mode in ("fast", "exact"):
        backend.set_prefill_mode(mode)
        try:
            y = torch.empty((M, N), dtype=torch.float32, device="cuda")
            backend.matmul_ex(w, x, y, "add", r)
            y_a = torch.empty((32, N), dtype=torch.float32, device="cuda")
            y_b = torch.empty((M - 32, N), dtype=torch.float32, device="cuda")
            backend.set_decode_mode("exact" if mode == "exact" else "stream")
            backend.matmul_ex(w, x[:32].contiguous(), y_a, "add", r[:32].contiguous())
            backend.matmul_ex(w, x[32:].contiguous(), y_b, "add", r[32:].contiguous())
            torch.cuda.synchronize()
            assert torch.equal(y[:32], y_a) and torch.equal(y[32:], y_b)
            ref = oracle.matmul_f64(q, s, x.float().cpu().numpy()) + r.double().cpu().numpy()
            assert oracle.rel_l2(y.cpu().numpy(), ref) < TIGHT
        finally:
            backend.set_prefill_mode("fast")
            backend.set_decode_mode("stream")
    if xdt == "f16":
        # prefill EXACT at these row counts: a tensor of zeros gives exact zeros (the exact integer operands)
        wz = backend.upload_quantized(np.zeros_like(q), s, 4)
        backend.set_prefill_mode("exact")
        try:
            assert not _run(backend, wz, x).any()
        finally:
            backend.set_prefill_mode("fast")
        wz.free()


def _node_reference(oracle, st, node, epi, edges, rows=None):
    """float64 oracle output of one stack node from the PLANAR buffers the stack kept."""
    qd, sd = st.planar[node.w]
    q = formats.unpack_planar(qd.cpu().numpy(), 4, node.N, node.K)
    s = sd.cpu().numpy().view(np.uint16).reshape(node.N, node.K // 32)
    x = edges[node.x] if rows is None else edges[node.x][rows]
    ref = oracle.matmul_f64(q, s, x.float().cpu().numpy())
    if epi == "add":
        r = edges[f"res.{node.N}"] if rows is None else edges[f"res.{node.N}"][rows]
        ref = ref + r.double().cpu().numpy()
    elif epi == "swiglu":
        h = node.N // 2
        ref = _silu_mul(ref[:, :h], ref[:, h:])
    return ref


@pytest.mark.timeout(900)
@pytest.mark.parametrize("form", ["per_linear", "fused", "fused_epilogues"])
def test_config5_full_size_stack(backend, oracle, form):
    """The 32-layer Llama-3-8B-shaped decode step through cybq_matmul_many at full size, batch 1 and 8:
    every node of the first, a middle and the last layer against the oracle; for the fused forms also
    one 512-token bf16 prefill chunk through the same node list."""
    from cyb_amd import stack
    shapes = None if form == "per_linear" else stack.fused_shapes()
    checked = (0, 15, 31)
    st = stack.build(backend, layers=32, seed=5, keep_planar=checked, shapes=shapes,
                     order=list(shapes) if shapes else None, epilogues=form == "fused_epilogues")
    per_layer = len(st.nodes) // 32
    assert per_layer == (7 if shapes is None else 4)
    epis = st.epilogues or ["none"] * len(st.nodes)
    mine = [i for i in range(len(st.nodes)) if i // per_layer in checked]
    for M in (1, 8, 512) if shapes is not None else (1, 8):
        edges = stack.edges_for(st, M, shapes=shapes, xdtype=torch.bfloat16 if M > 16 else None)
        xs, ys = [edges[n.x] for n in st.nodes], [edges[n.y] for n in st.nodes]
        for i in mine:                                  # the checked nodes write buffers of their own
            ys[i] = torch.full_like(ys[i], float("nan"))
        res = None
        if st.epilogues:
            res = [edges[f"res.{n.N}"] if e == "add" else None for n, e in zip(st.nodes, st.epilogues)]
        pl = backend.plan_many(st.weights, xs, ys, st.epilogues or None, res)
        backend.matmul_many(pl, M)
        torch.cuda.synchronize()
        for i in mine:
            node, epi = st.nodes[i], epis[i]
            if M <= 16:
                ref = _node_reference(oracle, st, node, epi, edges)
                assert oracle.rel_l2(ys[i].cpu().numpy(), ref) < TIGHT, (M, node.w, epi)
            else:
                rows = [0, M // 2, M - 1]
                ref = _node_reference(oracle, st, node, epi, edges, rows)
                assert oracle.rel_l2(ys[i][rows].cpu().numpy(), ref) < 2 * FAST, (M, node.w, epi)
                assert torch.isfinite(ys[i]).all()
        if M > 16:
            # every row of the widest and of the longest-K node of the last layer: float64 matmul on the
            # oracle's dequantised weights
            for i in mine[-per_layer:]:
                node, epi = st.nodes[i], epis[i]
                if epi == "swiglu" or node.N * node.K < 4096 * 14336:
                    continue
                qd, sd = st.planar[node.w]
                q = formats.unpack_planar(qd.cpu().numpy(), 4, node.N, node.K)
                s = sd.cpu().numpy().view(np.uint16).reshape(node.N, node.K // 32)
                wd = torch.from_numpy(oracle.dequant(q, s)).cuda().double()
                full = edges[node.x].double() @ wd.T
                if epi == "add":
                    full = full + edges[f"res.{node.N}"].double()
                err = ((ys[i].double() - full).norm() / full.norm()).item()
                assert err < 2 * FAST, (M, node.w, err)
                del wd, full
    assert st.weight_bytes == 32 * 122_683_392
    for w in st.weights:
        w.free()


def test_driver_events_and_rates(backend):
    """The caller loop in the reference's units: event order, token counts, positive rates."""
    from cyb_amd import driver, stack
    shapes = stack.fused_shapes({"q_proj": (512, 512), "k_proj": (512, 128), "v_proj": (512, 128), "o_proj": (512, 512),
                                 "gate_proj": (512, 1792), "up_proj": (512, 1792), "down_proj": (1792, 512)})
    st = stack.build(backend, layers=2, seed=7, shapes=shapes, order=list(shapes))
    evs = list(driver.ask(backend, st, prompt_tokens=300, new_tokens=5, chunk=128, shapes=shapes))
    pre = [e["Prefill"] for e in evs if "Prefill" in e]
    assert [p["done"] for p in pre] == [0, 128, 256, 300] and all(p["total"] == 300 for p in pre)
    assert [e["Delta"] for e in evs if "Delta" in e] == [0, 1, 2, 3, 4]
    ans = evs[-1]["Answer"]
    assert ans.tokens == 5 and ans.tok_in_s > 0 and ans.tok_out_s > 0 and ans.tok_per_s > 0
    # decode only, batch of 4
    evs = list(driver.ask(backend, st, prompt_tokens=0, new_tokens=3, batch=4, shapes=shapes))
    assert evs[-1]["Answer"].tokens == 12 and evs[-1]["Answer"].tok_in_s == 0.0
    with pytest.raises(ValueError):
        list(driver.ask(backend, st, 1, 1, batch=17, shapes=shapes))
    for w in st.weights:
        w.free()


@pytest.mark.parametrize("M,xdt", [(1, "f16"), (8, "f16"), (300, "bf16")])
def test_calls_can_be_captured_in_a_graph(backend, oracle, M, xdt):
    """Every call is a short run of plain kernel launches on the caller's stream (no allocation, no
    memset, no host synchronisation), so a caller may record a step into a HIP graph.  The graph is
    replayed several times with eager work and synchronisations in between, every replay checked
    bit for bit against the eager result (decode kernels; staging pass + multiply + slab adding for
    the prefill shape, whose 4096 columns split K over workgroups)."""
    K1, N1, K2, N2 = 512, 1024, 2048, 4096
    q1, s1 = _quant(oracle, 4, N1, K1, cfg=81)
    q2, s2 = _quant(oracle, 8, N2, K2, cfg=82)
    w1, w2 = backend.upload_quantized(q1, s1, 4), backend.upload_quantized(q2, s2, 8)
    x1, x2 = _x(M, K1, xdt, cfg=83), _x(M, K2, xdt, cfg=84)
    r = torch.from_numpy(synth.activations(85, M, N2)).cuda()
    h = torch.empty((M, N1), dtype=torch.float32, device="cuda")
    y = torch.empty((M, N2), dtype=torch.float32, device="cuda")

    def step(stream):
        backend.matmul(w1, x1, h, stream=stream)
        backend.matmul_ex(w2, x2, y, "add", r, stream=stream)

    step(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    h0, y0 = h.clone(), y.clone()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step(torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        h.zero_()
        y.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(h, h0) and torch.equal(y, y0)
        assert (x1.float() @ x1.float().T).sum().isfinite()          # eager work between replays


def test_first_call_of_a_kernel_may_sit_inside_a_capture(oracle):
    """No launch path changes a function attribute (cybq_init raised every kernel's dynamic LDS limit): a
    fresh context may record calls whose kernels it has never launched - kernels that need more than the
    default 64 KB of LDS among them - and the replay matches an eager run made afterwards."""
    from cyb_amd import Backend
    be = Backend(0)
    try:
        be.set_prefill_mode("exact")                       # EXACT prefill tiles stage 112 - 128 KB of operands in LDS
        N, K, M = 208, 2176, 77                            # shapes no other test uses
        q, s = _quant(oracle, 8, N, K, cfg=91)
        qw = be.upload_quantized(q, s, 8, formats.BLOCK_AOS)
        x = _x(M, K, "bf16", cfg=92)
        x32 = _x(12, K, "f32", cfg=93)                     # LDS decode kernel, fp32 rows: its largest LDS request
        y = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        y32 = torch.zeros((12, N), dtype=torch.float32, device="cuda")
        side = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            st = torch.cuda.current_stream().cuda_stream
            be.matmul(qw, x, y, stream=st)
            be.matmul(qw, x32, y32, stream=st)
        for _ in range(2):
            y.zero_()
            y32.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert oracle.rel_l2(y.cpu().numpy(), oracle.matmul_f64(q, s, x.float().cpu().numpy())) < TIGHT
            assert oracle.rel_l2(y32.cpu().numpy(), oracle.matmul_f64(q, s, x32.cpu().numpy())) < TIGHT
        ye = torch.zeros_like(y)
        be.matmul(qw, x, ye)
        torch.cuda.synchronize()
        assert torch.equal(ye, y)
        qw.free()
        # FAST mode, 50 rows on a wide output: the kernel whose waves split K (80 KB of LDS for its one exchange)
        be.set_prefill_mode("fast")
        N, K, M = 8192 + 64, 4096 + 128, 50
        q, s = _quant(oracle, 4, N, K, cfg=94)
        qw = be.upload_quantized(q, s, 4)
        x = _x(M, K, "bf16", cfg=95)
        y = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            be.matmul(qw, x, y, stream=torch.cuda.current_stream().cuda_stream)
        for _ in range(2):
            y.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert oracle.rel_l2(y.cpu().numpy(), oracle.matmul_f64(q, s, x.float().cpu().numpy())) < FAST
        ye = torch.zeros_like(y)
        be.matmul(qw, x, ye)
        torch.cuda.synchronize()
        assert torch.equal(ye, y)
        qw.free()
    finally:
        be.close()


def test_read_pattern_probes_run(backend, oracle):
    """The pure-read probes the benchmark records as ceilings: every pattern runs on the headline tensor's
    K and on a ragged tensor (flat patterns), and the strip patterns refuse shapes they do not cover."""
    q, s = _quant(oracle, 4, 272, 4096, cfg=61)
    w = backend.upload_quantized(q, s, 4)
    q2, s2 = _quant(oracle, 8, 40, 416, cfg=62)
    w2 = backend.upload_quantized(q2, s2, 8)
    xd = torch.zeros(8, dtype=torch.float16, device="cuda")            # (a plan wants edges; the probes read none)
    yd = torch.zeros(8, dtype=torch.float32, device="cuda")
    plan = backend.plan_many([w, w], [xd, xd], [yd, yd])
    plan2 = backend.plan_many([w2], [xd], [yd])
    for pattern in range(1, 7):
        backend.debug_read_pattern(plan, pattern)
    for pattern in (3, 4, 5, 6):
        backend.debug_read_pattern(plan2, pattern)
    torch.cuda.synchronize()
    for pattern in (1, 2, 0, 7):
        with pytest.raises(CybqError) as e:
            backend.debug_read_pattern(plan2, pattern)
        assert e.value.status == -7
    w.free()
    w2.free()


def test_container_to_backend(backend, oracle, tmp_path):
    from cyb_amd import container
    q, s = _quant(oracle, 4, 64, 256)
    path = str(tmp_path / "one.model")
    container.write_container(path, "one", "", [container.tensor_entry("lm_head.weight", q, s, 4, formats.BLOCK_AOS)])
    recs = container.load_into(backend, path)
    assert [r.name for r in recs] == ["lm_head.weight"]
    x = _x(3, 256, "f16")
    y = torch.empty((3, 64), dtype=torch.float32, device="cuda")
    backend.run(QMatMul(w="lm_head.weight", x="x", y="y", quant=4, M=3, N=64, K=256), {"x": x, "y": y})
    torch.cuda.synchronize()
    assert oracle.rel_l2(y.cpu().numpy(), oracle.matmul_f64(q, s, x.float().cpu().numpy())) < TIGHT
