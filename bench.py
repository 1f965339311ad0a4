#!/usr/bin/env python3
"""Benchmark of the block-quantized matmul hot path on one MI355X.

Headline workload (`config.workload`): the decode GEMV of a Llama-3-8B-shaped
gate/up projection - Q4 weights 4096 -> 14336 (N=14336, K=4096), batch 1, f16
activations, f32 output, seeded synthetic data.  One "step" is one invocation
of the op (one kernel launch) over one batch; consecutive steps walk over
distinct device copies of the weight tensor (more bytes than the 256 MB
last-level cache), so every step streams its weights from HBM.  Inputs are
resident in HBM before the timed region starts.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published
MALL_BYTES = 256 << 20
# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by a plain
# 256 MiB copy: FETCH x 1.9997, WRITE x 1.0000); profiles/decode_gemv_q4_4096x14336_m1.md
TRAFFIC_DECODE_BYTES = 33_270_500
TRAFFIC_PREFILL_M512_BYTES = 121_950_000     # multiply 113.5 MB + activation staging pass 8.4 MB


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def timed_many(be, plan, M, stream, torch):
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    be.matmul_many(plan, M, stream)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3      # seconds


def cpu_baseline(q, s, x32, alg_bytes, budget_s=12.0):
    """The CPU restatement (oracle, row-parallel fp32) timed on the host cores."""
    import numpy as np
    from tests.oracle_lib import Oracle
    ora = Oracle()
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        cores = os.cpu_count() or 1
    threads = max(1, min(16, cores))
    copies = [(q, s)] + [(q.copy(), s.copy()) for _ in range(3)]   # > L3 of any one CCD
    ora.matmul_mt(q, s, x32, threads)                               # warm-up, page-in
    reps, t0 = 0, time.perf_counter()
    while True:
        qq, ss = copies[reps % len(copies)]
        ora.matmul_mt(qq, ss, x32, threads)
        reps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or reps >= 4000:
            break
    # the same restatement on one thread (fixed summation order), a few passes
    r1, t1 = 0, time.perf_counter()
    while r1 < 40 and time.perf_counter() - t1 < 3.0:
        qq, ss = copies[r1 % len(copies)]
        ora.matmul_f32(qq, ss, x32)
        r1 += 1
    el1 = time.perf_counter() - t1
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            model = next((l.split(":", 1)[1].strip() for l in f if l.startswith("model name")), "")
    except OSError:
        pass
    return {"value": round(alg_bytes * reps / el / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{reps} passes of the same 4096->14336 Q4 batch-1 matmul over {len(copies)} weight copies, "
                      f"{el:.1f} s, C restatement (fp32, per-group scale, rows split over {threads} threads)",
            "us_per_pass": round(el / reps * 1e6, 1),
            "one_thread": {"value": round(alg_bytes * r1 / el1 / 1e9, 3), "unit": "GB/s", "us_per_pass": round(el1 / r1 * 1e6, 1),
                           "passes": r1},
            "host": {"cpus_available": cores, "cpu_model": model}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the prefill / sweep extras")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="no timing: a plain 256 MiB device copy (calibration), then the decode and prefill "
                         "kernels, for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the op would shard by rows of W "
              "for q/k/v/gate/up and by columns for o/down). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from cyb_amd import Backend, formats, synth

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    be = Backend(0)                      # raises if libcybq.so is missing
    stream = torch.cuda.current_stream().cuda_stream

    K, N, M, bits = 4096, 14336, 1, formats.Q4
    t0 = time.time()
    wf = synth.weights(2, N, K)
    q, s = formats.quantize(wf, bits)
    del wf
    x32 = synth.activations(2, M, K)
    x = torch.from_numpy(x32).to(dev).to(torch.float16)
    x32 = x.float().cpu().numpy()        # the f16-rounded activations, widened
    w0 = be.upload_quantized(q, s, bits)
    alg_w = formats.weight_bytes(bits, N, K)
    alg_bytes = formats.matmul_bytes(bits, N, K, M, 2, 4)
    copies = max(2, (3 * MALL_BYTES) // alg_w + 1)       # 24 copies, 793 MB
    ws = [w0] + [w0.clone() for _ in range(copies - 1)]
    ys = [torch.empty((M, N), dtype=torch.float32, device=dev) for _ in range(2)]
    log(f"setup {time.time() - t0:.1f}s: {copies} weight copies x {alg_w} B")

    # parity in the run that is timed: float64 matmul on the dequantised weights
    be.matmul(ws[-1], x, ys[0], stream=stream)
    torch.cuda.synchronize()
    ref = x32.astype(np.float64) @ formats.dequantize(q, s).astype(np.float64).T
    got = ys[0].cpu().numpy().astype(np.float64)
    rel_l2 = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))
    log(f"parity rel_l2 = {rel_l2:.3e}")
    if not rel_l2 < 1e-3:
        print(f"parity failed: rel_l2 = {rel_l2}", file=sys.stderr)
        sys.exit(1)

    def plan_of(n):
        return be.plan_many([ws[i % copies] for i in range(n)], [x] * n, [ys[i % 2] for i in range(n)])

    if args.traffic_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)                      # plain copy kernel of known size: 256 MiB read, 256 MiB written
        be.matmul_many(plan_of(100), M, stream)
        xp = torch.from_numpy(synth.activations(4, 512, K)).to(dev).to(torch.bfloat16)
        yp = torch.empty((512, N), dtype=torch.float32, device=dev)
        for i in range(10):
            be.matmul(ws[i % copies], xp, yp, stream=stream)
        torch.cuda.synchronize()
        log("traffic probe done")
        return

    if args.warmup > 0:
        be.matmul_many(plan_of(args.warmup), M, stream)
    plan = plan_of(args.steps)
    el = timed_many(be, plan, M, stream, torch)
    us = el / args.steps * 1e6
    gbs = alg_bytes / (el / args.steps) / 1e9
    log(f"decode GEMV: {us:.2f} us/launch, {gbs:.0f} GB/s")

    # one isolated launch (idle GPU before and after)
    lat = []
    one = plan_of(1)
    for _ in range(20):
        lat.append(timed_many(be, one, M, stream, torch) * 1e6)
    lat.sort()

    # spread: batches of 25 back-to-back launches (one pass over the weight copies), each timed on its own
    per = []
    batch = plan_of(copies)
    for _ in range(40):
        per.append(timed_many(be, batch, M, stream, torch) / copies * 1e6)
    per.sort()
    spread = {"min": round(per[0], 2), "median": round(per[len(per) // 2], 2), "p95": round(per[int(len(per) * 0.95) - 1], 2),
              "of": f"{len(per)} batches of {copies} back-to-back launches, us per launch"}

    result = {
        "metric": "Q4 GEMV GB/s at 4096x14336 b=1",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us * 1e-3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32 (f16 activations x exact int4 weights on f16 MFMA, fp32 accumulate, f16 scale applied in fp32)",
        "data": "synthetic (seeded Philox: W~N(0,0.02) quantised per 32-group, x~N(0,1))",
        "config": {"workload": "Q4 decode GEMV, K=4096 -> N=14336, M=1, x f16, y f32 (BASELINE configs[1])",
                   "weight_copies_rotated": int(copies), "algorithmic_bytes_per_step": int(alg_bytes)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": TRAFFIC_DECODE_BYTES},
        "parity_rel_l2": rel_l2,
        "single_launch_us": round(lat[len(lat) // 2], 2),
        "us_per_launch_spread": spread,
    }

    if not args.no_extra:
        extra = {}
        # prefill GEMM, M = 512, bf16 activations (the second kernel of the path)
        Mp = 512
        xp = torch.from_numpy(synth.activations(4, Mp, K)).to(dev).to(torch.bfloat16)
        yp = torch.empty((Mp, N), dtype=torch.float32, device=dev)
        be.matmul(w0, xp, yp, stream=stream)
        torch.cuda.synchronize()
        refp = xp.double() @ torch.from_numpy(formats.dequantize(q, s)).to(dev).double().T
        relp = float(((yp.double() - refp).norm() / refp.norm()).item())
        del refp
        nrep = 50
        planp = be.plan_many([ws[i % copies] for i in range(nrep)], [xp] * nrep, [yp] * nrep)
        be.matmul_many(planp, Mp, stream)
        elp = timed_many(be, planp, Mp, stream, torch) / nrep
        tfl = 2.0 * Mp * N * K / elp / 1e12
        extra["prefill_gemm_M512"] = {
            "workload": "Q4 prefill GEMM, M=512, K=4096 -> N=14336, X bf16, Y f32 (BASELINE configs[3])",
            "us": round(elp * 1e6, 1), "tflops": round(tfl, 1), "parity_rel_l2": relp,
            "roofline": {"bound": "mfma", "achieved": round(tfl, 1), "peak": MFMA_BF16_PEAK_TFLOPS,
                         "unit": "TFLOP/s", "frac": round(tfl / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": TRAFFIC_PREFILL_M512_BYTES}}
        log(f"prefill GEMM M=512: {elp * 1e6:.1f} us, {tfl:.1f} TFLOP/s, rel_l2 {relp:.2e}")
        # batch sweep of the decode kernel on the same shape
        sweep = {}
        for Mb in (4, 8, 16):
            xb = torch.from_numpy(synth.activations(3, Mb, K, outliers=0.001)).to(dev).to(torch.float16)
            yb = torch.empty((Mb, N), dtype=torch.float32, device=dev)
            n = 240
            pl = be.plan_many([ws[i % copies] for i in range(n)], [xb] * n, [yb] * n)
            be.matmul_many(pl, Mb, stream)
            e = timed_many(be, pl, Mb, stream, torch) / n
            sweep[f"M{Mb}"] = {"us": round(e * 1e6, 2),
                               "GB/s": round(formats.matmul_bytes(bits, N, K, Mb, 2, 4) / e / 1e9, 1)}
        extra["decode_batch_sweep_4096x14336"] = sweep
        # the sweep's second shape, the down projection (BASELINE configs[2]): 256 strips of 112 K tiles
        for t in ws[1:]:
            t.free()
        del ws[1:]
        qd, sd = formats.quantize(synth.weights(6, K, N), bits)
        wd = [be.upload_quantized(qd, sd, bits)]
        wd += [wd[0].clone() for _ in range(copies - 1)]
        del qd, sd
        sweep_d = {}
        for Mb in (1, 4, 8, 16):
            xb = torch.from_numpy(synth.activations(3, Mb, N, outliers=0.001)).to(dev).to(torch.float16)
            yb = torch.empty((Mb, K), dtype=torch.float32, device=dev)
            n = 240
            pl = be.plan_many([wd[i % copies] for i in range(n)], [xb] * n, [yb] * n)
            be.matmul_many(pl, Mb, stream)
            e = timed_many(be, pl, Mb, stream, torch) / n
            sweep_d[f"M{Mb}"] = {"us": round(e * 1e6, 2),
                                 "GB/s": round(formats.matmul_bytes(bits, K, N, Mb, 2, 4) / e / 1e9, 1)}
        extra["decode_batch_sweep_14336x4096"] = sweep_d
        for t in wd:
            t.free()
        del wd
        # the same kernel on Q8 blocks (twice the bytes per weight, half the unpack work per byte):
        # shows how much of the Q4 time is arithmetic rather than memory
        q8, s8 = formats.quantize(synth.weights(2, N, K), formats.Q8)
        n8 = max(2, (3 * MALL_BYTES) // formats.weight_bytes(formats.Q8, N, K) + 1)
        w8 = [be.upload_quantized(q8, s8, formats.Q8)]
        w8 += [w8[0].clone() for _ in range(n8 - 1)]
        del q8, s8
        q8res = {}
        for Mb in (1, 8):
            xb = torch.from_numpy(synth.activations(3, Mb, K)).to(dev).to(torch.float16)
            yb = torch.empty((Mb, N), dtype=torch.float32, device=dev)
            n = 240
            pl = be.plan_many([w8[i % n8] for i in range(n)], [xb] * n, [yb] * n)
            be.matmul_many(pl, Mb, stream)
            e = timed_many(be, pl, Mb, stream, torch) / n
            gbs = formats.matmul_bytes(formats.Q8, N, K, Mb, 2, 4) / e / 1e9
            q8res[f"M{Mb}"] = {"us": round(e * 1e6, 2), "GB/s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4)}
        extra["q8_decode_4096x14336"] = q8res
        for t in w8:
            t.free()
        del w8
        # the reference-shaped decode step: 32 layers x (q,k,v,o,gate,up,down), Q4, random init,
        # one native walk over the 224 linear nodes per step (BASELINE configs[4])
        from cyb_amd import stack as stk
        stack_out = {}
        for label, shapes, epis in (("per_linear_224_launches", None, False),
                                    ("qkv_and_gate_up_fused_128_launches", stk.fused_shapes(), False),
                                    ("fused_128_launches_swiglu_and_residual_epilogues", stk.fused_shapes(), True)):
            t0 = time.time()
            st = stk.build(be, layers=32, seed=5, shapes=shapes, order=list(shapes) if shapes else None, epilogues=epis)
            log(f"stack {label} built in {time.time() - t0:.1f}s: {st.weight_bytes} weight bytes")
            res = {"weight_bytes": int(st.weight_bytes), "launches_per_step": len(st.nodes)}
            for Ms in (1, 8):
                edges = stk.edges_for(st, Ms, shapes=shapes)
                pl = stk.plan(st, edges)
                be.matmul_many(pl, Ms, stream)
                reps = 20
                torch.cuda.synchronize()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                for _ in range(reps):
                    be.matmul_many(pl, Ms, stream)
                b.record()
                torch.cuda.synchronize()
                per = a.elapsed_time(b) * 1e-3 / reps
                res[f"M{Ms}"] = {"us_per_step": round(per * 1e6, 1),
                                 "GB/s": round(st.step_bytes(Ms) / per / 1e9, 1),
                                 "frac_of_hbm_peak": round(st.step_bytes(Ms) / per / 1e9 / HBM_PEAK_GBS, 4),
                                 "linear_stack_tok_per_s": round(Ms / per, 1)}
                log(f"decode stack {label} M={Ms}: {per * 1e6:.0f} us/step")
            if shapes is not None and not epis:
                # prefill of one 512-token chunk through the same stack (bf16 activations), and both
                # phases in the units the reference's UI reports (tok_in_s / tok_out_s,
                # /root/reference/shell/src/worlds/models/mod.rs:44-52): linears only, no attention
                Mp2 = 512
                edges = stk.edges_for(st, Mp2, shapes=shapes, xdtype=torch.bfloat16)
                pl = stk.plan(st, edges)
                be.matmul_many(pl, Mp2, stream)
                torch.cuda.synchronize()
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                for _ in range(3):
                    be.matmul_many(pl, Mp2, stream)
                b.record()
                torch.cuda.synchronize()
                per = a.elapsed_time(b) * 1e-3 / 3
                flops = sum(2.0 * Mp2 * w.N * w.K for w in st.weights)
                res["prefill_M512"] = {"ms_per_chunk": round(per * 1e3, 3), "TFLOP/s": round(flops / per / 1e12, 1),
                                       "frac_of_mfma_peak": round(flops / per / 1e12 / MFMA_BF16_PEAK_TFLOPS, 4)}
                res["linear_stack_tok_in_s"] = round(Mp2 / per, 1)
                res["linear_stack_tok_out_s"] = res["M1"]["linear_stack_tok_per_s"]
                log(f"prefill stack {label} M={Mp2}: {per * 1e3:.2f} ms/chunk, {flops / per / 1e12:.0f} TFLOP/s")
            stack_out[label] = res
            for t in st.weights:
                t.free()
            del st, pl, edges
        extra["decode_stack_llama3_8b_q4"] = stack_out
        result["extra"] = extra

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(q, s, x32, alg_bytes)
        log(f"cpu baseline: {result['cpu_baseline']}")

    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
