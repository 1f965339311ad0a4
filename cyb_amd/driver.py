"""A soma-style driver over the linear stack: the caller loop of the op, reporting in
the reference's own units.

The reference's mind streams events to its UI while it answers -
`Prefill { done, total }` while it reads the question, one `Delta` per generated
piece, then `Answer { tokens, tok_per_s, tok_in_s, tok_out_s, .. }`
(/root/reference/shell/src/worlds/soma_bridge.rs:252-277); the UI keeps running
means of `tok_in_s` / `tok_out_s` (/root/reference/shell/src/worlds/models/mod.rs:44-52)
and compares them with `SPEED_ANCHORS` (same file, :116).  This module walks the
same two phases over the quantised linears only:

  prefill  the prompt in chunks of `chunk` tokens, every chunk one pass of
           `cybq_matmul_many` over the stack with bf16 activations (M = chunk),
  decode   one pass per new token with f16 activations (M = batch).

Attention, norms, RoPE, sampling and the tokenizer are not part of the path, so the
rates are those of the weight-bound part of a step; they are upper bounds for a
whole model.  Nothing is computed on the host.
"""
from __future__ import annotations

import time
from dataclasses import dataclass
from typing import Dict, Iterator, Optional

from . import stack as stk
from .backend import Backend


@dataclass
class Answer:
    tokens: int            # generated tokens
    tok_per_s: float       # (prompt + generated) / wall time of the whole ask
    tok_in_s: float        # prompt tokens / prefill time
    tok_out_s: float       # generated tokens / decode time


def ask(backend: Backend, st: stk.LinearStack, prompt_tokens: int, new_tokens: int, chunk: int = 512,
        batch: int = 1, shapes: Optional[Dict[str, tuple]] = None, stream: int = 0) -> Iterator[dict]:
    """Yields {"Prefill": {"done", "total"}} per chunk, {"Delta": i} per decode step and finally
    {"Answer": Answer}.  Device work is timed with events on the launch stream."""
    import torch
    if prompt_tokens < 0 or new_tokens < 0 or chunk < 1 or batch < 1 or batch > 16:
        raise ValueError("prompt_tokens, new_tokens >= 0; chunk >= 1; 1 <= batch <= 16")
    t_wall = time.time()
    yield {"Prefill": {"done": 0, "total": prompt_tokens}}
    ms_in = 0.0
    plans = {}

    def plan_for(M: int, xdtype):
        if M not in plans:
            edges = stk.edges_for(st, M, shapes=shapes, xdtype=xdtype)
            plans[M] = (stk.plan(st, edges), edges)
        return plans[M][0]

    done = 0
    while done < prompt_tokens:
        M = min(chunk, prompt_tokens - done)
        pl = plan_for(M, torch.bfloat16 if M > 16 else torch.float16)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        backend.matmul_many(pl, M, stream)
        b.record()
        b.synchronize()
        ms_in += a.elapsed_time(b)
        done += M
        yield {"Prefill": {"done": done, "total": prompt_tokens}}

    ms_out = 0.0
    if new_tokens:
        pl = plan_for(batch, torch.float16)
        backend.matmul_many(pl, batch, stream)                 # first touch of this plan's buffers, untimed
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(new_tokens):
            backend.matmul_many(pl, batch, stream)
        b.record()
        b.synchronize()
        ms_out = a.elapsed_time(b)
        for i in range(new_tokens):
            yield {"Delta": i}
    wall = max(time.time() - t_wall, 1e-9)
    yield {"Answer": Answer(tokens=new_tokens * batch,
                            tok_per_s=(prompt_tokens + new_tokens * batch) / wall,
                            tok_in_s=prompt_tokens / (ms_in * 1e-3) if ms_in else 0.0,
                            tok_out_s=new_tokens * batch / (ms_out * 1e-3) if ms_out else 0.0)}


def main(argv=None) -> int:
    import argparse
    ap = argparse.ArgumentParser(description="prefill / decode rates of the quantised linear stack (Llama-3-8B shapes, random init)")
    ap.add_argument("--prompt", type=int, default=2048)
    ap.add_argument("--new", type=int, default=128)
    ap.add_argument("--chunk", type=int, default=512)
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--layers", type=int, default=32)
    ap.add_argument("--separate", action="store_true", help="q/k/v and gate/up as separate launches (224 per step)")
    ap.add_argument("--epilogues", action="store_true", help="SwiGLU and residual adds fused into the linears")
    args = ap.parse_args(argv)
    import torch
    torch.cuda.init()          # torch brings its own HIP runtime: let it find the device before libcybq does
    be = Backend(0)
    shapes = None if args.separate else stk.fused_shapes()
    st = stk.build(be, layers=args.layers, shapes=shapes, order=list(shapes) if shapes else None,
                   epilogues=args.epilogues and shapes is not None)
    for ev in ask(be, st, args.prompt, args.new, args.chunk, args.batch, shapes=shapes):
        if "Prefill" in ev:
            p = ev["Prefill"]
            print(f"reading {p['done']} / {p['total']}", flush=True)
        elif "Answer" in ev:
            a = ev["Answer"]
            print(f"tokens {a.tokens}  tok_in_s {a.tok_in_s:.1f}  tok_out_s {a.tok_out_s:.1f}  tok_per_s {a.tok_per_s:.1f}  "
                  f"({st.weight_bytes / 1e9:.2f} GB of Q{st.bits} weights, {len(st.nodes)} launches per step)", flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
