"""The decode-step linear stack: the caller loop around the op.

One decode step of a LlamaStyle model issues, per layer, the quantised matmuls
q, k, v, o, gate, up, down ("norm -> QKV -> RoPE -> KV cache -> attention -> O
proj -> residual -> norm -> FFN -> residual" x layers -
/root/reference/decide/pipeline.md:51).  This module builds that list of graph
nodes for a random-init Llama-3-8B-shaped model and runs it through
`cybq_matmul_many`.  The glue between the linears (norm, RoPE, attention,
SwiGLU) is not part of the path: every linear reads a fresh seeded N(0,1) f16
input of its width, so each output can be checked on its own.

Weights are generated and quantised on the device (torch.randn ->
cybq_quantize -> cybq_weight_from_device): 7 B weights never exist on the host.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List

from . import formats, synth
from .backend import Backend, QMatMul, QWeight

LINEAR_ORDER = ["q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj"]
_PREFIX = {"q_proj": "self_attn", "k_proj": "self_attn", "v_proj": "self_attn", "o_proj": "self_attn",
           "gate_proj": "mlp", "up_proj": "mlp", "down_proj": "mlp"}


def tensor_name(layer: int, lin: str) -> str:
    return f"model.layers.{layer}.{_PREFIX.get(lin, 'fused')}.{lin}.weight"


@dataclass
class LinearStack:
    backend: Backend
    layers: int
    bits: int
    nodes: List[QMatMul] = field(default_factory=list)
    weights: List[QWeight] = field(default_factory=list)
    planar: Dict[str, tuple] = field(default_factory=dict)     # name -> (q bytes, scales) kept for checks
    epilogues: List[str] = field(default_factory=list)         # per node: "none" | "add" | "swiglu" (empty = none anywhere)
    gammas: List[object] = field(default_factory=list)         # per node: RMSNorm weight folded in front of it, or None (empty = no norms)
    eps: float = 1e-5

    @property
    def weight_bytes(self) -> int:
        return sum(w.algorithmic_bytes for w in self.weights)

    def step_bytes(self, M: int) -> int:
        """Algorithmic HBM bytes of one step: every weight once, f16 inputs, f32 outputs."""
        return sum(formats.matmul_bytes(self.bits, w.N, w.K, M, 2, 4) for w in self.weights)


def fused_shapes(shapes: Dict[str, tuple] = None) -> Dict[str, tuple]:
    """q/k/v and gate/up read the same input: concatenating their rows at load time
    turns five launches into two (the outputs are column slices of one y)."""
    shapes = shapes or synth.LLAMA3_8B_LINEARS
    K = shapes["q_proj"][0]
    return {"qkv_proj": (K, shapes["q_proj"][1] + shapes["k_proj"][1] + shapes["v_proj"][1]),
            "o_proj": shapes["o_proj"],
            "gate_up_proj": (K, shapes["gate_proj"][1] + shapes["up_proj"][1]),
            "down_proj": shapes["down_proj"]}


NORMED = ("q_proj", "k_proj", "v_proj", "qkv_proj", "gate_proj", "up_proj", "gate_up_proj")      # linears that follow an RMSNorm


def build(backend: Backend, layers: int = 32, bits: int = formats.Q4, seed: int = 5, keep_planar=0,
          shapes: Dict[str, tuple] = None, order: List[str] = None, epilogues: bool = False, norms: bool = False) -> LinearStack:
    """Random-init stack with N(0, 0.02) weights quantised on the device.

    keep_planar: for the first that many layers (or for the layers listed), the PLANAR device
    buffers are kept in `stack.planar` so that a checker can pull them back and recompute outputs.
    epilogues: with the fused shapes, `gate_up_proj` becomes a strip-interleaved pair run with the
    SwiGLU epilogue (its output has half the columns) and `o_proj` / `down_proj` add a residual.
    norms: the linears that follow an RMSNorm in the decode loop (q / k / v, gate / up) get a seeded
    gamma (f16, 1 +- 0.1) per layer and norm, folded into their activation load."""
    import torch
    shapes = shapes or synth.LLAMA3_8B_LINEARS
    st = LinearStack(backend, layers, bits)
    gen = torch.Generator(device="cuda")
    gen.manual_seed((synth.BASE_SEED ^ seed) & 0x7FFFFFFF)
    order = order or [l for l in LINEAR_ORDER if l in shapes] or list(shapes)
    kept = set(range(keep_planar)) if isinstance(keep_planar, int) else set(keep_planar)
    for layer in range(layers):
        layer_gamma = {}
        for lin in order:
            K, N = shapes[lin]
            w = torch.empty((N, K), dtype=torch.float32, device="cuda").normal_(0.0, 0.02, generator=gen)
            qd = torch.empty(N * K * bits // 8, dtype=torch.uint8, device="cuda")
            sd = torch.empty(N * (K // 32), dtype=torch.int16, device="cuda")
            backend.quantize(bits, w, N, K, qd, sd)
            name = tensor_name(layer, lin)
            epi = "none"
            if epilogues and lin == "gate_up_proj":
                # rows [0, N/2) are the gate projection, [N/2, N) the up projection
                h = N // 2
                hq, hs = h * K * bits // 8, h * (K // 32)
                g = backend.weight_from_device(bits, h, K, qd[:hq], sd[:hs])
                u = backend.weight_from_device(bits, h, K, qd[hq:], sd[hs:])
                torch.cuda.synchronize()
                qw = backend.fuse_pairs(g, u, name=name)
                g.free()
                u.free()
                epi = "swiglu"
            else:
                qw = backend.weight_from_device(bits, N, K, qd, sd, name=name)
                if epilogues and lin in ("o_proj", "down_proj"):
                    epi = "add"
            torch.cuda.synchronize()              # qd / sd / w are released below
            st.weights.append(qw)
            st.nodes.append(QMatMul(w=name, x=f"in.{K}", y=f"out.{lin}", quant=bits, M=1, N=N, K=K))
            if epilogues:
                st.epilogues.append(epi)
            if norms:
                which = "input" if lin in ("q_proj", "k_proj", "v_proj", "qkv_proj") else "post_attention"
                if lin in NORMED and which not in layer_gamma:
                    layer_gamma[which] = (1.0 + 0.1 * torch.empty(K, dtype=torch.float32, device="cuda").normal_(generator=gen)).to(torch.float16)
                st.gammas.append(layer_gamma[which] if lin in NORMED else None)
            if layer in kept:
                st.planar[name] = (qd, sd)
            del w
    return st


def edges_for(stack: LinearStack, M: int, seed: int = 5, shapes: Dict[str, tuple] = None, xdtype=None):
    """Fresh seeded inputs (one per input width; f16 unless `xdtype` says otherwise) and f32
    outputs (one per linear kind)."""
    import torch
    shapes = shapes or synth.LLAMA3_8B_LINEARS
    edges = {}
    for i, K in enumerate(sorted({k for k, _ in shapes.values()})):
        x = torch.from_numpy(synth.activations(seed, M, K, stream=i)).cuda().to(xdtype or torch.float16)
        edges[f"in.{K}"] = x
    for lin in shapes:
        cols = shapes[lin][1] // 2 if (stack.epilogues and lin == "gate_up_proj") else shapes[lin][1]
        edges[f"out.{lin}"] = torch.empty((M, cols), dtype=torch.float32, device="cuda")
    if stack.epilogues:
        widths = sorted({shapes[lin][1] for lin in ("o_proj", "down_proj") if lin in shapes})
        for i, N in enumerate(widths):          # the residual stream entering o_proj / down_proj
            edges[f"res.{N}"] = torch.from_numpy(synth.activations(seed, M, N, stream=100 + i)).cuda()
    return edges


def plan(stack: LinearStack, edges):
    xs, ys = [edges[n.x] for n in stack.nodes], [edges[n.y] for n in stack.nodes]
    gammas = stack.gammas or None
    if not stack.epilogues:
        return stack.backend.plan_many(stack.weights, xs, ys, gammas=gammas, eps=stack.eps)
    res = [edges[f"res.{n.N}"] if e == "add" else None for n, e in zip(stack.nodes, stack.epilogues)]
    return stack.backend.plan_many(stack.weights, xs, ys, stack.epilogues, res, gammas=gammas, eps=stack.eps)
