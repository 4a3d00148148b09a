"""Toy parts that tests register to show that the framework's files need no change for a new
mixer, feed-forward, position encoding or architecture.  They are not models of anything."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Mapping, Optional

import torch

import plain
from longbow_quarrel_amd.config.base import ModelConfig
from longbow_quarrel_amd.model import ModelSpec, Run
from longbow_quarrel_amd.parts.base import (FEED_FORWARDS, MIXERS, POSITION_ENCODINGS, BuildEnv, FeedForward,
                                            LayerCache, Mixer, PartSpec, PositionEncoding, StateNeed, StepContext,
                                            TensorSpec)
from longbow_quarrel_amd.registry import register_architecture, unregister_architecture


class DecayMixer(Mixer):
    """State of its own: s <- decay * s + h for every token in order; out = s . W^T.
    The state (width floats per sequence) lives in the cache's fixed-size store."""

    def __init__(self, width: int, decay: float, prefix: str) -> None:
        self.width, self.decay, self.name = width, decay, prefix + ".mix.weight"
        self.w: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.name, (self.width, self.width))]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.w = tensors[self.name]

    def cache_need(self) -> StateNeed:
        return StateNeed((self.width,), torch.float32)

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[LayerCache]) -> torch.Tensor:
        states = torch.empty((ctx.rows, self.width), dtype=torch.float32, device=h.device)
        row = 0
        for slot, n in zip(ctx.host_slots, ctx.host_new):
            s = cache.state[slot]
            for _ in range(n):
                s = self.decay * s + h[row].float()
                states[row] = s
                row += 1
            cache.state[slot] = s
        out = ctx.ws.alloc((ctx.rows, self.width), torch.float32)
        x = states.to(self.w.dtype)
        ctx.kernels.linear(x, self.w, out)
        return out


class RoutedFeedForward(FeedForward):
    """A feed-forward with routing: each row goes through the one of `experts` matrices that its
    router score picks (arg-max of h . R^T, scores in 32-bit)."""

    def __init__(self, width: int, experts: int, prefix: str) -> None:
        self.width, self.experts, self.prefix = width, experts, prefix
        self.router: Optional[torch.Tensor] = None
        self.mats: List[torch.Tensor] = []

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(f"{self.prefix}.router.weight", (self.experts, self.width))]
        specs += [TensorSpec(f"{self.prefix}.experts.{e}.weight", (self.width, self.width)) for e in range(self.experts)]
        return specs

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.router = tensors[f"{self.prefix}.router.weight"]
        self.mats = [tensors[f"{self.prefix}.experts.{e}.weight"] for e in range(self.experts)]

    def forward(self, h: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        scores = h.float() @ self.router.float().t()
        pick = scores.argmax(dim=-1)
        out = ctx.ws.alloc((ctx.rows, self.width), torch.float32)
        out.zero_()
        for e in range(self.experts):
            idx = (pick == e).nonzero().flatten()
            if idx.numel():
                part = torch.empty((idx.numel(), self.width), dtype=torch.float32, device=h.device)
                ctx.kernels.linear(h[idx].contiguous(), self.mats[e], part)
                out[idx] = part
        return out


class ShiftEncoding(PositionEncoding):
    """Another position encoding: adds position * step to the first element of every head of q and k."""

    def __init__(self, head_dim: int, step: float) -> None:
        self.head_dim, self.step = head_dim, step

    def apply(self, q: torch.Tensor, k: torch.Tensor, ctx: StepContext) -> None:
        pos = ctx.row_pos[: q.shape[0]].to(q.dtype) * self.step
        for t in (q, k):
            t[:, :: self.head_dim] += pos[:, None]


@dataclass(frozen=True)
class ToyConfig(ModelConfig):
    width: int
    vocab: int
    heads: int
    kv_heads: int
    head_dim: int
    experts: int
    decay: float
    eps: float
    architecture = "ToyForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls(d["width"], d["vocab"], d["heads"], d["kv_heads"], d["head_dim"], d["experts"], d["decay"], d["eps"])

    def to_dict(self):
        return {"architectures": [self.architecture], "width": self.width, "vocab": self.vocab, "heads": self.heads,
                "kv_heads": self.kv_heads, "head_dim": self.head_dim, "experts": self.experts, "decay": self.decay,
                "eps": self.eps, "torch_dtype": "float32"}


def toy_spec(c: ToyConfig) -> ModelSpec:
    """Layer 0: decay mixer + routed feed-forward.  Layer 1: attention with the shift encoding +
    SwiGLU.  Layer 2: attention + SwiGLU.  The schedule runs layers 0, 1, 2, 1: layer 1 twice (each
    run with a cache of its own), and the run of layer 2 reads the keys and values that the first run
    of layer 1 wrote (it writes none)."""
    def norm(name):
        return PartSpec("rmsnorm", {"width": c.width, "eps": c.eps, "name": name})

    def attn(i):
        return PartSpec("gqa_attention", {"width": c.width, "heads": c.heads, "kv_heads": c.kv_heads,
                                          "head_dim": c.head_dim, "prefix": f"layers.{i}.attn",
                                          "position": PartSpec("toy_shift", {"head_dim": c.head_dim, "step": 0.01})})

    layers = [
        PartSpec("prenorm", {"mixer": PartSpec("toy_decay", {"width": c.width, "decay": c.decay, "prefix": "layers.0"}),
                             "feed_forward": PartSpec("toy_routed", {"width": c.width, "experts": c.experts,
                                                                     "prefix": "layers.0.ffn"}),
                             "mixer_norm": norm("layers.0.n1"), "ffn_norm": norm("layers.0.n2")}),
        PartSpec("prenorm", {"mixer": attn(1), "feed_forward": PartSpec("swiglu", {"width": c.width, "inner": 2 * c.width,
                                                                                  "prefix": "layers.1.mlp"}),
                             "mixer_norm": norm("layers.1.n1"), "ffn_norm": norm("layers.1.n2")}),
        PartSpec("prenorm", {"mixer": attn(2), "feed_forward": PartSpec("swiglu", {"width": c.width, "inner": 2 * c.width,
                                                                                  "prefix": "layers.2.mlp"}),
                             "mixer_norm": norm("layers.2.n1"), "ffn_norm": norm("layers.2.n2")}),
    ]
    return ModelSpec(vocab_size=c.vocab, width=c.width, embedding_name="embed.weight", layers=tuple(layers),
                     schedule=(Run(0), Run(1), Run(2, cache_of=1), Run(1)),
                     final_norm=norm("final.weight"), head_name=None, tie_head=True)


def register_toys() -> None:
    MIXERS.register("toy_decay", DecayMixer)
    FEED_FORWARDS.register("toy_routed", RoutedFeedForward)
    POSITION_ENCODINGS.register("toy_shift", ShiftEncoding)
    register_architecture("ToyForCausalLM", ToyConfig, toy_spec)


def unregister_toys() -> None:
    MIXERS.unregister("toy_decay")
    FEED_FORWARDS.unregister("toy_routed")
    POSITION_ENCODINGS.unregister("toy_shift")
    unregister_architecture("ToyForCausalLM")


TOY = {"architectures": ["ToyForCausalLM"], "width": 48, "vocab": 53, "heads": 4, "kv_heads": 2, "head_dim": 16,
       "experts": 3, "decay": 0.7, "eps": 1e-5}


def plain_toy(c: Dict, t: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """The toy model over one whole sequence with the plain functions, float64."""
    f64 = torch.float64
    w = lambda n: t[n].to(f64)
    x = w("embed.weight")[tokens]
    n_tok = len(tokens)
    kv = {}

    def shift(v, heads):
        v = v.clone().view(n_tok, heads, c["head_dim"])
        v[:, :, 0] += torch.arange(n_tok, dtype=f64)[:, None] * 0.01
        return v

    def attention(i, n, run, own_cache):
        q = shift(plain.linear(n, w(f"layers.{i}.attn.q_proj.weight")), c["heads"])
        if own_cache:
            k = shift(plain.linear(n, w(f"layers.{i}.attn.k_proj.weight")), c["kv_heads"])
            v = plain.linear(n, w(f"layers.{i}.attn.v_proj.weight")).view(n_tok, c["kv_heads"], c["head_dim"])
            kv[run] = (k, v)
        k, v = kv[run if own_cache else 1]
        o = plain.attention(q, k, v).reshape(n_tok, -1)
        return plain.linear(o, w(f"layers.{i}.attn.o_proj.weight"))

    def swiglu_ffn(i, n):
        g = plain.linear(n, w(f"layers.{i}.mlp.gate_proj.weight"))
        u = plain.linear(n, w(f"layers.{i}.mlp.up_proj.weight"))
        return plain.linear(plain.swiglu(g, u), w(f"layers.{i}.mlp.down_proj.weight"))

    for run, (layer, own) in enumerate(((0, True), (1, True), (2, False), (1, True))):
        n = plain.rms_norm(x, w(f"layers.{layer}.n1"), c["eps"])
        if layer == 0:
            s = torch.zeros(c["width"], dtype=f64)
            states = []
            for r in range(n_tok):
                s = c["decay"] * s + n[r]
                states.append(s)
            x = x + plain.linear(torch.stack(states), w("layers.0.mix.weight"))
            n = plain.rms_norm(x, w("layers.0.n2"), c["eps"])
            pick = plain.linear(n, w("layers.0.ffn.router.weight")).argmax(dim=-1)
            out = torch.stack([plain.linear(n[r : r + 1], w(f"layers.0.ffn.experts.{int(pick[r])}.weight"))[0]
                               for r in range(n_tok)])
            x = x + out
        else:
            x = x + attention(layer, n, run, own)
            n = plain.rms_norm(x, w(f"layers.{layer}.n2"), c["eps"])
            x = x + swiglu_ffn(layer, n)
    return plain.linear(plain.rms_norm(x, w("final.weight"), c["eps"]), w("embed.weight"))
