"""Toy parts that tests register to show that the framework's files need no change for a new
mixer, feed-forward, position encoding, embedding, step on the logits, kind of cache or architecture.
They are not models of anything."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Mapping, Optional

import torch

import plain
from longbow_quarrel_amd.cache import BLOCK_SIZE, CacheGroup, FreeList
from longbow_quarrel_amd.config.base import ModelConfig
from longbow_quarrel_amd.model import ModelSpec, Run
from longbow_quarrel_amd.parts.base import (EMBEDDINGS, FEED_FORWARDS, LOGIT_STEPS, MIXERS, POSITION_ENCODINGS,
                                            BuildEnv, CacheNeed, Embedding, FeedForward, LayerCache, LogitsStep,
                                            Mixer, PartSpec, PositionEncoding, StateNeed, StepContext, TensorSpec)
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

    # a rule of its own for what a captured decoding step is keyed by: bounds in steps of 500 tokens, and
    # "uneven" where one sequence holds more than three times another's tokens
    def length_bound(self, kernels, longest: int) -> int:
        return -(-longest // 500) * 500

    def lengths_uneven(self, kernels, lengths) -> bool:
        return max(lengths) > 3 * min(lengths)

    seen: List = []  # (max_len, uneven) of the decoding steps that reached forward

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: Optional[LayerCache]) -> torch.Tensor:
        if ctx.rows == len(ctx.host_slots):
            DecayMixer.seen.append((ctx.max_len, ctx.uneven))
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


class ScaledPositionalEmbedding(Embedding):
    """Another embedding: x = scale * E[token] + P[position], P a learned table of absolute positions."""

    def __init__(self, vocab: int, width: int, positions: int, scale: float) -> None:
        self.vocab, self.width, self.positions, self.scale = vocab, width, positions, scale
        self.table: Optional[torch.Tensor] = None
        self.pos_table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec("embed.weight", (self.vocab, self.width)),
                TensorSpec("embed.positions", (self.positions, self.width))]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.table, self.pos_table = tensors["embed.weight"], tensors["embed.positions"]

    def forward(self, ctx: StepContext) -> torch.Tensor:
        x = ctx.ws.alloc((ctx.rows, self.width), torch.float32, keep=True)
        ctx.kernels.embed(self.table, ctx.tokens, x)
        if not ctx.dry:
            x.mul_(self.scale).add_(self.pos_table[ctx.row_pos[: ctx.rows].long()].float())
        return x


class SoftCap(LogitsStep):
    """A step on the logits: cap * tanh(logits / cap)."""

    def __init__(self, cap: float) -> None:
        self.cap = cap

    def forward(self, logits: torch.Tensor, ctx: StepContext) -> None:
        if not ctx.dry:
            logits.copy_(self.cap * torch.tanh(logits / self.cap))


@dataclass(frozen=True)
class LatentNeed(CacheNeed):
    """A third kind of cache: one latent vector of `width` floats per position (neither keys and values
    per head nor a state of fixed size).  It builds its own group."""

    width: int

    def make_group(self, runs, n_blocks, max_slots, dtype, device):
        return LatentGroup(self, runs, n_blocks, max_slots, device)


class LatentView:
    """What the latent mixer receives as its cache."""

    def __init__(self, rows: torch.Tensor, owned: List[List[int]], write: bool = True) -> None:
        self.rows, self.owned, self.write = rows, owned, write

    def read_only(self) -> "LatentView":
        return LatentView(self.rows, self.owned, False)


class LatentGroup(CacheGroup):
    """rows [runs, blocks, BLOCK_SIZE, width] and, per slot, the list of blocks it owns (on the host:
    the toy mixer is written with host loops)."""

    def __init__(self, need: LatentNeed, runs: List[int], n_blocks: int, max_slots: int, device) -> None:
        self.layers = list(runs)
        self.blocks = FreeList(n_blocks, "latent block")
        self.rows = torch.zeros((len(runs), n_blocks, BLOCK_SIZE, need.width), dtype=torch.float32, device=device)
        self.owned: List[List[int]] = [[] for _ in range(max_slots)]

    def layer_view(self, layer: int) -> LatentView:
        return LatentView(self.rows[self.layers.index(layer)], self.owned)

    def free_blocks(self) -> int:
        return self.blocks.free_count

    def taken_blocks(self) -> int:
        return self.blocks.taken_count

    def blocks_for(self, tokens: int) -> int:
        return (tokens + BLOCK_SIZE - 1) // BLOCK_SIZE

    def blocks_missing(self, slot: int, new_len: int) -> int:
        return max(0, self.blocks_for(new_len) - len(self.owned[slot]))

    def ensure(self, slot: int, new_len: int) -> None:
        self.owned[slot].extend(self.blocks.take_many(self.blocks_missing(slot, new_len)))

    def release(self, slot: int) -> None:
        for b in self.owned[slot]:
            self.blocks.give(b)
        self.owned[slot] = []


class LatentMixer(Mixer):
    """c_t = h_t . Wc^T is stored for every position; m_t = sum_s softmax_s(c_t . c_s) c_s over s <= t;
    out = m_t . Wu^T."""

    def __init__(self, width: int, latent: int, prefix: str) -> None:
        self.width, self.latent, self.prefix = width, latent, prefix
        self.wc: Optional[torch.Tensor] = None
        self.wu: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.prefix + ".down.weight", (self.latent, self.width)),
                TensorSpec(self.prefix + ".up.weight", (self.width, self.latent))]

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.wc, self.wu = tensors[self.prefix + ".down.weight"], tensors[self.prefix + ".up.weight"]

    def cache_need(self) -> LatentNeed:
        return LatentNeed(self.latent)

    def forward(self, h: torch.Tensor, ctx: StepContext, cache: LatentView) -> torch.Tensor:
        c = torch.empty((ctx.rows, self.latent), dtype=torch.float32, device=h.device)
        ctx.kernels.linear(h.contiguous(), self.wc, c)
        mixed = torch.empty_like(c)
        row = 0
        for slot, start, n in zip(ctx.host_slots, ctx.host_start, ctx.host_new):
            owned = cache.owned[slot]
            for j in range(n):
                p = start + j
                cache.rows[owned[p // BLOCK_SIZE], p % BLOCK_SIZE] = c[row]
                past = torch.cat([cache.rows[b] for b in owned[: p // BLOCK_SIZE + 1]])[: p + 1]
                mixed[row] = torch.softmax(past @ c[row], dim=0) @ past
                row += 1
        out = ctx.ws.alloc((ctx.rows, self.width), torch.float32)
        ctx.kernels.linear(mixed.to(self.wu.dtype), self.wu, out)
        return out


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
    latent: int
    positions: int
    embed_scale: float
    cap: float
    architecture = "ToyForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls(*(d[k] for k in ("width", "vocab", "heads", "kv_heads", "head_dim", "experts", "decay", "eps",
                                    "latent", "positions", "embed_scale", "cap")))

    def to_dict(self):
        return {"architectures": [self.architecture], "width": self.width, "vocab": self.vocab, "heads": self.heads,
                "kv_heads": self.kv_heads, "head_dim": self.head_dim, "experts": self.experts, "decay": self.decay,
                "eps": self.eps, "latent": self.latent, "positions": self.positions, "embed_scale": self.embed_scale,
                "cap": self.cap, "torch_dtype": "float32"}


def toy_spec(c: ToyConfig) -> ModelSpec:
    """Layer 0: decay mixer + routed feed-forward.  Layer 1: attention with the shift encoding +
    SwiGLU.  Layer 2: attention + SwiGLU.  Layer 3: the latent mixer (a cache kind of its own) + SwiGLU.
    The schedule runs layers 0, 1, 2, 1, 3: layer 1 twice (each run with a cache of its own), and the run
    of layer 2 reads the keys and values that the first run of layer 1 wrote (it writes none).  The
    embedding is scaled and adds a learned absolute position; the logits are soft-capped."""
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
        PartSpec("prenorm", {"mixer": PartSpec("toy_latent", {"width": c.width, "latent": c.latent, "prefix": "layers.3.mix"}),
                             "feed_forward": PartSpec("swiglu", {"width": c.width, "inner": 2 * c.width,
                                                                 "prefix": "layers.3.mlp"}),
                             "mixer_norm": norm("layers.3.n1"), "ffn_norm": norm("layers.3.n2")}),
    ]
    return ModelSpec(vocab_size=c.vocab, width=c.width,
                     embedding=PartSpec("toy_scaled_positions", {"vocab": c.vocab, "width": c.width,
                                                                 "positions": c.positions, "scale": c.embed_scale}),
                     layers=tuple(layers), schedule=(Run(0), Run(1), Run(2, cache_of=1), Run(1), Run(3)),
                     final_norm=norm("final.weight"), head_name=None, tie_head=True,
                     logits_step=PartSpec("toy_soft_cap", {"cap": c.cap}), max_positions=c.positions)


def register_toys() -> None:
    MIXERS.register("toy_decay", DecayMixer)
    FEED_FORWARDS.register("toy_routed", RoutedFeedForward)
    POSITION_ENCODINGS.register("toy_shift", ShiftEncoding)
    MIXERS.register("toy_latent", LatentMixer)
    EMBEDDINGS.register("toy_scaled_positions", ScaledPositionalEmbedding)
    LOGIT_STEPS.register("toy_soft_cap", SoftCap)
    register_architecture("ToyForCausalLM", ToyConfig, toy_spec)


def unregister_toys() -> None:
    MIXERS.unregister("toy_decay")
    FEED_FORWARDS.unregister("toy_routed")
    POSITION_ENCODINGS.unregister("toy_shift")
    MIXERS.unregister("toy_latent")
    EMBEDDINGS.unregister("toy_scaled_positions")
    LOGIT_STEPS.unregister("toy_soft_cap")
    unregister_architecture("ToyForCausalLM")


TOY = {"architectures": ["ToyForCausalLM"], "width": 48, "vocab": 53, "heads": 4, "kv_heads": 2, "head_dim": 16,
       "experts": 3, "decay": 0.7, "eps": 1e-5, "latent": 6, "positions": 96, "embed_scale": 1.7, "cap": 4.0}


def plain_toy(c: Dict, t: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """The toy model over one whole sequence with the plain functions, float64."""
    f64 = torch.float64
    w = lambda n: t[n].to(f64)
    n_tok = len(tokens)
    x = c["embed_scale"] * w("embed.weight")[tokens] + w("embed.positions")[:n_tok]
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

    for run, (layer, own) in enumerate(((0, True), (1, True), (2, False), (1, True), (3, True))):
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
        elif layer == 3:
            lat = plain.linear(n, w("layers.3.mix.down.weight"))
            mixed = torch.stack([torch.softmax(lat[: r + 1] @ lat[r], dim=0) @ lat[: r + 1] for r in range(n_tok)])
            x = x + plain.linear(mixed, w("layers.3.mix.up.weight"))
            n = plain.rms_norm(x, w("layers.3.n2"), c["eps"])
            x = x + swiglu_ffn(3, n)
        else:
            x = x + attention(layer, n, run, own)
            n = plain.rms_norm(x, w(f"layers.{layer}.n2"), c["eps"])
            x = x + swiglu_ffn(layer, n)
    logits = plain.linear(plain.rms_norm(x, w("final.weight"), c["eps"]), w("embed.weight"))
    return c["cap"] * torch.tanh(logits / c["cap"])
