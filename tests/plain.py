"""Plain, slow implementation of the Llama 3 dense decoder and of the sampler.

Whole sequences, no cache, one function per part, float64 by default.  It shares
no code with the package under test: tests import the package for the engine
and this module for the expected values.  Every function cites the place in the
reference (paths relative to the reference's root) whose formula it follows.

`act` is an optional rounding hook.  The bfloat16 engine rounds activations at
fixed places (norm output, projections, attention output, the SwiGLU product);
passing `act=round_bf16` rounds at the same places so that the comparison sees
accumulation-order noise only.  The default is the identity: pure float64.
"""
from __future__ import annotations

import math
from typing import Callable, Optional, Sequence

import torch

F64 = torch.float64


def identity(x: torch.Tensor) -> torch.Tensor:
    return x


def round_bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.float32).to(torch.bfloat16).to(F64)


# --------------------------------------------------------------------------- parts


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * w, eps inside the root, weight after.

    internal/device/kernels.metal:905-942 (rmsnorm_f32_to_f16_v4),
    internal/device/cpu_ref.go:63-83 (CPURMSNorm).
    """
    x = x.to(F64)
    ms = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    return x / torch.sqrt(ms + eps) * w.to(F64)


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y[m, n] = sum_k x[m, k] * w[n, k]; weights are [out, in], no bias.

    internal/device/cpu_ref.go:85-100 (CPUMatMul, "B is transposed"),
    internal/device/kernels.metal:105-132 (linear_f16).
    """
    x = x.to(F64)
    w = w.to(F64)
    out = torch.zeros(x.shape[0], w.shape[0], dtype=F64)
    for n in range(w.shape[0]):
        out[:, n] = (x * w[n]).sum(dim=-1)
    return out


def rope_frequencies(head_dim: int, base: float) -> torch.Tensor:
    """f_i = base^(-2 i / head_dim) for i in [0, head_dim / 2).

    internal/device/kernels.metal:452 (pow(ropeTheta, -2 i / headDim)),
    internal/device/cpu_ref.go:116.
    """
    return torch.tensor(
        [math.pow(base, -2.0 * i / head_dim) for i in range(head_dim // 2)], dtype=F64
    )


def llama3_scaled_frequencies(
    freqs: torch.Tensor,
    factor: float,
    low_freq_factor: float,
    high_freq_factor: float,
    original_max_position: int,
) -> torch.Tensor:
    """The `llama3` rope_scaling type of config.json.  The reference has no
    frequency scaling (internal/device/kernels.metal:430-463 uses f_i as is), so
    nothing there fixes this rule; tests pin it by its invariants.  With
    wavelength L_i = 2 pi / f_i: L_i < original/high_freq_factor keeps f_i,
    L_i > original/low_freq_factor gives f_i / factor, and between the two
    s = (original / L_i - low) / (high - low), f_i' = (1 - s) f_i / factor + s f_i.
    """
    out = []
    lo_wavelen = original_max_position / low_freq_factor
    hi_wavelen = original_max_position / high_freq_factor
    for f in freqs.tolist():
        wavelen = 2.0 * math.pi / f
        if wavelen < hi_wavelen:
            out.append(f)
        elif wavelen > lo_wavelen:
            out.append(f / factor)
        else:
            s = (original_max_position / wavelen - low_freq_factor) / (
                high_freq_factor - low_freq_factor
            )
            out.append((1.0 - s) * f / factor + s * f)
    return torch.tensor(out, dtype=F64)


def rope(x: torch.Tensor, positions: Sequence[int], freqs: torch.Tensor) -> torch.Tensor:
    """Half-split rotation of x[t, heads, head_dim]: the pair is (i, i + hd/2),
    angle = position * f_i, x_i' = x_i cos - x_{i+hd/2} sin,
    x_{i+hd/2}' = x_i sin + x_{i+hd/2} cos.

    internal/device/kernels.metal:430-463 (rope_f16),
    internal/device/cpu_ref.go:103-129 (CPURoPE).
    """
    x = x.to(F64)
    t, heads, hd = x.shape
    half = hd // 2
    out = x.clone()
    for r in range(t):
        for i in range(half):
            ang = float(positions[r]) * float(freqs[i])
            c, s = math.cos(ang), math.sin(ang)
            a = x[r, :, i]
            b = x[r, :, i + half]
            out[r, :, i] = a * c - b * s
            out[r, :, i + half] = a * s + b * c
    return out


def attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    window: int = 0,
    scale: Optional[float] = None,
    rows: Optional[Sequence[int]] = None,
) -> torch.Tensor:
    """Causal grouped-query attention over one whole sequence (`rows`: only these positions'
    outputs are worked out, the others stay zero; for tests with thousands of keys).

    q[t, nh, hd], k[t, nkv, hd], v[t, nkv, hd] -> out[t, nh, hd].  Query head h
    reads kv head h // (nh / nkv); row p sees keys start..p with start = 0 or
    p - window + 1 when a window is active; score = q.k / sqrt(hd); softmax in
    full precision (the maximum starts from -inf here, not -10000).

    internal/device/kernels.metal:657-766 (att_fused_f16: kvh at :671,
    scale at :673, window start at :676, scores :696-705, softmax :708-752,
    values :755-765); host twin internal/device/cpu_ref.go:10-60.
    """
    q, k, v = q.to(F64), k.to(F64), v.to(F64)
    t, nh, hd = q.shape
    nkv = k.shape[1]
    group = nh // nkv
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    out = torch.zeros(t, nh, hd, dtype=F64)
    for p in (range(t) if rows is None else rows):
        start = p - window + 1 if (window > 0 and p >= window) else 0
        for h in range(nh):
            g = h // group
            scores = (k[start : p + 1, g] * q[p, h]).sum(dim=-1) * scale
            e = torch.exp(scores - scores.max())
            probs = e / e.sum()
            out[p, h] = (probs[:, None] * v[start : p + 1, g]).sum(dim=0)
    return out


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up with silu(g) = g / (1 + exp(-g)); no clamps.

    internal/device/cpu_ref.go:132-149 (CPUSwiGLU),
    internal/device/cuda_kernels.cu:28-37 (swiglu_kernel).
    """
    gate, up = gate.to(F64), up.to(F64)
    return gate / (1.0 + torch.exp(-gate)) * up


# --------------------------------------------------------------------------- model


class PlainLlama:
    """Weights by their safetensors names plus the numbers of config.json."""

    def __init__(self, config: dict, tensors: dict):
        self.c = config
        self.t = tensors
        c = config
        self.nh = c["num_attention_heads"]
        self.nkv = c.get("num_key_value_heads", self.nh)
        self.hd = c.get("head_dim") or c["hidden_size"] // self.nh
        self.eps = c.get("rms_norm_eps", 1e-5)
        freqs = rope_frequencies(self.hd, c.get("rope_theta", 10000.0))
        rs = c.get("rope_scaling")
        if rs and rs.get("rope_type", rs.get("type")) == "linear":
            freqs = freqs / rs["factor"]  # positions divided by the factor
        elif rs and rs.get("rope_type", rs.get("type")) != "default":
            freqs = llama3_scaled_frequencies(
                freqs,
                rs["factor"],
                rs["low_freq_factor"],
                rs["high_freq_factor"],
                rs["original_max_position_embeddings"],
            )
        self.freqs = freqs

    def w(self, name: str) -> torch.Tensor:
        return self.t[name].to(F64)

    def attention_block(self, layer: int, n: torch.Tensor, act: Callable) -> torch.Tensor:
        """Projections, rotation of q and k, attention, output projection.

        internal/device/metal.go:1377-1385 (q, k, v then RoPE on q and k),
        :1388-1424 (store, attend), :1428-1430 (output projection).
        """
        p = f"model.layers.{layer}.self_attn."
        t = n.shape[0]
        q = act(linear(n, self.w(p + "q_proj.weight"))).view(t, self.nh, self.hd)
        k = act(linear(n, self.w(p + "k_proj.weight"))).view(t, self.nkv, self.hd)
        v = act(linear(n, self.w(p + "v_proj.weight"))).view(t, self.nkv, self.hd)
        pos = list(range(t))
        q = act(rope(q, pos, self.freqs))
        k = act(rope(k, pos, self.freqs))
        o = act(attention(q, k, v)).reshape(t, self.nh * self.hd)
        return linear(o, self.w(p + "o_proj.weight"))

    def feed_forward(self, layer: int, n: torch.Tensor, act: Callable) -> torch.Tensor:
        """down(silu(gate(n)) * up(n)).  internal/device/metal.go:1464-1471."""
        p = f"model.layers.{layer}.mlp."
        g = linear(n, self.w(p + "gate_proj.weight"))
        u = linear(n, self.w(p + "up_proj.weight"))
        h = act(swiglu(g, u))
        return linear(h, self.w(p + "down_proj.weight"))

    def decoder_layer(self, layer: int, x: torch.Tensor, act: Callable) -> torch.Tensor:
        """Pre-norm block: x += attn(norm(x)); x += ffn(norm(x)).

        internal/device/metal.go:1326-1527 (Tensor.Layer: norm :1349, residual
        :1434, second norm :1451, residual :1474).
        """
        p = f"model.layers.{layer}."
        n = act(rms_norm(x, self.w(p + "input_layernorm.weight"), self.eps))
        x = x + self.attention_block(layer, n, act)
        n = act(rms_norm(x, self.w(p + "post_attention_layernorm.weight"), self.eps))
        x = x + self.feed_forward(layer, n, act)
        return x

    def forward(self, tokens: Sequence[int], act: Callable = identity) -> torch.Tensor:
        """Logits [len(tokens), vocab] of one whole sequence.

        Embedding row copy: internal/engine/engine.go:1365, 1375; layers
        :1409-1472; final norm and output head :1547-1561; the head is the
        embedding when the file has no output matrix (:1106-1116).
        """
        emb = self.w("model.embed_tokens.weight")
        x = emb[torch.tensor(list(tokens), dtype=torch.long)]
        for layer in range(self.c["num_hidden_layers"]):
            x = self.decoder_layer(layer, x, act)
        n = act(rms_norm(x, self.w("model.norm.weight"), self.eps))
        head = self.w("lm_head.weight") if "lm_head.weight" in self.t else emb
        return linear(n, head)


# --------------------------------------------------------------------------- sampler


def apply_repetition_penalty(logits: torch.Tensor, history: Sequence[int], penalty: float) -> torch.Tensor:
    """Each distinct id among the last 64 of the history: logit /= penalty if
    positive, else *= penalty.  Active when penalty > 1.

    internal/engine/sampler.go:249-275 (applyRepetitionPenalty), :77-79.
    """
    out = logits.clone()
    if penalty > 1.0 and len(history) > 0:
        for tok in set(history[-64:]):
            if tok < out.numel():
                out[tok] = out[tok] / penalty if out[tok] > 0 else out[tok] * penalty
    return out


def arg_max(logits: torch.Tensor) -> int:
    """First maximal index.  internal/engine/sampler.go:282-307 (argMax)."""
    best, idx = None, 0
    for i, v in enumerate(logits.tolist()):
        if best is None or v > best:
            best, idx = v, i
    return idx


def candidate_distribution(
    logits: torch.Tensor, temperature: float, top_k: int, top_p: float
) -> dict:
    """The distribution the reference draws from, as {token id: probability}.

    softmax(logits / T) in float64 (internal/engine/sampler.go:125-156), drop
    p <= 1e-10 (:158-166), sort descending (:92-94), keep the first k if
    0 < k < n (:309-314), then the shortest prefix whose mass reaches top_p,
    renormalised, if 0 < top_p < 1 (:316-339).  The draw itself is
    r = U[0,1) * sum(p), first candidate whose running sum exceeds r
    (:168-184), so this dict is the law of the drawn token.
    """
    z = logits.to(F64) / temperature
    e = torch.exp(z - z.max())
    probs = e / e.sum()
    cands = [(i, p) for i, p in enumerate(probs.tolist()) if p > 1e-10]
    cands.sort(key=lambda c: (-c[1], c[0]))
    if 0 < top_k < len(cands):
        cands = cands[:top_k]
    if 0.0 < top_p < 1.0:
        acc = 0.0
        for n, (_, p) in enumerate(cands):
            acc += p
            if acc >= top_p:
                cands = cands[: n + 1]
                break
    total = sum(p for _, p in cands)
    return {i: p / total for i, p in cands}


def draw(dist: dict, u: float) -> int:
    """Inverse-CDF draw over the candidates in descending order of probability.

    internal/engine/sampler.go:168-184 (sampleFromCandidates).
    """
    items = sorted(dist.items(), key=lambda c: (-c[1], c[0]))
    r = u * sum(p for _, p in items)
    acc = 0.0
    for i, p in items:
        acc += p
        if r < acc:
            return i
    return items[0][0]
