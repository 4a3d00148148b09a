"""Rotary position encoding with half-split pairs (i, i + hd/2).

f_i = base^(-2 i / hd), angle = position * f_i
(internal/device/kernels.metal:430-463, host twin internal/device/cpu_ref.go:103-129).
The optional scaling of the frequencies has no counterpart in the reference.
`linear` divides every f_i by the factor.  `llama3`: with wavelength
L_i = 2 pi / f_i, L_i < original / high_freq_factor keeps f_i,
L_i > original / low_freq_factor gives f_i / factor, and between the two
s = (original / L_i - low) / (high - low), f_i' = (1 - s) f_i / factor + s f_i.

The table is computed once in float64 and handed to the kernel as a parameter,
so the kernel knows nothing about scaling types.
"""
from __future__ import annotations

import math
from typing import List, Mapping, Optional

import torch

from .base import POSITION_ENCODINGS, BuildEnv, PositionEncoding, StepContext


def rotary_frequencies(head_dim: int, base: float, scaling: Optional[Mapping] = None) -> List[float]:
    freqs = [base ** (-2.0 * i / head_dim) for i in range(head_dim // 2)]
    if not scaling:
        return freqs
    factor = float(scaling["factor"])
    kind = scaling.get("rope_type", "llama3")
    if kind == "linear":  # positions divided by the factor
        return [f / factor for f in freqs]
    if kind != "llama3":
        raise ValueError(f"rope scaling type {kind!r} is not known (known: 'linear', 'llama3')")
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    original = float(scaling["original_max_position_embeddings"])
    out = []
    for f in freqs:
        wavelen = 2.0 * math.pi / f
        if wavelen < original / high:
            out.append(f)
        elif wavelen > original / low:
            out.append(f / factor)
        else:
            s = (original / wavelen - low) / (high - low)
            out.append((1.0 - s) * f / factor + s * f)
    return out


@POSITION_ENCODINGS.register("rope")
class RotaryEncoding(PositionEncoding):
    graph_safe = True

    def __init__(self, head_dim: int, base: float, scaling: Optional[Mapping] = None) -> None:
        self.head_dim = int(head_dim)
        self.base = float(base)
        self.scaling = dict(scaling) if scaling else None
        self.table = rotary_frequencies(self.head_dim, self.base, self.scaling)

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        self.rotary_frequencies = torch.tensor(self.table, dtype=torch.float64, device=env.device)

    def cos_sin(self, ctx: StepContext) -> torch.Tensor:
        """cos and sin of every row's angles, float32 [rows, head_dim/2, 2]: the same for every layer
        of a step that rotates with these frequencies, so it is computed once and shared."""
        key = ("rope_cos_sin", tuple(self.table))
        table = ctx.shared.get(key)
        if table is None:
            table = ctx.ws.alloc((ctx.rows, self.head_dim // 2, 2), torch.float32, keep=True)
            ctx.kernels.rope_table(self.rotary_frequencies, ctx.row_pos, table)
            ctx.shared[key] = table
        return table

    def apply(self, q: torch.Tensor, k: torch.Tensor, ctx: StepContext) -> None:
        heads = q.shape[1] // self.head_dim
        kv_heads = k.shape[1] // self.head_dim
        ctx.kernels.rope_store(q, None, None, heads, 0, self.head_dim, self.rotary_frequencies, ctx.row_pos)
        ctx.kernels.rope_store(k, None, None, kv_heads, 0, self.head_dim, self.rotary_frequencies, ctx.row_pos)


@POSITION_ENCODINGS.register("none")
class NoPositionEncoding(PositionEncoding):
    graph_safe = True

    """Leaves q and k as they are (the mixer sees order through the causal mask only)."""

    def __init__(self, **_unused) -> None:
        pass

    def apply(self, q: torch.Tensor, k: torch.Tensor, ctx: StepContext) -> None:
        return None
