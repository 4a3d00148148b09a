"""Causal grouped-query attention over the paged cache.

q = n Wq^T, k = n Wk^T, v = n Wv^T (no biases), heads are contiguous blocks of
head_dim columns; q and k are position-encoded, k and v are written to the
cache, each row attends to the keys of its own sequence up to its own position,
then the output projection (internal/device/metal.go:1377-1430).  Query head h
reads kv head h // (heads / kv_heads); scores are scaled by `scale`
(1/sqrt(head_dim) in the reference, internal/device/kernels.metal:671-673).

The three projection matrices are concatenated at bind time so that one matrix
product makes q, k and v.
"""
from __future__ import annotations

import math
from typing import Dict, List, Mapping, Optional

import torch

from .base import (MIXERS, POSITION_ENCODINGS, BuildEnv, KVNeed, LayerCache, Mixer, PartSpec,
                   NormedRows, StepContext, TensorSpec, build_part, product_weight, project, project_into,
                   project_normed)


@MIXERS.register("gqa_attention")
class GQAttention(Mixer):
    @property
    def graph_safe(self) -> bool:
        return self.position.graph_safe

    def __init__(self, width: int, heads: int, kv_heads: int, head_dim: int, position: PartSpec,
                 prefix: str, scale: Optional[float] = None, window: int = 0,
                 names: Optional[Mapping[str, str]] = None) -> None:
        if heads % kv_heads != 0:
            raise ValueError(f"{heads} heads cannot share {kv_heads} kv heads evenly")
        self.width, self.heads, self.kv_heads, self.head_dim = int(width), int(heads), int(kv_heads), int(head_dim)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.window = int(window)
        n = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight"}
        n.update(names or {})
        self.names: Dict[str, str] = {key: f"{prefix}.{val}" for key, val in n.items()}
        self.position = build_part(POSITION_ENCODINGS, position)
        self.q_width = self.heads * self.head_dim
        self.kv_width = self.kv_heads * self.head_dim
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [
            TensorSpec(self.names["q"], (self.q_width, self.width)),
            TensorSpec(self.names["k"], (self.kv_width, self.width)),
            TensorSpec(self.names["v"], (self.kv_width, self.width)),
            TensorSpec(self.names["o"], (self.width, self.q_width)),
        ] + self.position.tensor_specs()

    def bind(self, tensors: Mapping[str, torch.Tensor], env: BuildEnv) -> None:
        super().bind(tensors, env)
        q, k, v = (tensors[self.names[key]] for key in ("q", "k", "v"))
        if not (q.dtype == k.dtype == v.dtype):
            raise ValueError(f"{self.names['q']}: q, k and v projections are stored in different dtypes")
        self.w_qkv = product_weight(env, torch.cat([q, k, v], dim=0))
        self.w_o = product_weight(env, tensors[self.names["o"]])
        self.position.bind(tensors, env)

    def cache_need(self) -> KVNeed:
        return KVNeed(self.kv_heads, self.head_dim, self.window)

    takes_normed_rows = True
    takes_residual_sink = True

    # the attention kernel's own rules, where the kernel object has them
    def length_bound(self, kernels, longest: int) -> int:
        ask = getattr(kernels, "decode_length_bound", None)
        return ask(longest) if ask is not None else super().length_bound(kernels, longest)

    def lengths_uneven(self, kernels, lengths) -> bool:
        ask = getattr(kernels, "decode_lengths_uneven", None)
        return bool(ask(lengths)) if ask is not None and self.window == 0 else False

    def _rotate_and_store(self, q, k, v, freqs, ctx: StepContext, cache: LayerCache) -> None:
        kn = ctx.kernels
        if freqs is None:
            self.position.apply(q, k, ctx)
        if cache.write:
            # the step's table of cos and sin, where the position encoding keeps one (the same for every layer)
            by_groups = getattr(kn, "rope_store_takes_table", lambda rows: False)(q.shape[0])
            table = self.position.cos_sin(ctx) if (by_groups and freqs is not None
                                                   and hasattr(self.position, "cos_sin")) else None
            kn.rope_store(q, k, v, self.heads, self.kv_heads, self.head_dim, freqs, ctx.row_pos,
                          ctx.row_seq, ctx.seq_slot, cache.block_table, cache.k, cache.v, cache.block_size,
                          cos_sin=table, cu_rows=ctx.cu_rows if table is not None else None)
        elif freqs is not None:
            kn.rope_store(q, None, None, self.heads, 0, self.head_dim, freqs, ctx.row_pos)

    def forward(self, h, ctx: StepContext, cache: Optional[LayerCache], sink=None) -> Optional[torch.Tensor]:
        if cache is None or cache.k is None:
            raise RuntimeError("attention needs a key/value cache")
        kn = ctx.kernels
        rows = h.shape[0]
        freqs = self.position.rotary_frequencies
        shape = (ctx.dtype, self.heads, self.kv_heads, self.head_dim, cache.block_size)
        # a decoding step can leave the rotation and the cache write to the attention kernel itself
        folded = (ctx.decode and cache.write and freqs is not None and hasattr(self.position, "cos_sin")
                  and getattr(kn, "attention_folds_rope", lambda *a: False)(*shape))
        width = self.q_width + 2 * self.kv_width
        # ... and then also the adding up of q, k and v, where the product would rather share K over blocks
        # (a few dozen rows: its columns alone are too few for the chip)
        pieces = 1
        if (folded and not isinstance(h, NormedRows) and self.w_qkv.dtype == h.dtype
                and getattr(kn, "attention_adds_pieces", lambda *a: False)(*shape)):
            pieces = kn.linear_pieces(h.dtype, rows, width, self.width)
        # A step of a few dozen to a few hundred rows that writes the cache through `rope_store`: the same, with
        # the pieces added up by the kernel that rotates (its columns alone would leave most of the chip idle,
        # every block reading all the rows).
        stored_pieces = False
        if (pieces == 1 and not folded and cache.write and freqs is not None and not isinstance(h, NormedRows)
                and self.w_qkv.dtype == h.dtype
                and getattr(kn, "rope_store_adds_pieces", lambda *a: False)(ctx.dtype, rows, self.heads, self.kv_heads,
                                                                            self.head_dim)):
            pieces = kn.linear_pieces(h.dtype, rows, width, self.width)
            stored_pieces = pieces > 1
        if stored_pieces:
            qkv = ctx.ws.alloc((pieces, rows, width), torch.float32)
            project(kn, ctx, h, self.w_qkv, qkv)
            q = ctx.ws.alloc((rows, self.q_width), ctx.dtype)
            kn.rope_store_pieces(qkv, q, self.heads, self.kv_heads, self.head_dim, freqs, ctx.row_pos, ctx.row_seq,
                                 ctx.seq_slot, cache.block_table, cache.k, cache.v, cache.block_size)
            k = v = None
        elif pieces > 1:
            qkv = ctx.ws.alloc((pieces, rows, width), torch.float32)
            project(kn, ctx, h, self.w_qkv, qkv)
            first, stride = qkv[0], qkv.stride(0)
        else:
            qkv = first = ctx.ws.alloc((rows, width), ctx.dtype)
            stride = 0
            if not project_normed(kn, ctx, h, self.w_qkv, qkv):
                if isinstance(h, NormedRows):
                    h = h.tensor(ctx)
                project(kn, ctx, h, self.w_qkv, qkv)
        if not stored_pieces:
            q = first[:, : self.q_width]
            k = first[:, self.q_width : self.q_width + self.kv_width]
            v = first[:, self.q_width + self.kv_width :]
        att = ctx.ws.alloc((rows, self.q_width), ctx.dtype)
        need = kn.attention_workspace(ctx.dtype, rows, self.heads, self.kv_heads, self.head_dim,
                                      cache.block_size, ctx.decode, ctx.max_len)
        scratch = ctx.ws.alloc((need,), torch.float32) if need else None
        if folded:
            more = dict(pieces=pieces, piece_stride=stride) if pieces > 1 else {}
            kn.attention(q, att, self.heads, self.kv_heads, self.head_dim, ctx.row_pos, ctx.row_seq,
                         ctx.seq_slot, ctx.cu_rows, cache.block_table, cache.k, cache.v, cache.block_size,
                         self.scale, self.window, decode=True, max_len=ctx.max_len, workspace=scratch,
                         k_new=k, v_new=v, cos_sin=self.position.cos_sin(ctx), uneven=ctx.uneven, **more)
        else:
            if not stored_pieces:  # (else q is rotated and the cache written already)
                self._rotate_and_store(q, k, v, freqs, ctx, cache)
            kn.attention(q, att, self.heads, self.kv_heads, self.head_dim, ctx.row_pos, ctx.row_seq,
                         ctx.seq_slot, ctx.cu_rows, cache.block_table, cache.k, cache.v, cache.block_size,
                         self.scale, self.window, decode=ctx.decode, max_len=ctx.max_len, workspace=scratch,
                         uneven=ctx.uneven)
        return project_into(kn, ctx, att, self.w_o, sink)
