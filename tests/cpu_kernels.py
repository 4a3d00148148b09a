"""A stand-in for the kernel library, written with torch operators on the CPU.

It exists only so that tests without a GPU can drive the engine's own code
(step function, cache, block tables, generation loop) and compare with the plain
implementation.  The package never imports it; on the product path there is no
CPU fallback.  Same method names and argument meanings as `HipKernels`.
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from longbow_quarrel_amd.kernels.dry import query


class CpuKernels:
    name = "cpu-test-standin"

    def __init__(self) -> None:
        self.force_generic = False
        self.calls = []

    def use_stream(self, stream) -> None:
        pass

    def embed(self, table, tokens, out):
        t = tokens[: out.shape[0]].long()
        known = (t >= 0) & (t < table.shape[0])  # no row of the table: zeros, as the library does
        out.copy_(table[t.clamp(0, table.shape[0] - 1)].float() * known[:, None])

    @staticmethod
    def _whole(delta, like):
        d = delta.float()
        return d.sum(0) if d.dim() == like.dim() + 1 else d

    @query
    def linear_pieces(self, dtype, m, n, k):
        return 1

    @query
    def linear_fused_parts(self, dtype, m, n, k):
        return 0

    def rmsnorm(self, x, weight, eps, out, delta=None):
        if delta is not None:
            x += self._whole(delta, x)
        ms = (x * x).sum(-1, keepdim=True) / x.shape[-1]
        out.copy_((x / torch.sqrt(ms + eps) * weight).to(out.dtype))

    def add(self, x, delta):
        x += self._whole(delta, x)

    def cast(self, src, out):
        out.copy_(src.to(out.dtype))

    def linear(self, x, w, out):
        assert x.dtype == w.dtype
        out.copy_((x.float() @ w.float().t()).to(out.dtype))

    def swiglu(self, gate_up, out):
        inner = out.shape[1]
        g = gate_up[:, :inner].float()
        u = gate_up[:, inner:].float()
        out.copy_((g / (1 + torch.exp(-g)) * u).to(out.dtype))

    def gather_rows(self, x, rows, out, delta=None):
        idx = rows[: out.shape[0]].long()
        v = x[idx]
        if delta is not None:
            v = v + self._whole(delta, x)[idx]
        out.copy_(v)

    @staticmethod
    def _rotate(x, heads, hd, freqs, pos):
        rows = x.shape[0]
        v = x[:, : heads * hd].float().reshape(rows, heads, hd).double()
        ang = pos[:rows].double()[:, None] * freqs[None, :]
        c, s = torch.cos(ang).float()[:, None, :], torch.sin(ang).float()[:, None, :]
        half = hd // 2
        a, b = v[..., :half].float(), v[..., half:].float()
        return torch.cat([a * c - b * s, a * s + b * c], dim=-1).reshape(rows, heads * hd)

    def rope_table(self, freqs, row_pos, table):
        ang = row_pos[: table.shape[0]].double()[:, None] * freqs.double()[None, :]
        table[:, :, 0] = torch.cos(ang).float()
        table[:, :, 1] = torch.sin(ang).float()

    def rope_store(self, q, k, v, heads, kv_heads, head_dim, freqs, row_pos, row_seq=None, seq_slot=None,
                   block_table=None, kcache=None, vcache=None, block_size=0, cos_sin=None, cu_rows=None):
        rows = q.shape[0]
        if freqs is not None:
            q[:, : heads * head_dim] = self._rotate(q, heads, head_dim, freqs, row_pos).to(q.dtype)
        if kcache is None:
            return
        kr = self._rotate(k, kv_heads, head_dim, freqs, row_pos) if freqs is not None \
            else k[:, : kv_heads * head_dim].float()
        kr = kr.to(q.dtype).reshape(rows, kv_heads, head_dim)
        vr = v[:, : kv_heads * head_dim].reshape(rows, kv_heads, head_dim)
        for r in range(rows):
            p = int(row_pos[r])
            slot = int(seq_slot[int(row_seq[r])])
            blk = int(block_table[slot, p // block_size])
            off = p % block_size
            kcache[blk, :, off, :] = kr[r]
            vcache[blk, :, :, off] = vr[r]

    @query
    def attention_workspace(self, dtype, rows, heads, kv_heads, head_dim, block_size, decode, max_len):
        return 0

    def attention(self, q, out, heads, kv_heads, head_dim, row_pos, row_seq, seq_slot, cu_rows, block_table,
                  kcache, vcache, block_size, scale, window=0, decode=False, max_len=0, workspace=None, uneven=False):
        rows = q.shape[0]
        group = heads // kv_heads
        for r in range(rows):
            p = int(row_pos[r])
            slot = int(seq_slot[int(row_seq[r])])
            lo = p - window + 1 if (window > 0 and p >= window) else 0
            ts = list(range(lo, p + 1))
            blks = [int(block_table[slot, t // block_size]) for t in ts]
            offs = [t % block_size for t in ts]
            kk = torch.stack([kcache[b, :, o, :] for b, o in zip(blks, offs)]).float()  # [T, kvh, hd]
            vv = torch.stack([vcache[b, :, :, o] for b, o in zip(blks, offs)]).float()
            for h in range(heads):
                g = h // group
                qv = q[r, h * head_dim : (h + 1) * head_dim].float()
                s = (kk[:, g] @ qv) * scale
                pr = torch.softmax(s, dim=0)
                out[r, h * head_dim : (h + 1) * head_dim] = (pr[:, None] * vv[:, g]).sum(0).to(out.dtype)

    # greedy sampling and the upkeep of a decoding batch's arrays, so that the generation loop runs here too
    def argmax(self, logits, out, scratch=None, seq_slot=None, recent=None, recent_n=None):
        rows = logits.shape[0]
        best = logits.argmax(dim=-1).to(torch.int32)
        bad = ~torch.isfinite(logits).all(dim=-1)
        out[:rows] = torch.where(bad, torch.full_like(best, -1), best)

    def advance(self, row_pos, seq_start, seq_len, batch):
        for t in (row_pos, seq_start, seq_len):
            t[:batch] += 1
