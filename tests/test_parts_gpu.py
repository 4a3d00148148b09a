"""Each part of a layer alone on the GPU against its plain formula: norm, position encoding, the
attention mixer, the feed-forward, and their arrangement in a block."""
import math

import pytest
import torch

import plain
from helpers import rel_err
from longbow_quarrel_amd.cache import CacheManager
from longbow_quarrel_amd.parts import (BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS, BuildEnv,
                                       PartSpec, StepContext, Workspace, build_part)
from longbow_quarrel_amd.weights import random_tensors

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


@pytest.fixture(scope="module")
def kn():
    from longbow_quarrel_amd.kernels.hip import HipKernels

    return HipKernels()


def i32(v):
    return torch.tensor(list(v), dtype=torch.int32, device=DEV)


def context(kn, dtype, lengths, new, slots):
    """Sequences that already hold lengths[b] - new[b] tokens and bring new[b] rows each."""
    row_seq, row_pos, cu, starts = [], [], [0], []
    for b, (n, m) in enumerate(zip(lengths, new)):
        row_seq += [b] * m
        row_pos += list(range(n - m, n))
        cu.append(cu[-1] + m)
        starts.append(n - m)
    rows = sum(new)
    return StepContext(kernels=kn, dtype=dtype, device=DEV, ws=Workspace(DEV), rows=rows, batch=len(lengths),
                       tokens=i32([0] * rows), row_seq=i32(row_seq), row_pos=i32(row_pos), seq_slot=i32(slots),
                       seq_start=i32(starts), seq_len=i32(lengths), cu_rows=i32(cu), host_slots=list(slots),
                       host_start=starts, host_new=list(new), max_new=max(new), max_len=max(lengths),
                       decode=all(m == 1 for m in new))


def bound(part, env, dtype, std=0.3, seed=5):
    tensors = random_tensors(part.tensor_specs(), seed, dtype, std, device=DEV)
    for s in part.tensor_specs():
        if s.kind == "vector32":
            tensors[s.name] = (tensors[s.name].float() + torch.randn(s.shape, device=DEV) * 0.3)
    part.bind(tensors, env)
    return {k: v.cpu() for k, v in tensors.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_part(kn, dtype):
    env = BuildEnv(dtype, DEV, kn)
    norm = build_part(NORMS, PartSpec("rmsnorm", {"width": 200, "eps": 3e-6, "name": "n.weight"}))
    t = bound(norm, env, dtype)
    ctx = context(kn, dtype, [5], [5], [0])
    x = torch.randn((5, 200), device=DEV) * 3
    d = torch.randn((5, 200), device=DEV)
    x0 = x.clone()
    out = norm.forward(x, ctx, delta=d)
    assert out.dtype == dtype
    assert rel_err(out, plain.rms_norm((x0 + d).cpu(), t["n.weight"], 3e-6)) < (2e-6 if dtype == torch.float32 else 5e-3)
    assert rel_err(x, (x0 + d).cpu()) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotary_encoding_alone_with_and_without_scaling(kn, dtype):
    env = BuildEnv(dtype, DEV, kn)
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 64}
    for sc in (None, scaling, {"rope_type": "linear", "factor": 4.0}):
        pos = build_part(POSITION_ENCODINGS, PartSpec("rope", {"head_dim": 32, "base": 500000.0, "scaling": sc}))
        pos.bind({}, env)
        want_f = plain.rope_frequencies(32, 500000.0)
        if sc and sc["rope_type"] == "linear":
            want_f = want_f / 4.0
        elif sc:
            want_f = plain.llama3_scaled_frequencies(want_f, 8.0, 1.0, 4.0, 64)
        assert torch.allclose(pos.rotary_frequencies.cpu(), want_f, rtol=1e-14, atol=0)
        ctx = context(kn, dtype, [300, 7], [4, 2], [1, 0])
        q = torch.randn((6, 3 * 32), device=DEV).to(dtype)
        k = torch.randn((6, 1 * 32), device=DEV).to(dtype)
        q0, k0 = q.clone(), k.clone()
        pos.apply(q, k, ctx)
        p = [296, 297, 298, 299, 5, 6]
        lim = 2e-6 if dtype == torch.float32 else 5e-3
        assert rel_err(q.view(6, 3, 32), plain.rope(q0.cpu().view(6, 3, 32), p, want_f)) < lim
        assert rel_err(k.view(6, 1, 32), plain.rope(k0.cpu().view(6, 1, 32), p, want_f)) < lim


def plain_attention_block(t, prefix, n, heads, kv_heads, hd, freqs, act, window=0, scale=None):
    tt = n.shape[0]
    q = act(plain.linear(n, t[prefix + ".q_proj.weight"])).view(tt, heads, hd)
    k = act(plain.linear(n, t[prefix + ".k_proj.weight"])).view(tt, kv_heads, hd)
    v = act(plain.linear(n, t[prefix + ".v_proj.weight"])).view(tt, kv_heads, hd)
    pos = list(range(tt))
    q, k = act(plain.rope(q, pos, freqs)), act(plain.rope(k, pos, freqs))
    o = act(plain.attention(q, k, v, window=window, scale=scale)).reshape(tt, heads * hd)
    return plain.linear(o, t[prefix + ".o_proj.weight"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,hd,window,scale", [(4, 2, 64, 0, None), (6, 3, 48, 0, 0.2), (3, 1, 32, 37, None)])
def test_attention_mixer_alone_prompt_then_steps(kn, dtype, heads, kv_heads, hd, window, scale):
    """The mixer with its own cache: a prompt of 90 rows in one step, then 45 rows one by one, against
    plain attention over the whole 135 (window and scale are parameters of the part)."""
    env = BuildEnv(dtype, DEV, kn)
    width = 72
    spec = PartSpec("gqa_attention", {"width": width, "heads": heads, "kv_heads": kv_heads, "head_dim": hd,
                                      "prefix": "att", "window": window, "scale": scale,
                                      "position": PartSpec("rope", {"head_dim": hd, "base": 10000.0})})
    mixer = build_part(MIXERS, spec)
    t = bound(mixer, env, dtype)
    act = plain.identity if dtype == torch.float32 else plain.round_bf16
    cache = CacheManager({0: mixer.cache_need()}, 512, 4, dtype, DEV)
    slot = cache.acquire()
    other = cache.acquire()  # a second live sequence, so that slot and batch index differ
    total = 135
    h = (torch.randn((total, width), device=DEV)).to(dtype)
    want = plain_attention_block(t, "att", h.cpu().double(), heads, kv_heads, hd, plain.rope_frequencies(hd, 10000.0),
                                 act, window=window, scale=scale)
    got = []
    done = 0
    for n_new in [90] + [1] * 45:
        cache.reserve({slot: n_new, other: 1})
        ctx = context(kn, dtype, [cache.length(other) + 1, done + n_new], [1, n_new], [other, slot])
        rows = torch.cat([h[:1], h[done : done + n_new]])
        out = mixer.forward(rows.contiguous(), ctx, cache.layer_views()[0])
        torch.cuda.synchronize()
        got.append(out[1:].clone())
        cache.advance({slot: n_new, other: 1})
        done += n_new
    got = torch.cat(got)
    assert got.dtype == torch.float32
    assert rel_err(got, want) < (2e-5 if dtype == torch.float32 else 1.5e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width,inner,rows", [(72, 200, 9), (64, 132, 70), (80, 52, 3)])
def test_swiglu_feed_forward_alone(kn, dtype, width, inner, rows):
    env = BuildEnv(dtype, DEV, kn)
    ffn = build_part(FEED_FORWARDS, PartSpec("swiglu", {"width": width, "inner": inner, "prefix": "mlp"}))
    t = bound(ffn, env, dtype)
    assert ffn.fused == (dtype == torch.bfloat16 and inner % 8 == 0)
    act = plain.identity if dtype == torch.float32 else plain.round_bf16
    h = torch.randn((rows, width), device=DEV).to(dtype)
    ctx = context(kn, dtype, [rows], [rows], [0])
    out = ffn.forward(h, ctx)
    hd = h.cpu().double()
    g, u = plain.linear(hd, t["mlp.gate_proj.weight"]), plain.linear(hd, t["mlp.up_proj.weight"])
    want = plain.linear(act(plain.swiglu(g, u)), t["mlp.down_proj.weight"])
    assert rel_err(out, want) < (2e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prenorm_block_alone(kn, dtype):
    """x += mixer(norm(x)); x += ffn(norm(x)), with the second add left pending for the next norm."""
    env = BuildEnv(dtype, DEV, kn)
    width, heads, kv_heads, hd, inner = 64, 4, 2, 16, 96
    spec = PartSpec("prenorm", {
        "mixer": PartSpec("gqa_attention", {"width": width, "heads": heads, "kv_heads": kv_heads, "head_dim": hd,
                                            "prefix": "b.att", "position": PartSpec("rope", {"head_dim": hd, "base": 100.0})}),
        "feed_forward": PartSpec("swiglu", {"width": width, "inner": inner, "prefix": "b.mlp"}),
        "mixer_norm": PartSpec("rmsnorm", {"width": width, "eps": 1e-5, "name": "b.n1"}),
        "ffn_norm": PartSpec("rmsnorm", {"width": width, "eps": 1e-5, "name": "b.n2"})})
    block = build_part(BLOCKS, spec)
    t = bound(block, env, dtype)
    act = plain.identity if dtype == torch.float32 else plain.round_bf16
    cache = CacheManager({0: block.mixer.cache_need()}, 256, 2, dtype, DEV)
    slot = cache.acquire()
    rows = 50
    x = torch.randn((rows, width), device=DEV)
    pending = torch.randn((rows, width), device=DEV) * 0.1
    xd = (x + pending).cpu().double()
    cache.reserve({slot: rows})
    ctx = context(kn, dtype, [rows], [rows], [slot])
    new_pending = block.forward(x, pending, ctx, cache.layer_views()[0])
    n = act(plain.rms_norm(xd, t["b.n1"], 1e-5))
    mid = xd + plain_attention_block(t, "b.att", n, heads, kv_heads, hd, plain.rope_frequencies(hd, 100.0), act)
    n2 = act(plain.rms_norm(mid, t["b.n2"], 1e-5))
    g, u = plain.linear(n2, t["b.mlp.gate_proj.weight"]), plain.linear(n2, t["b.mlp.up_proj.weight"])
    ffn = plain.linear(act(plain.swiglu(g, u)), t["b.mlp.down_proj.weight"])
    lim = 2e-5 if dtype == torch.float32 else 1.5e-2
    assert rel_err(x, mid) < lim  # the stream holds everything but the feed-forward's share
    assert rel_err(new_pending, ffn) < lim
