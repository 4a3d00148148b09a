"""Pins the plain implementation by what fixes it beside the reference's text: vectors the
reference's own tests hold, special cases that reduce to a library routine, and invariants, each
chosen so that a plausible mistake (a wrong sign or pairing, a norm in the wrong place) fails it."""
import math

import pytest
import torch

import plain

F64 = torch.float64


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=F64) * scale


# --------------------------------------------------------------------------- RMSNorm

def test_rms_norm_unit_weight_is_the_library_expression():
    x = rnd((3, 50), 1, 4.0)
    want = x / torch.sqrt(torch.mean(x * x, dim=-1, keepdim=True) + 1e-5)
    assert torch.allclose(plain.rms_norm(x, torch.ones(50), 1e-5), want, rtol=1e-12, atol=0)


def test_rms_norm_eps_is_inside_the_root_and_weight_comes_after():
    x = torch.full((1, 4), 2.0, dtype=F64)
    w = torch.tensor([1.0, 2.0, 3.0, 4.0], dtype=F64)
    # mean(x^2) = 4; with eps = 5 the divisor is sqrt(9) = 3, not sqrt(4) + 5 = 7
    got = plain.rms_norm(x, w, 5.0)
    assert torch.allclose(got, 2.0 / 3.0 * w, rtol=1e-12, atol=0)
    # no mean subtraction: a constant row is not mapped to zero
    assert float(got.abs().min()) > 0.5


def test_rms_norm_is_scale_invariant_and_has_unit_rms():
    x = rnd((2, 64), 2)
    a = plain.rms_norm(x, torch.ones(64), 1e-12)
    b = plain.rms_norm(x * 37.0, torch.ones(64), 1e-12)
    assert torch.allclose(a, b, rtol=1e-9, atol=0)
    assert torch.allclose((a * a).mean(dim=-1), torch.ones(2, dtype=F64), rtol=1e-9, atol=0)


def test_rms_norm_reference_vector():
    """2 x 4096 random in +-5, weights in [0, 2), eps 1e-5, recomputed in float64
    (internal/device/rmsnorm_test.go:16-77)."""
    g = torch.Generator().manual_seed(3)
    x = (torch.rand((2, 4096), generator=g, dtype=F64) - 0.5) * 10
    w = torch.rand((4096,), generator=g, dtype=F64) * 2
    want = torch.empty_like(x)
    for i in range(2):
        ss = sum(float(v) ** 2 for v in x[i])
        scale = 1.0 / math.sqrt(ss / 4096 + 1e-5)
        want[i] = x[i] * scale * w
    assert torch.allclose(plain.rms_norm(x, w, 1e-5), want, rtol=1e-10, atol=0)


# --------------------------------------------------------------------------- linear

def test_linear_is_x_times_w_transposed():
    x, w = rnd((5, 7), 4), rnd((3, 7), 5)
    assert torch.allclose(plain.linear(x, w), x @ w.t(), rtol=1e-12, atol=1e-14)
    assert plain.linear(x, w).shape == (5, 3)


# --------------------------------------------------------------------------- rotation

def test_rope_frequencies_ends():
    """f_0 = 1 and f_last = base^(-(hd-2)/hd) (internal/device/rope_attention_test.go:62-91)."""
    f = plain.rope_frequencies(128, 10000.0)
    assert f.shape == (64,)
    assert float(f[0]) == 1.0
    assert math.isclose(float(f[-1]), 10000.0 ** (-(126.0) / 128.0), rel_tol=1e-12)


def test_rope_position_zero_is_identity():
    x = rnd((1, 3, 16), 6)
    assert torch.equal(plain.rope(x, [0], plain.rope_frequencies(16, 1e4)), x)


def test_rope_head_dim_two_is_a_plane_rotation():
    x = torch.tensor([[[1.0, 0.0]]], dtype=F64)
    got = plain.rope(x, [3], plain.rope_frequencies(2, 1e4))
    # counter-clockwise by 3 rad: (cos 3, sin 3); a flipped sign would give (cos 3, -sin 3)
    assert torch.allclose(got[0, 0], torch.tensor([math.cos(3.0), math.sin(3.0)], dtype=F64), atol=1e-15)


def test_rope_pairs_are_half_split_not_adjacent():
    hd = 8
    f = plain.rope_frequencies(hd, 100.0)
    x = torch.zeros((1, 1, hd), dtype=F64)
    x[0, 0, 1] = 1.0  # lives in pair (1, 5) when pairs are (i, i + hd/2); in pair (0, 1) if adjacent
    got = plain.rope(x, [2], f)
    ang = 2 * float(f[1])
    want = torch.zeros(hd, dtype=F64)
    want[1], want[5] = math.cos(ang), math.sin(ang)
    assert torch.allclose(got[0, 0], want, atol=1e-15)


def test_rope_reference_vector():
    """hd 128, 32 heads, pos 5, theta 1e4, input i / 100 (internal/device/rope_test.go:10-65)."""
    hd, nh, pos = 128, 32, 5
    x = (torch.arange(nh * hd, dtype=F64) / 100.0).view(1, nh, hd)
    got = plain.rope(x, [pos], plain.rope_frequencies(hd, 10000.0))
    for h in (0, 7, 31):
        for i in (0, 1, 31, 63):
            th = pos * 10000.0 ** (-2.0 * i / hd)
            v0, v1 = float(x[0, h, i]), float(x[0, h, i + 64])
            assert math.isclose(float(got[0, h, i]), v0 * math.cos(th) - v1 * math.sin(th), rel_tol=1e-12, abs_tol=1e-12)
            assert math.isclose(float(got[0, h, i + 64]), v0 * math.sin(th) + v1 * math.cos(th), rel_tol=1e-12, abs_tol=1e-12)


def test_rope_preserves_pair_norms_and_depends_on_distance_only():
    hd = 32
    f = plain.rope_frequencies(hd, 5e5)
    q, k = rnd((1, 1, hd), 7), rnd((1, 1, hd), 8)
    rq = plain.rope(q, [11], f)
    assert torch.allclose(rq[..., :16] ** 2 + rq[..., 16:] ** 2, q[..., :16] ** 2 + q[..., 16:] ** 2, rtol=1e-12)
    dots = []
    for shift in (0, 5, 1000):
        a = plain.rope(q, [9 + shift], f)
        b = plain.rope(k, [4 + shift], f)
        dots.append(float((a * b).sum()))
    assert math.isclose(dots[0], dots[1], rel_tol=1e-9) and math.isclose(dots[0], dots[2], rel_tol=1e-9)
    # and it does depend on the distance
    c = float((plain.rope(q, [9], f) * plain.rope(k, [5], f)).sum())
    assert abs(c - dots[0]) > 1e-6


def test_rope_same_rotation_for_every_head():
    """q and k with different head counts get the same per-head rotation
    (internal/device/rope_gqa_test.go:10-79)."""
    hd = 16
    f = plain.rope_frequencies(hd, 1e4)
    one = rnd((1, 1, hd), 9)
    many = one.expand(1, 5, hd).clone()
    got = plain.rope(many, [7], f)
    for h in range(5):
        assert torch.equal(got[0, h], plain.rope(one, [7], f)[0, 0])


# --------------------------------------------------------------------------- llama3 frequency scaling

def test_llama3_scaling_invariants():
    base = plain.rope_frequencies(32, 500000.0)
    sc = plain.llama3_scaled_frequencies(base, 8.0, 1.0, 4.0, 64)
    lo_wl, hi_wl = 64 / 1.0, 64 / 4.0
    kinds = set()
    for f, g in zip(base.tolist(), sc.tolist()):
        wl = 2 * math.pi / f
        assert f / 8.0 - 1e-18 <= g <= f + 1e-18
        if wl < hi_wl:
            assert g == f
            kinds.add("kept")
        elif wl > lo_wl:
            assert math.isclose(g, f / 8.0, rel_tol=1e-15)
            kinds.add("divided")
        else:
            kinds.add("blend")
    assert kinds == {"kept", "divided", "blend"}  # this configuration exercises all three branches
    assert all(a >= b for a, b in zip(sc.tolist(), sc.tolist()[1:]))  # still non-increasing


def test_llama3_blend_at_hand_worked_points():
    """Inside the blend the weight is linear in original / wavelength (not in the wavelength): with low 1,
    high 4 and factor 8, original / wavelength = 2.5 gives s = (2.5 - 1) / (4 - 1) = 0.5 and
    f' = 0.5 f / 8 + 0.5 f = 0.5625 f; 1.75 gives s = 0.25 and f' = 0.75 f / 8 + 0.25 f = 0.34375 f.
    (A blend linear in the wavelength would give 0.825 f and 0.5 f.)  Both the plain function and the
    engine's table are held to these.  Parity unpinned: the reference has no frequency scaling at all
    (internal/device/kernels.metal:430-463 rotates with the base frequencies as they are), so these points hold
    the rule as config.json's `llama3` type is read here, not a vector of the reference's."""
    from longbow_quarrel_amd.parts.rope import rotary_frequencies

    hd, theta = 32, 500000.0
    base = plain.rope_frequencies(hd, theta)
    for ratio, want in ((2.5, 0.5625), (1.75, 0.34375), (1.0, 0.125), (4.0, 1.0)):
        for i in (3, 7, 12):
            f = float(base[i])
            original = ratio * 2 * math.pi / f  # so that original / wavelength_i is the ratio
            got = float(plain.llama3_scaled_frequencies(base, 8.0, 1.0, 4.0, original)[i])
            assert math.isclose(got / f, want, rel_tol=1e-12), (ratio, i)
            table = rotary_frequencies(hd, theta, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                                   "high_freq_factor": 4.0,
                                                   "original_max_position_embeddings": original})
            assert math.isclose(table[i] / f, want, rel_tol=1e-12), (ratio, i)
            assert math.isclose(table[0], 1.0) and len(table) == hd // 2


def test_llama3_scaling_reduces_to_identity():
    base = plain.rope_frequencies(64, 10000.0)
    assert torch.allclose(plain.llama3_scaled_frequencies(base, 1.0, 1.0, 4.0, 64), base, rtol=1e-15)
    assert torch.equal(plain.llama3_scaled_frequencies(base, 8.0, 1.0, 4.0, 10 ** 12), base)


def test_llama3_scaling_is_continuous_at_both_thresholds():
    orig, lo, hi, factor = 8192, 1.0, 4.0, 32.0
    for wl, want_ratio in ((orig / hi, 1.0), (orig / lo, 1.0 / factor)):
        for eps in (-1e-9, 1e-9):
            f = 2 * math.pi / (wl * (1 + eps))
            g = float(plain.llama3_scaled_frequencies(torch.tensor([f], dtype=F64), factor, lo, hi, orig)[0])
            assert math.isclose(g / f, want_ratio, rel_tol=1e-6)


# --------------------------------------------------------------------------- attention

def test_attention_without_groups_is_library_attention():
    t, nh, hd = 9, 3, 8
    q, k, v = rnd((t, nh, hd), 10), rnd((t, nh, hd), 11), rnd((t, nh, hd), 12)
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(plain.attention(q, k, v), want, rtol=1e-10, atol=1e-12)


def test_attention_group_mapping_is_integer_division():
    """Consecutive query heads share a kv head: h // (nh / nkv) (internal/device/kernels.metal:671)."""
    t, nh, nkv, hd = 6, 4, 2, 8
    q, k, v = rnd((t, nh, hd), 13), rnd((t, nkv, hd), 14), rnd((t, nkv, hd), 15)
    got = plain.attention(q, k, v)
    for h in range(nh):
        g = h // 2  # an interleaved mapping would be h % 2
        alone = plain.attention(q[:, h : h + 1], k[:, g : g + 1], v[:, g : g + 1])
        assert torch.allclose(got[:, h], alone[:, 0], rtol=1e-12, atol=1e-14)


def test_attention_single_key_and_equal_scores():
    q, k, v = rnd((1, 2, 4), 16), rnd((1, 1, 4), 17), rnd((1, 1, 4), 18)
    out = plain.attention(q, k, v)
    assert torch.allclose(out[0, 0], v[0, 0]) and torch.allclose(out[0, 1], v[0, 0])
    t = 5
    v = rnd((t, 1, 4), 19)
    out = plain.attention(torch.zeros((t, 1, 4), dtype=F64), rnd((t, 1, 4), 20), v)
    for p in range(t):
        assert torch.allclose(out[p, 0], v[: p + 1, 0].mean(dim=0), rtol=1e-12)


def test_attention_is_causal_and_windowed():
    t, hd = 10, 4
    q, k, v = rnd((t, 1, hd), 21), rnd((t, 1, hd), 22), rnd((t, 1, hd), 23)
    base = plain.attention(q, k, v)
    k2, v2 = k.clone(), v.clone()
    k2[6] += 5.0
    v2[6] -= 3.0
    changed = plain.attention(q, k2, v2)
    assert torch.equal(base[:6], changed[:6]) and not torch.allclose(base[6:], changed[6:])
    w = plain.attention(q, k, v, window=3)
    assert torch.allclose(w[:3], base[:3], rtol=1e-12)  # p < window: all keys
    alone = plain.attention(q[5:8], k[5:8], v[5:8])
    assert torch.allclose(w[7], alone[2], rtol=1e-12)  # p = 7 sees keys 5, 6, 7 only


def test_attention_reference_vectors():
    """Constant q = k = v = 0.1 over 256 keys returns 0.1 (internal/device/attention_test.go:10-55);
    4:2 heads, hd 32, pos 2 with q_h = h + 1, K = (p+1)(g+1), V = p + g + i + 2
    (internal/device/gqa_test.go:21-135)."""
    out = plain.attention(torch.full((256, 8, 128), 0.1, dtype=F64), torch.full((256, 8, 128), 0.1, dtype=F64),
                          torch.full((256, 8, 128), 0.1, dtype=F64))
    assert torch.allclose(out[255], torch.full((8, 128), 0.1, dtype=F64), rtol=1e-12)
    nh, nkv, hd, pos = 4, 2, 32, 2
    q = torch.zeros((pos + 1, nh, hd), dtype=F64)
    k = torch.zeros((pos + 1, nkv, hd), dtype=F64)
    v = torch.zeros((pos + 1, nkv, hd), dtype=F64)
    for h in range(nh):
        q[pos, h, :] = h + 1
    for p in range(pos + 1):
        for g in range(nkv):
            k[p, g, :] = (p + 1) * (g + 1)
            v[p, g, :] = torch.arange(hd, dtype=F64) + (p + 1) + (g + 1)
    out = plain.attention(q, k, v)[pos]
    for h in range(nh):
        g = h // (nh // nkv)
        scores = [hd * (h + 1) * (p + 1) * (g + 1) / math.sqrt(hd) for p in range(pos + 1)]
        mx = max(scores)
        e = [math.exp(s - mx) for s in scores]
        for i in (0, 5, 31):
            want = sum(ei / sum(e) * ((p + 1) + (g + 1) + i) for p, ei in enumerate(e))
            assert math.isclose(float(out[h, i]), want, rel_tol=1e-10)


# --------------------------------------------------------------------------- SwiGLU

def test_swiglu_is_library_silu_times_up():
    g, u = rnd((4, 9), 24, 3.0), rnd((4, 9), 25)
    assert torch.allclose(plain.swiglu(g, u), torch.nn.functional.silu(g) * u, rtol=1e-12, atol=1e-15)
    assert torch.equal(plain.swiglu(torch.zeros(3, dtype=F64), torch.ones(3, dtype=F64)), torch.zeros(3, dtype=F64))
    assert torch.allclose(plain.swiglu(torch.tensor([40.0], dtype=F64), torch.tensor([2.0], dtype=F64)),
                          torch.tensor([80.0], dtype=F64))
    # the gate is the activated operand: swapping the operands gives something else
    assert not torch.allclose(plain.swiglu(g, u), plain.swiglu(u, g))


# --------------------------------------------------------------------------- whole model

def tiny_model(layers=1, tie=False, seed=0):
    cfg = {"num_hidden_layers": layers, "hidden_size": 16, "num_attention_heads": 2, "num_key_value_heads": 1,
           "head_dim": 8, "intermediate_size": 24, "vocab_size": 11, "rms_norm_eps": 1e-5, "rope_theta": 100.0}
    t = {"model.embed_tokens.weight": rnd((11, 16), seed + 1, 0.5), "model.norm.weight": rnd((16,), seed + 2).abs()}
    if not tie:
        t["lm_head.weight"] = rnd((11, 16), seed + 3, 0.5)
    for l in range(layers):
        p = f"model.layers.{l}."
        t[p + "input_layernorm.weight"] = rnd((16,), seed + 10 * l + 4).abs()
        t[p + "post_attention_layernorm.weight"] = rnd((16,), seed + 10 * l + 5).abs()
        t[p + "self_attn.q_proj.weight"] = rnd((16, 16), seed + 10 * l + 6, 0.3)
        t[p + "self_attn.k_proj.weight"] = rnd((8, 16), seed + 10 * l + 7, 0.3)
        t[p + "self_attn.v_proj.weight"] = rnd((8, 16), seed + 10 * l + 8, 0.3)
        t[p + "self_attn.o_proj.weight"] = rnd((16, 16), seed + 10 * l + 9, 0.3)
        t[p + "mlp.gate_proj.weight"] = rnd((24, 16), seed + 10 * l + 10, 0.3)
        t[p + "mlp.up_proj.weight"] = rnd((24, 16), seed + 10 * l + 11, 0.3)
        t[p + "mlp.down_proj.weight"] = rnd((16, 24), seed + 10 * l + 12, 0.3)
    return cfg, t


def test_model_without_layers_is_norm_of_embedding_times_head():
    cfg, t = tiny_model(layers=0)
    toks = [3, 0, 10]
    want = plain.linear(plain.rms_norm(t["model.embed_tokens.weight"][toks], t["model.norm.weight"], 1e-5),
                        t["lm_head.weight"])
    assert torch.allclose(plain.PlainLlama(cfg, t).forward(toks), want, rtol=1e-12)


def test_tied_head_is_the_embedding():
    cfg, t = tiny_model(layers=1, tie=True)
    got = plain.PlainLlama(cfg, t).forward([1, 2, 3])
    t2 = dict(t)
    t2["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    assert torch.equal(got, plain.PlainLlama(cfg, t2).forward([1, 2, 3]))


def test_layer_with_zero_output_projections_is_the_identity():
    cfg, t = tiny_model(layers=2)
    for l in range(2):
        t[f"model.layers.{l}.self_attn.o_proj.weight"].zero_()
        t[f"model.layers.{l}.mlp.down_proj.weight"].zero_()
    cfg0, t0 = dict(cfg, num_hidden_layers=0), t
    assert torch.allclose(plain.PlainLlama(cfg, t).forward([4, 5, 6, 7]), plain.PlainLlama(cfg0, t0).forward([4, 5, 6, 7]),
                          rtol=1e-12)


def test_model_is_causal_and_uses_the_residual_stream():
    cfg, t = tiny_model(layers=2)
    m = plain.PlainLlama(cfg, t)
    a = m.forward([1, 2, 3, 4, 5])
    b = m.forward([1, 2, 3, 9, 5])
    assert torch.equal(a[:3], b[:3]) and not torch.allclose(a[3:], b[3:])
    # the residual carries the embedding through: dropping it (x = f(x) instead of x + f(x)) changes the result
    x = t["model.embed_tokens.weight"][[1, 2]]
    step = m.decoder_layer(0, x, plain.identity)
    n = plain.rms_norm(x, t["model.layers.0.input_layernorm.weight"], 1e-5)
    after_attn = x + m.attention_block(0, n, plain.identity)
    n2 = plain.rms_norm(after_attn, t["model.layers.0.post_attention_layernorm.weight"], 1e-5)  # norm of the *updated* stream
    assert torch.allclose(step, after_attn + m.feed_forward(0, n2, plain.identity), rtol=1e-12)


# --------------------------------------------------------------------------- sampler

def test_sampler_reference_vectors():
    """internal/engine/sampler_test.go:9-106."""
    assert plain.arg_max(torch.tensor([1.0, 5.0, 2.0, 0.5])) == 1
    assert plain.arg_max(torch.tensor([2.0, 7.0, 7.0])) == 1  # first maximal index
    d = plain.candidate_distribution(torch.tensor([2.0, 10.0, 5.0, 1.0]), 1.0, 1, 1.0)
    assert list(d) == [1] and d[1] == 1.0
    d = plain.candidate_distribution(torch.tensor([2.0, 10.0, 5.0, 1.0]), 1.0, 2, 1.0)
    assert set(d) == {1, 2}
    d = plain.candidate_distribution(torch.tensor([-0.91, -1.20, -1.61, -2.30]), 1.0, 0, 0.5)
    assert set(d) == {0, 1} and math.isclose(sum(d.values()), 1.0)
    pen = plain.apply_repetition_penalty(torch.tensor([0.8, 1.0, 0.8]), [1], 2.0)
    assert plain.arg_max(pen) != 1 and float(pen[1]) == 0.5
    pen = plain.apply_repetition_penalty(torch.tensor([-1.0, 1.0]), [0, 0, 1], 2.0)
    assert pen.tolist() == [-2.0, 0.5]  # negative logits are multiplied, each distinct id once


def test_sampler_penalty_window_is_the_last_64():
    logits = torch.ones(100)
    hist = list(range(100))
    pen = plain.apply_repetition_penalty(logits, hist, 2.0)
    assert pen[:36].tolist() == [1.0] * 36 and pen[36:].tolist() == [0.5] * 64


def test_sampler_distribution_and_draw():
    logits = torch.tensor([0.0, math.log(2.0), math.log(4.0), -50.0])
    d = plain.candidate_distribution(logits, 1.0, 0, 1.0)
    assert set(d) == {0, 1, 2}  # p <= 1e-10 is dropped
    assert math.isclose(d[2], 4 / 7, rel_tol=1e-6) and math.isclose(d[0], 1 / 7, rel_tol=1e-6)
    assert plain.draw(d, 0.0) == 2 and plain.draw(d, 0.57) == 2 and plain.draw(d, 0.58) == 1 and plain.draw(d, 0.99) == 0
    hot = plain.candidate_distribution(logits, 0.01, 0, 1.0)
    assert max(hot, key=hot.get) == 2 and hot[2] > 0.999999
