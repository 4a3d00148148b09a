"""bench.py's arithmetic and its refusal of more than one GPU (no GPU needed), and the driver's smoke entry."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402
import longbow_quarrel_amd as lq  # noqa: E402


def test_more_than_one_gpu_is_refused_with_one_line_and_exit_2():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 2
    lines = [ln for ln in out.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1 and "one GPU" in lines[0]


def test_bytes_and_flops_of_the_8b_shape_by_hand():
    c = lq.LlamaConfig.from_dict(dict(bench.CONFIG_8B))
    d, i, v, layers = 4096, 14336, 128256, 32
    # q, k, v, o, gate, up, down in bfloat16 and the two norms' gains in float32, a layer; the head; the final norm
    per_layer = 2 * (d * 6144 + d * d + 3 * d * i) + 2 * 4 * d
    assert bench.weight_bytes_per_step(c) == layers * per_layer + 2 * v * d + 4 * d
    assert 15.0e9 < bench.weight_bytes_per_step(c) < 15.1e9  # 7.5 G parameters without the embedding table
    # keys and values of one token: 8 kv heads of 128, two bytes each, in every layer
    assert bench.kv_bytes_per_token(c) == 2 * 8 * 128 * 2 * layers == 131072
    # 2 flops a multiply-add: the matrices once a token, the head once, causal attention over t (t + 1) / 2 pairs
    t = 2048
    linear = 2 * t * (per_layer - 8 * d) / 2
    attention = 2 * 2 * 32 * 128 * t * (t + 1) / 2
    assert bench.prefill_flops(c, t) == pytest.approx(layers * (linear + attention) + 2 * d * v, rel=1e-12)
    assert 2.9e13 < bench.prefill_flops(c, t) < 3.1e13
    # the 32-bit path: every matrix and the cache at four bytes an entry, the norms' gains as before
    assert bench.weight_bytes_per_step(c, 4) == layers * (2 * per_layer - 2 * 4 * d) + 4 * v * d + 4 * d
    assert bench.kv_bytes_per_token(c, 4) == 2 * 131072


def test_the_other_shapes_are_the_family_s_sizes():
    b1 = lq.LlamaConfig.from_dict(dict(bench.SHAPES["1b"]))
    assert (b1.hidden_size, b1.num_hidden_layers, b1.head_dim, b1.tie_word_embeddings) == (2048, 16, 64, True)
    b70 = lq.LlamaConfig.from_dict(dict(bench.SHAPES["70b"]))
    assert (b70.hidden_size, b70.num_hidden_layers, b70.num_attention_heads, b70.intermediate_size) == (8192, 80, 64, 28672)
    assert 138.9e9 < bench.weight_bytes_per_step(b70) < 139.1e9  # 141 GB with the embedding table, which a step does not read


@pytest.mark.gpu
def test_smoke_entry_runs(capsys):
    import __graft_entry__

    __graft_entry__.smoke()
    assert "smoke ok" in capsys.readouterr().out
