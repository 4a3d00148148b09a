"""bin/trace_run replays the same requests whole, with the last 32 tokens one by one, and in batches
of unequal lengths (slots reused), in float32 and in bfloat16; all against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain
from helpers import TINY_B, TINY_C, TOL_BF16, TOL_F32, random_tokens, read_folder, rel_err, write_folder

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = (40, 70, 33, 129, 3)


def replay(folder, dtype, steps, out_dir, max_tokens, extra=()):
    """Feeds the steps one at a time, each only after the previous `done` line, as a driver would."""
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                             "--out", out_dir, "--max-tokens", str(max_tokens), *extra],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    try:
        for st in steps:
            proc.stdin.write(json.dumps(st) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {st['step']}", (line, proc.stderr.read()[-3000:] if proc.poll() is not None else "")
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0, proc.stderr.read()[-3000:]
    finally:
        if proc.poll() is None:
            proc.kill()


def read_step(out_dir, step, vocab):
    return torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, vocab).copy())


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg, std in (("b", TINY_B, 0.02), ("c", TINY_C, 0.15)):
        folder = write_folder(tmp_path_factory.mktemp(name), cfg, seed=21, std=std)
        c, tensors = read_folder(folder)
        reqs = {f"r{i}": random_tokens(n, cfg["vocab_size"], 300 + i) for i, n in enumerate(LENGTHS)}
        out[name] = (folder, cfg, plain.PlainLlama(c, tensors), reqs)
    return out


@pytest.mark.parametrize("name", ["b", "c"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_whole_tail_and_batched(models, tmp_path, name, dtype):
    folder, cfg, ref, reqs = models[name]
    vocab = cfg["vocab_size"]
    act = plain.identity if dtype == "float32" else plain.round_bf16
    tol = TOL_F32 if dtype == "float32" else TOL_BF16
    want = {rid: ref.forward(toks, act) for rid, toks in reqs.items()}

    # --- each request alone and whole: one step each, ended at once; 192 tokens hold the longest
    steps = [{"step": i, "entries": [{"id": rid, "tokens": toks, "want": list(range(len(toks)))}], "end": [rid]}
             for i, (rid, toks) in enumerate(reqs.items())]
    out = str(tmp_path / "whole")
    replay(folder, dtype, steps, out, max_tokens=192)
    for i, rid in enumerate(reqs):
        assert rel_err(read_step(out, i, vocab), want[rid]) < tol

    # --- the last 32 tokens one by one
    steps, expect = [], []
    n = 0
    for rid, toks in reqs.items():
        if len(toks) <= 32:
            continue
        head = len(toks) - 32
        steps.append({"step": n, "entries": [{"id": rid, "tokens": toks[:head], "want": [head - 1]}], "end": []})
        expect.append((n, want[rid][head - 1 : head]))
        n += 1
        for j in range(head, len(toks)):
            steps.append({"step": n, "entries": [{"id": rid, "tokens": [toks[j]], "want": [0]}],
                          "end": [rid] if j == len(toks) - 1 else []})
            expect.append((n, want[rid][j : j + 1]))
            n += 1
    out = str(tmp_path / "tail")
    replay(folder, dtype, steps, out, max_tokens=192)
    for step, w in expect:
        assert rel_err(read_step(out, step, vocab), w) < tol, step

    # --- batches of unequal lengths, one after another; shorter requests end earlier; a step in
    # which nothing is wanted writes no file
    steps, expect = [], []
    n = 0
    for group in (["r0", "r1", "r2"], ["r3", "r4", "r0"]):
        heads = {rid: max(1, len(reqs[rid]) - 5 - 2 * k) for k, rid in enumerate(group)}
        entries = [{"id": rid, "tokens": reqs[rid][: heads[rid]], "want": [0, heads[rid] - 1]} for rid in group]
        done = [rid for rid in group if heads[rid] == len(reqs[rid])]
        steps.append({"step": n, "entries": entries, "end": done})
        expect.append((n, torch.cat([want[rid][[0, heads[rid] - 1]] for rid in group])))
        n += 1
        pos = dict(heads)
        quiet = True
        while any(pos[rid] < len(reqs[rid]) for rid in group):
            live = [rid for rid in group if pos[rid] < len(reqs[rid])]
            wants = [] if quiet else [0]
            entries = [{"id": rid, "tokens": [reqs[rid][pos[rid]]], "want": wants} for rid in live]
            if not quiet:
                expect.append((n, torch.stack([want[rid][pos[rid]] for rid in live])))
            quiet = False
            for rid in live:
                pos[rid] += 1
            steps.append({"step": n, "entries": entries, "end": [rid for rid in live if pos[rid] == len(reqs[rid])]})
            n += 1
    out = str(tmp_path / "batched")
    # live at once: at most 64 + 128 + 64 (first group) or 192 + 64 + 64 (second) tokens in units of 64
    replay(folder, dtype, steps, out, max_tokens=320)
    for step, w in expect:
        assert rel_err(read_step(out, step, vocab), w) < tol, step
    assert not os.path.exists(os.path.join(out, "1.f32"))  # nothing was wanted in step 1


def test_replay_dumps_the_residual_stream_after_every_layer(models, tmp_path):
    """--dump-activations: the stream after the embedding and after each layer, for a prompt step and for a
    decoding step (where the products add into the stream themselves), against the plain layers."""
    folder, cfg, ref, reqs = models["b"]
    toks = reqs["r0"]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:-1], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[-1:], "want": [0]}], "end": ["a"]}]
    dump = str(tmp_path / "acts")
    replay(folder, "float32", steps, str(tmp_path / "o"), 64, extra=["--dump-activations", dump])
    emb = ref.w("model.embed_tokens.weight")
    x = emb[torch.tensor(toks, dtype=torch.long)]
    width = cfg["hidden_size"]

    def dumped(step, name):
        return torch.from_numpy(np.fromfile(os.path.join(dump, f"{step}.{name}.f32"), dtype="<f4").reshape(-1, width).copy())

    assert rel_err(dumped(0, "embed"), x[:-1]) < 1e-6 and rel_err(dumped(1, "embed"), x[-1:]) < 1e-6
    for layer in range(cfg["num_hidden_layers"]):
        x = ref.decoder_layer(layer, x, plain.identity)
        assert rel_err(dumped(0, f"run{layer}"), x[:-1]) < TOL_F32, layer
        assert rel_err(dumped(1, f"run{layer}"), x[-1:]) < TOL_F32, layer


def test_replay_refuses_more_tokens_than_the_cache_was_sized_for(models, tmp_path):
    folder, cfg, ref, reqs = models["b"]
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(tmp_path / "o"), "--max-tokens", "64"],
                          input=json.dumps({"step": 0, "entries": [{"id": "x", "tokens": reqs["r1"], "want": []}], "end": []}) + "\n",
                          capture_output=True, text=True, timeout=300)
    # 70 tokens into a cache made for 64: refused before anything runs (as too long for one sequence
    # of this cache; a second request that no longer fits beside the first is refused as "cache is full")
    assert proc.returncode != 0 and "64 tokens a sequence may have" in proc.stderr
