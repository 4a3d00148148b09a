"""The engine on the GPU against the plain implementation, in float32 and in bfloat16: each
request alone and whole; with the last 32 tokens one by one; in batches of unequal lengths whose
shorter requests end earlier, one batch after another so that slots are used again; long decoding;
the first tokens of a sequence; greedy generation through the entry point; toy parts."""
import os
import subprocess
import sys

import pytest
import torch

import helpers
import longbow_quarrel_amd as lq
import plain
import toy_parts
from helpers import TINY_A, TINY_B, TINY_C, TOL_BF16, TOL_F32, TOL_F32_HARSH, random_tokens, read_folder, rel_err, write_folder
from longbow_quarrel_amd.engine import StepEntry
from longbow_quarrel_amd.loading import random_engine
from longbow_quarrel_amd.weights import random_tensors

pytestmark = pytest.mark.gpu

# (configuration, std of the random weights): the third has weights large enough that attention is
# peaked, so that a key read from the wrong place changes the logits by far more than any tolerance
CASES = {"a": (TINY_A, 0.02), "b": (TINY_B, 0.02), "c_sharp": (TINY_C, 0.15)}
LENGTHS = (70, 5, 33, 1, 65, 130)
_cache = {}


def setup_case(tmp_path_factory, name, dtype):
    key = (name, dtype)
    if key not in _cache:
        cfg, std = CASES[name]
        folder = write_folder(tmp_path_factory.mktemp(f"{name}_{dtype}"), cfg, seed=7, std=std)
        # requests longer than the tiny configurations' max_position_embeddings run here: say so
        eng = lq.load_engine(folder, dtype=dtype, max_tokens=2048, max_sequence_tokens=2048)
        c, tensors = read_folder(folder)
        ref = plain.PlainLlama(c, tensors)
        act = plain.identity if dtype == "float32" else plain.round_bf16
        reqs = [random_tokens(n, cfg["vocab_size"], 100 + n) for n in LENGTHS]
        want = [ref.forward(r, act) for r in reqs]
        _cache[key] = (eng, ref, act, reqs, want, folder)
    return _cache[key]


def tol(dtype):
    return TOL_F32 if dtype == "float32" else TOL_BF16


PARAMS = [(n, d) for n in CASES for d in ("float32", "bfloat16")]


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_each_request_alone_and_whole(tmp_path_factory, name, dtype):
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, name, dtype)
    for r, w in zip(reqs, want):
        s = eng.new_sequence()
        got = eng.step([StepEntry(s, r, range(len(r)))])
        eng.release(s)
        assert got.shape == w.shape and rel_err(got, w) < tol(dtype)


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_last_32_tokens_one_by_one(tmp_path_factory, name, dtype):
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, name, dtype)
    for r, w in zip(reqs, want):
        if len(r) <= 32:
            continue
        s = eng.new_sequence()
        head = len(r) - 32
        got = [eng.step([StepEntry(s, r[:head], range(head))])]
        got += [eng.step([StepEntry(s, [t], [0])]) for t in r[head:]]
        eng.release(s)
        got = torch.cat(got)
        assert rel_err(got, w) < tol(dtype)
        # the first decoded token and a prompt's end are where a cache fault would show first
        assert rel_err(got[head - 1], w[head - 1]) < tol(dtype) and rel_err(got[head], w[head]) < tol(dtype)


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_unequal_batches_one_after_another_reuse_slots(tmp_path_factory, name, dtype):
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, name, dtype)
    used = []
    for group in ([0, 1, 2], [3, 4, 5], [5, 0]):
        slots = {i: eng.new_sequence() for i in group}
        used.append(sorted(slots.values()))
        split = {i: max(1, len(reqs[i]) - 4 - 3 * j) for j, i in enumerate(group)}
        out = eng.step([StepEntry(slots[i], reqs[i][: split[i]], range(split[i])) for i in group])
        at = 0
        for i in group:
            assert rel_err(out[at : at + split[i]], want[i][: split[i]]) < tol(dtype)
            at += split[i]
        pos = dict(split)
        for i in group:
            if pos[i] == len(reqs[i]):
                eng.release(slots[i])
        while any(pos[i] < len(reqs[i]) for i in group):
            live = [i for i in group if pos[i] < len(reqs[i])]
            out = eng.step([StepEntry(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                assert rel_err(out[j], want[i][pos[i]]) < tol(dtype), (i, pos[i])
                pos[i] += 1
                if pos[i] == len(reqs[i]):
                    eng.release(slots[i])
    assert used[0] == used[1]  # the second batch ran on the slots the first gave back
    assert eng.cache.slots.taken_count == 0 and all(g.blocks.taken_count == 0 for g in eng.cache.kv_groups)


@pytest.mark.parametrize("name,dtype", [("a", "float32"), ("c_sharp", "float32"), ("c_sharp", "bfloat16"), ("b", "bfloat16")])
def test_long_decoding(tmp_path_factory, name, dtype):
    """10 prompt tokens, then 290 tokens one by one: across four cache blocks and three attention splits."""
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, name, dtype)
    cfg = CASES[name][0]
    toks = random_tokens(300, cfg["vocab_size"], 77)
    w = ref.forward(toks, act)
    s = eng.new_sequence()
    got = [eng.step([StepEntry(s, toks[:10], range(10))])]
    got += [eng.step([StepEntry(s, [t], [0])]) for t in toks[10:]]
    eng.release(s)
    got = torch.cat(got)
    for lo in range(0, 300, 50):  # localise a fault to the place where it starts
        assert rel_err(got[lo : lo + 50], w[lo : lo + 50]) < tol(dtype), lo


@pytest.mark.parametrize("name,dtype", PARAMS)
def test_first_tokens_of_a_sequence(tmp_path_factory, name, dtype):
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, name, dtype)
    toks = reqs[0][:3]
    w = ref.forward(toks, act)
    slots = [eng.new_sequence() for _ in range(3)]
    # three sequences of 1, 2 and 3 tokens in one step, then the shorter ones catch up one token at a time
    out = eng.step([StepEntry(slots[0], toks[:1], [0]), StepEntry(slots[1], toks[:2], [0, 1]),
                    StepEntry(slots[2], toks[:3], [0, 1, 2])])
    for row, p in enumerate([0, 0, 1, 0, 1, 2]):
        assert rel_err(out[row], w[p]) < tol(dtype)
    out = eng.step([StepEntry(slots[0], [toks[1]], [0]), StepEntry(slots[1], [toks[2]], [0])])
    assert rel_err(out[0], w[1]) < tol(dtype) and rel_err(out[1], w[2]) < tol(dtype)
    for s in slots:
        eng.release(s)


def test_float32_logits_do_not_depend_on_the_cutting_at_all(tmp_path_factory):
    """In the float32 path every sum has an order fixed by the position alone: bit-equal results."""
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, "c_sharp", "float32")
    r = reqs[5]
    s = eng.new_sequence()
    whole = eng.step([StepEntry(s, r, range(len(r)))])
    eng.release(s)
    s, other = eng.new_sequence(), eng.new_sequence()
    parts = [eng.step([StepEntry(other, reqs[0], []), StepEntry(s, r[:50], range(50))])]
    parts.append(eng.step([StepEntry(s, r[50:51], [0]), StepEntry(other, [1], [])])[:1])
    parts.append(eng.step([StepEntry(s, r[51:], range(len(r) - 51))]))
    eng.release(s)
    eng.release(other)
    assert torch.equal(torch.cat(parts), whole)


@pytest.mark.parametrize("name,dtype", [("a", "float32"), ("c_sharp", "float32")])
def test_greedy_generation_through_the_entry_point(tmp_path_factory, name, dtype):
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, name, dtype)
    prompts = [reqs[1], reqs[3], reqs[2], reqs[0][:9]]
    expect = []
    for p in prompts:
        seq, out = list(p), []
        for _ in range(10):
            t = plain.arg_max(ref.forward(seq)[-1])
            out.append(t)
            seq.append(t)
        expect.append(out)
    for graphs in (False, True):
        res = lq.generate(eng, prompts, 10, lq.SamplingParams(temperature=0.0), stop_ids=[], max_batch=3,
                          use_graphs=graphs)
        assert res.tokens == expect and res.batches == 2
    # a stop id ends its sequence early and is not returned; the others go on
    stop = expect[0][4]
    res = lq.generate(eng, prompts, 10, stop_ids=[stop], max_batch=4)
    for got, exp in zip(res.tokens, expect):
        cut = exp.index(stop) if stop in exp else len(exp)
        assert got == exp[:cut]
    assert eng.cache.slots.taken_count == 0


def test_generation_in_bfloat16_graphs_and_direct_steps_agree(tmp_path_factory):
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, "c_sharp", "bfloat16")
    prompts = [reqs[1], reqs[2], reqs[4]]
    for params in (lq.SamplingParams(), lq.SamplingParams(temperature=0.8, top_k=40, top_p=0.95,
                                                          repetition_penalty=1.1, seed=3)):
        a = lq.generate(eng, prompts, 70, params, stop_ids=[], use_graphs=False)
        b = lq.generate(eng, prompts, 70, params, stop_ids=[], use_graphs=True)
        assert a.tokens == b.tokens and all(len(t) == 70 for t in a.tokens)
    # a sequence's sampled tokens do not depend on what else is in its batch
    alone = lq.generate(eng, prompts[:1], 20, lq.SamplingParams(temperature=0.8, seed=3), stop_ids=[])
    batch = lq.generate(eng, prompts, 20, lq.SamplingParams(temperature=0.8, seed=3), stop_ids=[])
    assert alone.tokens[0] == batch.tokens[0]


def test_steps_queued_ahead_of_the_host_and_a_sequence_that_stops_in_between(tmp_path_factory):
    """Captured steps are queued one ahead of the host.  A sequence that ends on a stop id leaves a step
    behind that ran for one sequence too many; the others go on from that step's tokens.  Greedy and seeded
    sampling through graphs equal direct steps, with run-ahead and without it."""
    from longbow_quarrel_amd.engine.generate import EngineBackend, GenerationLoop

    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, "c_sharp", "bfloat16")
    prompts = [reqs[1], reqs[2], reqs[4], reqs[0]]
    for params in (lq.SamplingParams(), lq.SamplingParams(temperature=0.9, top_k=50, seed=11)):
        free = lq.generate(eng, prompts, 24, params, stop_ids=[], use_graphs=False)
        stop = free.tokens[2][7]
        direct = lq.generate(eng, prompts, 24, params, stop_ids=[stop], use_graphs=False)
        assert direct.finish[2] == "stop" and "length" in direct.finish
        for ahead in (True, False):
            be = EngineBackend(eng, params)
            be.run_ahead = ahead
            got = GenerationLoop(be, max_batch=3).run(prompts, 24, stop_ids=[stop])
            assert got.tokens == direct.tokens and got.finish == direct.finish, (params, ahead)
            assert (be.steps_ahead > 0) == ahead
            be.close()
    assert eng.cache.slots.taken_count == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_freed_block_goes_to_a_survivor_while_a_step_is_queued_and_a_batch_follows_one_that_stopped(
        tmp_path_factory, dtype):
    """With real captured graphs and a stream that runs behind the host: the orders of events that
    `helpers.stopping_scenarios` sets up, against direct steps."""
    folder = write_folder(tmp_path_factory.mktemp("stopping"), TINY_A, seed=7)
    eng = lq.load_engine(folder, dtype=dtype, max_tokens=256, max_sequence_tokens=4096)
    helpers.stopping_scenarios(eng)


def test_many_requests_of_random_lengths_through_captured_steps_equal_direct_steps(tmp_path_factory):
    """Dozens of requests of random lengths with stop ids that end sequences at random steps, batches one after
    another on reused slots, in a pool that just holds a batch: captured steps queued one ahead of the host (their
    block-table entries and step arrays go up without waiting for the device) give the tokens of direct steps."""
    import random

    rng = random.Random(11)
    folder = write_folder(tmp_path_factory.mktemp("many"), TINY_C, seed=3, std=0.05)
    vocab = TINY_C["vocab_size"]
    for trial in range(4):
        n_req, new = rng.randrange(8, 30), rng.randrange(5, 70)
        prompts = [random_tokens(rng.randrange(1, 180), vocab, 1000 * trial + i) for i in range(n_req)]
        need = 64 * ((max(len(p) for p in prompts) + new + 63) // 64)
        eng = lq.load_engine(folder, dtype="float32", max_tokens=need * rng.randrange(1, 4), max_sequence_tokens=4096)
        stops = [rng.randrange(vocab) for _ in range(rng.randrange(0, 10))]
        max_batch = rng.randrange(1, 12)
        direct = lq.generate(eng, prompts, new, stop_ids=stops, max_batch=max_batch, use_graphs=False)
        captured = lq.generate(eng, prompts, new, stop_ids=stops, max_batch=max_batch, use_graphs=True)
        assert captured.tokens == direct.tokens and captured.finish == direct.finish, trial
        assert eng.cache.free_blocks() == eng.cache.n_blocks and eng.cache.slots.taken_count == 0


@pytest.mark.parametrize("n_prompts,max_batch", [(6, 3), (2, 1)])
def test_batches_of_one_size_one_after_another_through_captured_graphs(tmp_path_factory, n_prompts, max_batch):
    """The second batch finds a captured graph of its own size, on the same slots, whose arrays still hold
    the first batch's last tokens and positions: they must be written anew.  Greedy tokens through graphs,
    through direct steps and from the plain implementation agree."""
    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, "c_sharp", "float32")
    prompts = [reqs[i % len(reqs)][: 4 + 3 * i] for i in range(n_prompts)]
    expect = []
    for p in prompts:
        seq, out = list(p), []
        for _ in range(5):
            out.append(plain.arg_max(ref.forward(seq)[-1]))
            seq.append(out[-1])
        expect.append(out)
    for graphs in (True, False):
        res = lq.generate(eng, prompts, 5, lq.SamplingParams(), stop_ids=[], max_batch=max_batch, use_graphs=graphs)
        assert res.tokens == expect and res.batches == -(-n_prompts // max_batch), graphs
    eng16 = setup_case(tmp_path_factory, "c_sharp", "bfloat16")[0]
    sampled = lq.SamplingParams(temperature=0.8, top_k=40, top_p=0.95, repetition_penalty=1.1, seed=5)
    a = lq.generate(eng16, prompts, 12, sampled, stop_ids=[], max_batch=max_batch, use_graphs=True)
    b = lq.generate(eng16, prompts, 12, sampled, stop_ids=[], max_batch=max_batch, use_graphs=False)
    assert a.tokens == b.tokens
    assert eng.cache.slots.taken_count == 0 and eng16.cache.slots.taken_count == 0


def test_non_finite_logits_stop_generation_with_an_error(tmp_path_factory):
    """Direct and captured steps alike: a row of logits with an infinity raises NonFiniteLogits naming
    the request, and the slots come back."""
    folder = write_folder(tmp_path_factory.mktemp("nonfinite"), TINY_C, seed=2)
    for dtype in ("float32", "bfloat16"):
        eng = lq.load_engine(folder, dtype=dtype, max_tokens=512)
        prompts = [[5, 6, 7], [8, 9]]
        for graphs in (False, True):
            assert lq.generate(eng, prompts, 4, stop_ids=[], use_graphs=graphs).finish == ["length", "length"]
        head = eng.model.head
        saved = head[17].clone()
        head[17] = float("inf") if dtype == "float32" else 3e38  # bfloat16: the products overflow to infinity
        for graphs in (False, True):
            with pytest.raises(lq.NonFiniteLogits, match="request 0"):
                lq.generate(eng, prompts, 4, stop_ids=[], use_graphs=graphs)
            assert eng.cache.slots.taken_count == 0
        # a NaN inside the model, through captured steps
        head[17] = saved
        eng.model.blocks[0].ffn.w_down[3, :] = float("nan")
        with pytest.raises(lq.NonFiniteLogits):
            lq.generate(eng, prompts, 4, stop_ids=[], use_graphs=True)
        assert eng.cache.slots.taken_count == 0


# wide enough for the kernels that fold a block's add and norm into the projections around them
# (a few rows, at least 2 048 output columns): no size a power of two except the head size
WIDE = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 2176, "intermediate_size": 2312,
    "num_hidden_layers": 3, "num_attention_heads": 17, "num_key_value_heads": 1, "head_dim": 128,
    "vocab_size": 2053, "max_position_embeddings": 512, "rms_norm_eps": 2e-6, "rope_theta": 40000.0,
    "rope_scaling": None, "tie_word_embeddings": False, "torch_dtype": "bfloat16",
    "bos_token_id": 1, "eos_token_id": 2,
}


def test_decoding_with_add_and_norm_folded_into_the_projections(tmp_path_factory):
    """A step of a few rows adds each projection's result into the stream in the projection itself
    and leaves the norm to the projection that follows (the final norm to the head, where every row's
    logits are wanted): against the plain implementation, as is the same engine with these kernels
    switched off."""
    folder = write_folder(tmp_path_factory.mktemp("wide"), WIDE, seed=3, std=0.03)
    eng = lq.load_engine(folder, dtype="bfloat16", max_tokens=1024)
    kn = eng.kernels
    c, tensors = read_folder(folder)
    ref = plain.PlainLlama(c, tensors)
    reqs = [random_tokens(n, WIDE["vocab_size"], 300 + n) for n in (9, 21, 14)]
    want = [ref.forward(r, plain.round_bf16) for r in reqs]
    calls = {"residual": 0, "normed": 0}
    res, nrm = kn.linear_residual, kn.linear_scaled

    def counted(name, fn):
        def f(*a, **k):
            calls[name] += 1
            return fn(*a, **k)
        return f

    def decode_all():
        """prompts of 5 tokens in one step, then one token each until the shortest ends, and on"""
        slots = [eng.new_sequence() for _ in reqs]
        out = [[] for _ in reqs]
        first = eng.step([StepEntry(s, r[:5], range(5)) for s, r in zip(slots, reqs)])
        for i in range(len(reqs)):
            out[i].append(first[5 * i : 5 * i + 5])
        pos = 5
        while any(pos < len(r) for r in reqs):
            live = [i for i, r in enumerate(reqs) if pos < len(r)]
            got = eng.step([StepEntry(slots[i], [reqs[i][pos]], [0]) for i in live])
            for j, i in enumerate(live):
                out[i].append(got[j : j + 1])
            pos += 1
        for s in slots:
            eng.release(s)
        return [torch.cat(o) for o in out]

    kn.linear_residual, kn.linear_scaled = counted("residual", res), counted("normed", nrm)
    try:
        fused = decode_all()
    finally:
        kn.linear_residual, kn.linear_scaled = res, nrm
    layers = WIDE["num_hidden_layers"]
    steps = max(len(r) for r in reqs) - 5
    # (the prompts' step has 15 rows: there the pipelined tiles take the products whose K is a multiple of 64, all
    # but the feed-forward's last, which still adds into the stream itself)
    assert calls["residual"] == 2 * layers * steps + layers and calls["normed"] == 2 * layers * steps
    for got, w in zip(fused, want):
        assert rel_err(got, w) < TOL_BF16
    parts = kn.linear_fused_parts
    kn.linear_fused_parts = lambda *a: 0
    try:
        separate = decode_all()
    finally:
        kn.linear_fused_parts = parts
    for got, w in zip(separate, want):
        assert rel_err(got, w) < TOL_BF16
    assert not any(torch.equal(a, b) for a, b in zip(fused, separate))  # they are two ways indeed
    # a prompt long enough for the tiled matrix-core kernels and their K-shared products
    long_prompt = random_tokens(300, WIDE["vocab_size"], 9)
    s = eng.new_sequence()
    got = eng.step([StepEntry(s, long_prompt, range(300))])
    eng.release(s)
    assert rel_err(got, ref.forward(long_prompt, plain.round_bf16)) < TOL_BF16
    # prompts of 33 to 256 rows: the pipelined tiles that cover all rows (64, 128 and 256 of them)
    for n in (50, 100, 200):
        s = eng.new_sequence()
        got = eng.step([StepEntry(s, long_prompt[:n], range(n))])
        eng.release(s)
        assert rel_err(got, ref.forward(long_prompt[:n], plain.round_bf16)) < TOL_BF16
    # and inside a captured step
    g1 = lq.generate(eng, [r[:6] for r in reqs], 10, params=lq.SamplingParams(temperature=0.0), stop_ids=[], use_graphs=True)
    g2 = lq.generate(eng, [r[:6] for r in reqs], 10, params=lq.SamplingParams(temperature=0.0), stop_ids=[], use_graphs=False)
    assert g1.tokens == g2.tokens


def test_packed_weights_and_a_packed_tied_table_give_the_bits_of_dense_ones(tmp_path_factory):
    """Wide weights are held packed (8 rows' slabs of 64 k side by side), the table of a tied head too, which the
    embedding then reads in that order: the same logits, bit for bit, as an engine whose kernel object packs nothing,
    for prompts of every kind of product (a few rows, 33 to 256, more) and for decoding steps."""
    from longbow_quarrel_amd.kernels.hip import HipKernels

    cfg = dict(WIDE, intermediate_size=2304, vocab_size=2056, tie_word_embeddings=True, num_hidden_layers=2)
    folder = write_folder(tmp_path_factory.mktemp("packed"), cfg, seed=5, std=0.03)
    engines = []
    for pack in (True, False):
        kn = HipKernels()
        kn.pack_weights = pack
        engines.append(lq.load_engine(folder, dtype="bfloat16", max_tokens=2048, kernels=kn))
    packed, dense = engines
    mixer, ff = packed.model.blocks[0].mixer, packed.model.blocks[0].ffn
    for w in (mixer.w_qkv, mixer.w_o, ff.w_gate_up, ff.w_down, packed.model.head, packed.model.embedding.table):
        assert getattr(w, "packed", False)
    assert packed.model.head is packed.model.embedding.table
    assert not any(getattr(w, "packed", False) for w in (dense.model.head, dense.model.blocks[0].mixer.w_qkv))
    c, tensors = read_folder(folder)
    ref = plain.PlainLlama(c, tensors)
    prompt = random_tokens(400, cfg["vocab_size"], 77)
    for n in (3, 16, 40, 130, 400):
        outs = []
        for eng in engines:
            s = eng.new_sequence()
            first = eng.step([StepEntry(s, prompt[:n], range(n))])
            nxt = [eng.step([StepEntry(s, [prompt[n + i]], [0])]) for i in range(3)] if n < 400 else []
            eng.release(s)
            outs.append(torch.cat([first] + nxt))
        assert torch.equal(outs[0], outs[1]), n
        if n == 130:
            assert rel_err(outs[0][:n], ref.forward(prompt[:n], plain.round_bf16)) < TOL_BF16


def test_loading_a_model_takes_the_room_of_its_weights_and_a_layer_more(tmp_path_factory):
    """Weights that a part keeps in another form (packed, q k and v as one matrix, gate and up interleaved) give
    their source back as soon as the part is bound: the most memory in use while a model loads stays near what
    the loaded model holds, not twice that (a 70B shape's 141 GB would not fit twice)."""
    cfg = dict(WIDE, intermediate_size=2304, num_hidden_layers=8, vocab_size=2056)
    folder = write_folder(tmp_path_factory.mktemp("room"), cfg, seed=7, std=0.03)
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    before = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    eng = lq.load_engine(folder, dtype="bfloat16", max_tokens=64)
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated() - before
    most = torch.cuda.max_memory_allocated() - before
    layer = held / cfg["num_hidden_layers"]
    assert getattr(eng.model.blocks[0].mixer.w_qkv, "packed", False)
    assert most < held + 2.5 * layer, (held, most)


def test_decoding_batches_that_shrink_from_40_rows_to_one(tmp_path_factory):
    """40 sequences that end one after the other: decoding steps of 40 down to 1 row take the pipelined
    64-row tiles (above 12 rows: K shared between blocks, the pieces added by the norms), then the
    matrix-vector kernels with the norms folded into the products, against the plain implementation.  From
    13 rows on q, k and v leave their product in pieces too, which the decoding attention adds up (a width
    that is a multiple of 256, so that K can be shared, and no more than 16 heads a kv head, which is what the
    matrix-core decoding attention takes)."""
    wide = dict(WIDE, hidden_size=2304, num_attention_heads=18, num_key_value_heads=2)
    folder = write_folder(tmp_path_factory.mktemp("wide64"), wide, seed=4, std=0.03)
    eng = lq.load_engine(folder, dtype="bfloat16", max_tokens=64 * 48)
    kn = eng.kernels
    in_pieces = set()
    attention = kn.attention

    def watched(q, *a, **k):
        if k.get("pieces", 1) > 1:
            in_pieces.add(q.shape[0])
        return attention(q, *a, **k)

    kn.attention = watched
    c, tensors = read_folder(folder)
    ref = plain.PlainLlama(c, tensors)
    reqs = [random_tokens(4 + (i * 7) % 23, WIDE["vocab_size"], 500 + i) for i in range(40)]
    want = [ref.forward(r, plain.round_bf16) for r in reqs]
    slots = [eng.new_sequence() for _ in reqs]
    out = [[] for _ in reqs]
    first = eng.step([StepEntry(s, r[:3], range(3)) for s, r in zip(slots, reqs)])
    for i in range(len(reqs)):
        out[i].append(first[3 * i : 3 * i + 3])
    pos = 3
    rows_seen = set()
    while any(pos < len(r) for r in reqs):
        live = [i for i, r in enumerate(reqs) if pos < len(r)]
        rows_seen.add(len(live))
        got = eng.step([StepEntry(slots[i], [reqs[i][pos]], [0]) for i in live])
        for j, i in enumerate(live):
            out[i].append(got[j : j + 1])
        pos += 1
    kn.attention = attention
    for i, w in enumerate(want):
        assert rel_err(torch.cat(out[i]), w) < TOL_BF16, i
    assert any(r > 32 for r in rows_seen) and any(12 < r <= 32 for r in rows_seen) and any(r <= 12 for r in rows_seen)
    assert any(r > 32 for r in in_pieces) and any(12 < r <= 32 for r in in_pieces) and not any(r <= 12 for r in in_pieces)


def test_device_time_by_operation_with_events_around_every_kernel_call(tmp_path_factory):
    """`TimedKernels` stands in for the kernel object of an engine: the same logits, and a report that names
    every operation a step launched with its calls and a positive time (the products by their sizes)."""
    from longbow_quarrel_amd.kernels.timed import TimedKernels

    eng, ref, act, reqs, want, _ = setup_case(tmp_path_factory, "b", "bfloat16")
    r = reqs[0]
    s = eng.new_sequence()
    plain_run = eng.step([StepEntry(s, r, range(len(r)))])
    eng.release(s)
    real = eng.kernels
    timed = TimedKernels(real)
    eng.kernels = timed
    try:
        s = eng.new_sequence()
        got = eng.step([StepEntry(s, r, range(len(r)))])
        eng.step([StepEntry(s, [3], [0])])
        eng.release(s)
        report = timed.report()
    finally:
        eng.kernels = real
    assert torch.equal(got, plain_run)
    layers = TINY_B["num_hidden_layers"]
    assert report["attention"][0] == 2 * layers and report["embed"][0] == 2
    products = [k for k in report if k.startswith("linear")]
    assert any(k.endswith(f"x {TINY_B['vocab_size']} x {TINY_B['hidden_size']}") for k in products)  # the head
    assert all(calls > 0 and ms > 0 for calls, ms in report.values())
    timed.reset()
    assert timed.report() == {}


def test_the_float32_path_at_the_width_of_a_real_model(tmp_path_factory):
    """One layer with the 8B shape's width, heads and head size (4 096 wide, 32 heads over 8 of 128; the inner width and
    the vocabulary no powers of two) in true float32: whole prompts of 1 to 150 tokens against the float64 plain
    implementation (the K of the products is 4 096 and 5 000 here, where the tiny configurations end at 520), and a
    request fed whole, with its last tokens one by one, and inside a batch of unequal lengths gives the same bits."""
    cfg = {
        "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "intermediate_size": 5000,
        "num_hidden_layers": 1, "num_attention_heads": 32, "num_key_value_heads": 8, "head_dim": 128,
        "vocab_size": 1031, "max_position_embeddings": 512, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
        "rope_scaling": None, "tie_word_embeddings": False, "torch_dtype": "float32", "bos_token_id": 1, "eos_token_id": 2,
    }
    folder = write_folder(tmp_path_factory.mktemp("wide32"), cfg, seed=12, std=0.02)
    c, tensors = read_folder(folder)
    ref = plain.PlainLlama(c, tensors)
    eng = lq.load_engine(folder, dtype="float32", max_tokens=1024)
    reqs = [random_tokens(n, cfg["vocab_size"], 900 + n) for n in (150, 1, 40, 17)]
    whole = []
    for r in reqs:
        s = eng.new_sequence()
        whole.append(eng.step([StepEntry(s, r, range(len(r)))]))
        eng.release(s)
        assert rel_err(whole[-1], ref.forward(r)) < TOL_F32, len(r)
    # the last 20 tokens of the first request one by one
    s = eng.new_sequence()
    got = [eng.step([StepEntry(s, reqs[0][:130], range(130))])]
    got += [eng.step([StepEntry(s, [t], [0])]) for t in reqs[0][130:]]
    eng.release(s)
    assert torch.equal(torch.cat(got), whole[0])
    # all four in one batch, cut at other places, the shorter ones ending earlier
    slots = [eng.new_sequence() for _ in reqs]
    cuts = [100, 1, 33, 16]
    out = eng.step([StepEntry(sl, r[:n], range(n)) for sl, r, n in zip(slots, reqs, cuts)])
    at = 0
    for i, n in enumerate(cuts):
        assert torch.equal(out[at : at + n], whole[i][:n]), i
        at += n
    pos = list(cuts)
    while any(p < len(r) for p, r in zip(pos, reqs)):
        live = [i for i, r in enumerate(reqs) if pos[i] < len(r)]
        out = eng.step([StepEntry(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
        for j, i in enumerate(live):
            assert torch.equal(out[j], whole[i][pos[i]]), (i, pos[i])
            pos[i] += 1
    for sl in slots:
        eng.release(sl)
    assert eng.cache.slots.taken_count == 0


LONG = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 256, "intermediate_size": 264,
    "num_hidden_layers": 2, "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 128,
    "vocab_size": 331, "max_position_embeddings": 4096, "rms_norm_eps": 1e-5, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 512},
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "bos_token_id": 1, "eos_token_id": 2,
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_sequence_longer_than_one_split_of_decode_attention(tmp_path_factory, dtype):
    """1 300 tokens with the 8B head shape: the prompt in unequal cuts (many cache blocks a row tile),
    then tokens one by one across the 1 024-key split boundary (two splits and their merge), with a
    short sequence decoding in the same batch."""
    folder = write_folder(tmp_path_factory.mktemp(f"long_{dtype}"), LONG, seed=9, std=0.08)
    c, tensors = read_folder(folder)
    ref = plain.PlainLlama(c, tensors)
    act = plain.identity if dtype == "float32" else plain.round_bf16
    n, head = 1300, 1010
    req = random_tokens(n, LONG["vocab_size"], 77)
    short = req[500:560]
    want, want_short = ref.forward(req, act), ref.forward(short, act)
    eng = lq.load_engine(folder, dtype=dtype, max_tokens=2048)
    a, b = eng.new_sequence(), eng.new_sequence()
    got = [eng.step([StepEntry(a, req[lo:hi], range(hi - lo))]) for lo, hi in ((0, 700), (700, 701), (701, head))]
    eng.step([StepEntry(b, short[:20], [])])
    got_short = []
    for i in range(head, n):
        entries = [StepEntry(a, [req[i]], [0])]
        j = 20 + i - head
        if j < len(short):
            entries.append(StepEntry(b, [short[j]], [0]))
        out = eng.step(entries)
        got.append(out[:1])
        if j < len(short):
            got_short.append(out[1:2])
    got, got_short = torch.cat(got), torch.cat(got_short)
    assert rel_err(got[:head], want[:head]) < tol(dtype)
    assert rel_err(got[head:], want[head:]) < tol(dtype)
    assert rel_err(got[1020:1030], want[1020:1030]) < tol(dtype)  # the rows around the split boundary
    assert rel_err(got_short, want_short[20:]) < tol(dtype)
    # a step of more than a thousand rows (in bfloat16 the rotation then takes eight positions a workgroup):
    # one sequence goes on from position 5, the other starts beside it
    eng.release(a)
    eng.release(b)
    a, b = eng.new_sequence(), eng.new_sequence()
    first = eng.step([StepEntry(a, req[:5], range(5))])
    rest = eng.step([StepEntry(a, req[5:], range(n - 5)), StepEntry(b, short, range(len(short)))])
    assert rel_err(torch.cat([first, rest[: n - 5]]), want) < tol(dtype)
    assert rel_err(rest[n - 5 :], want_short) < tol(dtype)


def test_generation_through_graphs_on_the_matrix_core_decode_path_across_a_length_bucket(tmp_path_factory):
    """The head shape of the 8B model (head size 128, 4 query heads a kv head), bfloat16, prompts of about
    1 000 tokens, 70 new tokens: the decoding steps run captured (rotation and cache write folded into the
    attention kernel, splits merged by tickets), the longest sequence crosses 1 024 tokens, so a second
    graph with a larger bound is captured on the way.  The tokens equal those of direct steps, and the
    logits around the crossing agree with the plain implementation."""
    from longbow_quarrel_amd.engine.generate import EngineBackend, GenerationLoop

    folder = write_folder(tmp_path_factory.mktemp("long_graph"), LONG, seed=9, std=0.08)
    c, tensors = read_folder(folder)
    ref = plain.PlainLlama(c, tensors)
    eng = lq.load_engine(folder, dtype="bfloat16", max_tokens=4096)
    assert eng.kernels.attention_folds_rope(eng.dtype, 8, 2, 128, 64)
    prompts = [random_tokens(n, LONG["vocab_size"], 600 + n) for n in (1000, 985, 300)]
    runs = {}
    for graphs in (False, True):
        be = EngineBackend(eng, lq.SamplingParams(), use_graphs=graphs)
        be.keep_logits = True
        seen = []

        def callback(request, token, be=be, seen=seen):
            if request == 0:
                seen.append(be.last_logits[0].clone())

        res = GenerationLoop(be, max_batch=3).run(prompts, 70, stop_ids=[], callback=callback)
        if graphs:
            # the second graph's attention needs more workspace than the first had: the first one went
            assert (3, 2048, False) in be.graphs.graphs and be.graphs.captures == 2
        be.close()
        runs[graphs] = (res.tokens, torch.stack(seen))
    assert runs[True][0] == runs[False][0] and all(len(t) == 70 for t in runs[True][0])
    assert torch.equal(runs[True][1], runs[False][1])  # the same kernels on the same inputs
    # request 0 holds 1 000 + k tokens when its token k + 1 is sampled: k = 20..30 straddles the crossing
    seq = prompts[0] + runs[True][0][0]
    want = ref.forward(seq[:1040], plain.round_bf16)
    for k in range(15, 35):
        assert rel_err(runs[True][1][k], want[1000 + k - 1]) < TOL_BF16, k
    assert eng.cache.slots.taken_count == 0


def test_generation_with_sequences_of_very_unequal_lengths(tmp_path_factory):
    """Prompts of 1 400, 300, 290 and 310 tokens in one batch on the 8B head shape: the decoding steps tell the
    attention kernel that the lengths are uneven, and it shares the long sequence's keys out over the
    workgroups that the short ones leave free.  The hint reaches the kernel in captured and in direct steps
    alike (the tokens and the logits of both are equal), the logits agree with the plain implementation, and
    once the long sequence has ended the rest goes on without the hint."""
    from longbow_quarrel_amd.engine.generate import EngineBackend, GenerationLoop

    folder = write_folder(tmp_path_factory.mktemp("uneven"), LONG, seed=10, std=0.08)
    c, tensors = read_folder(folder)
    ref = plain.PlainLlama(c, tensors)
    eng = lq.load_engine(folder, dtype="bfloat16", max_tokens=4096)
    kn = eng.kernels
    lengths_uneven = eng.lengths_uneven  # the engine asks the model, the model its mixers, they the kernel object
    assert lengths_uneven([1401, 61, 26, 301]) and not lengths_uneven([530] * 8) and not lengths_uneven([900])
    assert not lengths_uneven([1000, 985, 300]) and lengths_uneven([3000, 1000])
    assert eng.length_bound(1) == eng.length_bound(1024) == 1024 and eng.length_bound(1025) == 2048
    prompts = [random_tokens(n, LONG["vocab_size"], 800 + n) for n in (300, 290, 310, 1400)]
    hints = []
    attention = kn.attention

    def watched(*a, **k):
        if k.get("decode"):
            hints.append(bool(k.get("uneven")))
        return attention(*a, **k)

    runs = {}
    kn.attention = watched
    try:
        for graphs in (False, True):
            be = EngineBackend(eng, lq.SamplingParams(), use_graphs=graphs)
            be.keep_logits = True
            seen, seen_long = [], []

            def callback(request, token, be=be, seen=seen, seen_long=seen_long):
                if request == 0:
                    seen.append(be.last_logits[0].clone())
                if request == 3:  # (the last row for as long as it lives)
                    seen_long.append(be.last_logits[3].clone())

            del hints[:]
            # the long request may take 12 tokens, the others 30: the last 18 steps hold three short sequences
            loop = GenerationLoop(be, max_batch=4)
            limits = loop._token_limits
            loop._token_limits = lambda prompts, n: [12 if len(p) > 1000 else n for p in prompts]
            res = loop.run(prompts, 30, stop_ids=[], callback=callback)
            be.close()
            runs[graphs] = (res.tokens, torch.stack(seen), list(hints), torch.stack(seen_long))
    finally:
        kn.attention = attention
    assert runs[True][0] == runs[False][0] and [len(t) for t in runs[True][0]] == [30, 30, 30, 12]
    assert torch.equal(runs[True][1], runs[False][1])
    assert any(runs[False][2]) and not all(runs[False][2])  # with the long sequence, and without it
    assert any(runs[True][2]) and not all(runs[True][2])    # (captured steps: the calls of the captures)
    seq = prompts[0] + runs[True][0][0]
    want = ref.forward(seq, plain.round_bf16)
    for k in range(1, 30):  # request 0 holds 300 + k tokens when its token k + 1 is sampled
        assert rel_err(runs[True][1][k], want[300 + k - 1]) < TOL_BF16, k
    long_seq = prompts[3] + runs[True][0][3]
    want_long = ref.forward(long_seq, plain.round_bf16)
    assert torch.equal(runs[True][3], runs[False][3])
    for k in range(1, 12):  # the long request, whose keys the workgroups share out
        assert rel_err(runs[True][3][k], want_long[1400 + k - 1]) < TOL_BF16, k
    assert eng.cache.slots.taken_count == 0


LARGE = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 520, "intermediate_size": 500, "num_hidden_layers": 3,
    "num_attention_heads": 6, "num_key_value_heads": 1, "head_dim": 144, "vocab_size": 97,
    "max_position_embeddings": 4096, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "rope_scaling": None,
    "tie_word_embeddings": False, "torch_dtype": "bfloat16", "bos_token_id": 1, "eos_token_id": 2,
}


def test_large_weights_on_the_size_agnostic_attention_kernel(tmp_path_factory):
    """Head size 144 (no matrix-core attention kernel takes it), width 520, weights of standard deviation
    0.1 and norm gains of 1 +- 0.4: five times the weights of the other tests, so that attention is sharp
    and one activation that rounds the other way moves the logits by per cents.  The fixed bfloat16 bound
    of the other tests is below this model's own rounding noise, which is therefore measured here: the
    plain implementation with the same rounding places, its values before rounding moved by what the
    order of a float32 sum moves them (3e-6), differs from itself by 3 to 4e-2 a row.  The engine has to
    stay below that against the plain implementation, be as close to the unrounded model as the rounded
    plain one is, and in float32 meet the usual bound."""
    from longbow_quarrel_amd.weights.safetensors_io import write_safetensors

    folder = write_folder(tmp_path_factory.mktemp("large"), LARGE, seed=6, std=0.1)
    c, tensors = read_folder(folder)
    gen = torch.Generator().manual_seed(6)
    for name in list(tensors):
        if "norm" in name:
            tensors[name] = (1.0 + 0.4 * torch.randn(tensors[name].shape, generator=gen)).to(tensors[name].dtype)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    ref = plain.PlainLlama(c, {n: (t.float() if "norm" in n else t) for n, t in tensors.items()})
    toks = random_tokens(150, LARGE["vocab_size"], 75)
    head = len(toks) - 32

    def jitter(x):
        g = torch.Generator().manual_seed(1)
        return plain.round_bf16(x * (1.0 + 3e-6 * (torch.rand(x.shape, generator=g, dtype=torch.float64) - 0.5)))

    exact, rounded, moved = (ref.forward(toks, a) for a in (plain.identity, plain.round_bf16, jitter))

    def replay(dtype):
        eng = lq.load_engine(folder, dtype=dtype, max_tokens=512)
        s = eng.new_sequence()
        got = [eng.step([StepEntry(s, toks[:head], range(head))])]
        got += [eng.step([StepEntry(s, [t], [0])]) for t in toks[head:]]
        eng.release(s)
        return torch.cat(got)

    def worst_row(a, b):
        return max(rel_err(a[i], b[i]) for i in range(len(toks)))

    assert worst_row(replay("float32"), exact) < TOL_F32_HARSH
    got = replay("bfloat16")
    noise = worst_row(moved, rounded)
    assert 1e-2 < noise < 1e-1  # what this test is about: the model's own noise is above the fixed bound
    assert worst_row(got, rounded) < noise
    assert worst_row(got, exact) < 1.1 * worst_row(rounded, exact)
    assert rel_err(got, rounded) < TOL_BF16  # over all rows together the fixed bound still holds


def test_the_reference_style_interface(tmp_path_factory):
    """new_engine / infer / infer_with_callback / infer_with_logits / close (internal/engine/engine.go:380,
    1273-1296) give what `generate` gives for one sequence; the embedding look-ups give the table's rows."""
    eng, ref, act, reqs, want, folder = setup_case(tmp_path_factory, "b", "float32")
    prompt = reqs[2][:12]
    q = lq.new_engine(folder, dtype="float32", kv_cache_size=256)
    greedy = lq.generate(eng, [prompt], 9, lq.SamplingParams(), stop_ids=[5, 7]).tokens[0]
    assert q.infer(prompt, 9) == greedy == q.infer(prompt, 9, lq.SamplerConfig())
    seen = []
    assert q.infer_with_callback(prompt, 9, None, seen.append) == greedy and seen == greedy
    ids, logits = q.infer_with_logits(prompt, 9)
    assert ids == greedy and logits.shape == (TINY_B["vocab_size"],)
    whole = ref.forward(prompt + greedy[:-1], plain.identity)
    assert rel_err(logits, whole[-1]) < TOL_F32  # the logits the last id was taken from
    cfg = lq.SamplerConfig(temperature=0.8, top_k=40, top_p=0.95, rep_penalty=1.1, seed=4)
    assert q.infer(prompt, 9, cfg) == lq.generate(eng, [prompt], 9, cfg.params(), stop_ids=[5, 7]).tokens[0]
    # GetEmbedding(s) / EmbeddingDim (engine.go:1809-1858): rows of the table as they are stored
    _, tensors = read_folder(folder)
    table = tensors["model.embed_tokens.weight"].float()
    assert q.embedding_dim() == TINY_B["hidden_size"] == table.shape[1]
    assert torch.equal(q.get_embeddings([5, 0, 383]).cpu(), table[[5, 0, 383]])
    assert torch.equal(q.get_embedding(17).cpu(), table[17])
    with pytest.raises(ValueError, match="out of vocab range"):
        q.get_embedding(TINY_B["vocab_size"])
    q.close()


def test_command_line_generates_the_same_greedy_tokens(tmp_path_factory):
    eng, ref, act, reqs, want, folder = setup_case(tmp_path_factory, "a", "float32")
    prompt = reqs[1]
    expect = lq.generate(eng, [prompt], 6, stop_ids=[]).tokens[0]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    # eos is id 2 in this configuration; the command line stops there as generation does
    cut = expect.index(2) if 2 in expect else len(expect)
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "quarrel"), "-model", folder, "-prompt",
                          " ".join(map(str, prompt)), "-n", "6", "-temp", "0", "-penalty", "1", "-dtype", "float32"],
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.strip().splitlines()[-1].split() == [str(t) for t in expect[:cut]]
    assert f"{cut} tokens in" in out.stdout
    # prompts from a file (two requests, one batch), the other spelling of the token count, and a stop id of
    # the caller's: request 0 ends before the token it would have produced third
    other = reqs[0]
    both = lq.generate(eng, [prompt, other], 6, stop_ids=[]).tokens
    stop = both[0][2]
    expect2 = lq.generate(eng, [prompt, other], 6, extra_stop_ids=[stop]).tokens
    assert len(expect2[0]) <= 2
    path = os.path.join(folder, "prompts.txt")
    with open(path, "w") as f:
        f.write(" ".join(map(str, prompt)) + "\n\n" + ",".join(map(str, other)) + "\n")
    out = subprocess.run([sys.executable, os.path.join(root, "bin", "quarrel"), "-model", folder, "-prompt-file", path,
                          "-max-new-tokens", "6", "-stop-id", str(stop), "-temp", "0", "-penalty", "1",
                          "-dtype", "float32"], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    lines = out.stdout.strip().splitlines()[-2:]
    assert [line.split()[1:] for line in lines] == [[str(t) for t in ids] for ids in expect2]
    assert [line.split()[0] for line in lines] == ["[0]", "[1]"]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_parts_on_the_gpu(dtype):
    """A mixer with state of its own, a feed-forward with routing, another position encoding, a layer
    that runs twice and one that reads another's cache: registered, built and stepped here."""
    toy_parts.register_toys()
    try:
        cfg = toy_parts.ToyConfig.from_dict(toy_parts.TOY)
        eng = random_engine(cfg, seed=3, dtype=dtype, max_tokens=512, std=0.2)
        tensors = {k: v.cpu() for k, v in random_tensors(eng.model.tensor_specs(), 3, eng.dtype, 0.2, device=eng.device).items()}
        a, b = random_tokens(40, 53, 1), random_tokens(9, 53, 2)
        wa, wb = (toy_parts.plain_toy(toy_parts.TOY, tensors, t) for t in (a, b))
        # the toy's plain twin rounds nothing: with weights of standard deviation 0.2 the engine's bfloat16
        # activations differ from it by 0.7e-2 to 1.9e-2 over several seeds; the 32-bit run is what pins the parts
        limit = TOL_F32 if dtype == "float32" else 3e-2
        sa, sb = eng.new_sequence(), eng.new_sequence()
        out = eng.step([StepEntry(sa, a[:17], range(17)), StepEntry(sb, b[:8], range(8))])
        assert rel_err(out[:17], wa[:17]) < limit and rel_err(out[17:], wb[:8]) < limit
        out = eng.step([StepEntry(sa, a[17:18], [0]), StepEntry(sb, b[8:], [0])])
        assert rel_err(out[0], wa[17]) < limit and rel_err(out[1], wb[8]) < limit
        eng.release(sb)
        assert rel_err(eng.step([StepEntry(sa, a[18:], range(22))]), wa[18:]) < limit
        eng.release(sa)
        s = eng.new_sequence()
        assert rel_err(eng.step([StepEntry(s, b, range(9))]), wb) < limit
        res = lq.generate(eng, [a[:5], b[:3]], 4, stop_ids=[])  # generation falls back to direct steps
        assert [len(t) for t in res.tokens] == [4, 4]
    finally:
        toy_parts.unregister_toys()
