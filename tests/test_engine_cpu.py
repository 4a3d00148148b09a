"""The engine's own code (step function, cache, block tables, schedule) driven on the CPU through
a stand-in for the kernel library, against the plain implementation.  The GPU tests repeat the
comparisons with the real kernels; these catch faults of the batching and the cache without one."""
import pytest
import torch

import longbow_quarrel_amd as lq
import plain
import toy_parts
from cpu_kernels import CpuKernels
from helpers import TINY_A, TINY_B, TINY_C, random_tokens, read_folder, rel_err, stopping_scenarios, write_folder
from longbow_quarrel_amd.cache import CacheFull
from longbow_quarrel_amd.engine import StepEntry
from longbow_quarrel_amd.loading import random_engine
from longbow_quarrel_amd.weights import random_tensors

TOL = 1e-5


def make(tmp_path, cfg, seed=7, max_tokens=1024, max_sequence_tokens=4096):
    folder = write_folder(tmp_path, cfg, seed, dtype=torch.float32)
    # the requests here are longer than the tiny configurations' max_position_embeddings: say so
    eng = lq.load_engine(folder, dtype="float32", max_tokens=max_tokens, device="cpu", kernels=CpuKernels(),
                         max_sequence_tokens=max_sequence_tokens)
    c, tensors = read_folder(folder)
    return eng, plain.PlainLlama(c, tensors)


@pytest.mark.parametrize("cfg", [TINY_A, TINY_B, TINY_C])
def test_whole_cut_and_batched_agree_with_the_plain_implementation(tmp_path, cfg):
    eng, ref = make(tmp_path, cfg)
    reqs = [random_tokens(n, cfg["vocab_size"], n) for n in (70, 5, 33, 1, 65)]
    want = [ref.forward(r) for r in reqs]
    for r, w in zip(reqs, want):  # each request alone and whole
        s = eng.new_sequence()
        assert rel_err(eng.step([StepEntry(s, r, range(len(r)))]), w) < TOL
        eng.release(s)
    s = eng.new_sequence()  # prompt, then the last 32 one by one
    r, w = reqs[0], want[0]
    got = [eng.step([StepEntry(s, r[:-32], range(len(r) - 32))])]
    got += [eng.step([StepEntry(s, [t], [0])]) for t in r[-32:]]
    assert rel_err(torch.cat(got), w) < TOL
    eng.release(s)
    # two batches of unequal lengths on the same slots; shorter requests end earlier
    for group in ([0, 1, 2], [3, 4]):
        slots = {i: eng.new_sequence() for i in group}
        split = {i: max(1, len(reqs[i]) - 3 - i) for i in group}
        out = eng.step([StepEntry(slots[i], reqs[i][: split[i]], range(split[i])) for i in group])
        at = 0
        for i in group:
            assert rel_err(out[at : at + split[i]], want[i][: split[i]]) < TOL
            at += split[i]
        pos = dict(split)
        for i in group:
            if pos[i] == len(reqs[i]):
                eng.release(slots[i])
        while any(pos[i] < len(reqs[i]) for i in group):
            live = [i for i in group if pos[i] < len(reqs[i])]
            out = eng.step([StepEntry(slots[i], [reqs[i][pos[i]]], [0]) for i in live])
            for j, i in enumerate(live):
                assert rel_err(out[j], want[i][pos[i]]) < TOL
                pos[i] += 1
                if pos[i] == len(reqs[i]):
                    eng.release(slots[i])
    assert eng.cache.slots.taken_count == 0 and all(g.blocks.taken_count == 0 for g in eng.cache.kv_groups)


def test_chunked_prompts_and_mixed_steps(tmp_path):
    eng, ref = make(tmp_path, TINY_A)
    a, b = random_tokens(150, 256, 1), random_tokens(90, 256, 2)
    wa, wb = ref.forward(a), ref.forward(b)
    sa, sb = eng.new_sequence(), eng.new_sequence()
    o1 = eng.step([StepEntry(sa, a[:64], [63])])
    o2 = eng.step([StepEntry(sa, a[64:100], [0, 35]), StepEntry(sb, b[:90], [89])])  # a continues, b starts
    o3 = eng.step([StepEntry(sa, a[100:], [49])])
    assert rel_err(o1[0], wa[63]) < TOL and rel_err(o2[:2], wa[[64, 99]]) < TOL
    assert rel_err(o2[2], wb[89]) < TOL and rel_err(o3[0], wa[149]) < TOL


def test_a_step_knows_when_every_row_is_wanted_in_order(tmp_path):
    """`want_all` in the step's context (what lets the head take the stream's rows as they stand): set where
    the wanted places are all the step's rows in their order, and only there."""
    eng, ref = make(tmp_path, TINY_A)
    seen = []
    make_context = eng.make_context

    def recording(*a, **k):
        ctx = make_context(*a, **k)
        seen.append(ctx.want_all)
        return ctx

    eng.make_context = recording
    a, b = random_tokens(9, 256, 1), random_tokens(5, 256, 2)
    wa, wb = ref.forward(a), ref.forward(b)
    sa, sb = eng.new_sequence(), eng.new_sequence()
    o = eng.step([StepEntry(sa, a[:4], range(4)), StepEntry(sb, b[:2], range(2))])  # all six rows
    assert rel_err(o[:4], wa[:4]) < TOL and rel_err(o[4:], wb[:2]) < TOL
    eng.step([StepEntry(sa, a[4:6], [1]), StepEntry(sb, b[2:4], [0, 1])])            # one row missing
    eng.step([StepEntry(sa, a[6:8], [1, 0])])                                        # out of order
    o = eng.step([StepEntry(sa, a[8:], [0]), StepEntry(sb, b[4:], [0])])             # a decoding step
    assert rel_err(o[0], wa[8]) < TOL and rel_err(o[1], wb[4]) < TOL
    assert seen == [True, False, False, True]


def test_every_product_weight_is_offered_to_the_kernels_once_when_weights_are_bound(tmp_path):
    """A kernel object with `pack_weight` is asked once for each matrix of a product (q, k and v as one, o, gate and
    up as one, down, the head), and what it hands back is what the parts keep; a tied table is offered once and then
    serves the embedding and the head.  One without the method gets dense tensors, as the stand-in of these tests."""
    class Marked(torch.Tensor):
        pass

    class Packing(CpuKernels):
        def __init__(self):
            super().__init__()
            self.offered = []

        def pack_weight(self, w):
            self.offered.append(tuple(w.shape))
            return w.as_subclass(Marked)

    for cfg in (TINY_A, TINY_B):
        folder = write_folder(tmp_path / ("tied" if cfg["tie_word_embeddings"] else "untied"), cfg, seed=2)
        kn = Packing()
        eng = lq.load_engine(folder, dtype="float32", max_tokens=256, device="cpu", kernels=kn)
        m = eng.model
        layers, width, inner = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"]
        hd = cfg.get("head_dim") or width // cfg["num_attention_heads"]
        qkv = (cfg["num_attention_heads"] + 2 * cfg["num_key_value_heads"]) * hd
        want = [(qkv, width), (width, cfg["num_attention_heads"] * hd), (2 * inner, width), (width, inner)] * layers
        want.append((cfg["vocab_size"], width))
        assert sorted(kn.offered) == sorted(want)
        for b in m.blocks:
            assert all(isinstance(w, Marked) for w in (b.mixer.w_qkv, b.mixer.w_o, b.ffn.w_gate_up, b.ffn.w_down))
        # a dict that the caller gives up is emptied part by part; one that it keeps is left alone
        from longbow_quarrel_amd.model import DecoderModel
        from longbow_quarrel_amd.registry import spec_from_config
        for consume in (True, False):
            again = DecoderModel(spec_from_config(eng.config))
            given = dict(read_folder(folder)[1])
            count = len(given)
            again.bind(given, eng.env, consume=consume)
            assert len(given) == (0 if consume else count)
        assert isinstance(m.head, Marked)
        if cfg["tie_word_embeddings"]:
            assert m.head is m.embedding.table
        else:
            assert not isinstance(m.embedding.table, Marked)
        # and the engine still gives the plain implementation's logits
        c, tensors = read_folder(folder)
        toks = random_tokens(9, cfg["vocab_size"], 4)
        s = eng.new_sequence()
        got = eng.step([StepEntry(s, toks, range(9))])
        eng.release(s)
        assert rel_err(got, plain.PlainLlama(c, tensors).forward(toks, plain.identity)) < 1e-5


def test_a_released_slot_leaves_no_trace(tmp_path):
    eng, ref = make(tmp_path, TINY_C, max_tokens=256)
    first = random_tokens(130, 331, 3)
    s = eng.new_sequence()
    eng.step([StepEntry(s, first, [])])
    eng.release(s)
    second = random_tokens(77, 331, 4)
    t = eng.new_sequence()
    assert t == s
    got = eng.step([StepEntry(t, second, range(77))])
    assert rel_err(got, ref.forward(second)) < TOL


def test_step_refuses_bad_input_and_a_full_cache_changes_nothing(tmp_path):
    eng, ref = make(tmp_path, TINY_A, max_tokens=128)
    s = eng.new_sequence()
    for bad in ([StepEntry(s, [256], [0])], [StepEntry(s, [-1], [])], [StepEntry(s, [], [])],
                [StepEntry(s, [1, 2], [2])], [StepEntry(s, [1], [0]), StepEntry(s, [2], [0])],
                [StepEntry(s + 1, [1], [0])], []):
        with pytest.raises(ValueError):
            eng.step(bad)
    toks = random_tokens(100, 256, 5)
    eng.step([StepEntry(s, toks[:60], [])])
    with pytest.raises(CacheFull):
        eng.step([StepEntry(s, toks[:90], [])])
    assert eng.length(s) == 60
    got = eng.step([StepEntry(s, toks[60:], [39])])
    assert rel_err(got[0], ref.forward(toks)[99]) < TOL
    eng.release(s)
    assert eng.step([StepEntry(eng.new_sequence(), [3], [])]) is None  # nothing wanted, nothing returned


def test_a_sequence_is_bounded_by_the_configuration_or_by_the_caller(tmp_path):
    """Past `max_sequence_tokens` a step is refused before anything changes, naming the slot; the default
    bound is the configuration's max_position_embeddings (internal/engine/kv_cache.go:121-124 refuses a
    position past the cache's length the same way)."""
    from longbow_quarrel_amd.engine import SequenceTooLong

    eng, ref = make(tmp_path, TINY_A, max_sequence_tokens=None)
    assert eng.max_sequence_tokens == TINY_A["max_position_embeddings"] == 128
    toks = random_tokens(140, 256, 8)
    a, b = eng.new_sequence(), eng.new_sequence()
    with pytest.raises(SequenceTooLong, match=f"slot {a}"):
        eng.step([StepEntry(a, toks[:129], [])])
    eng.step([StepEntry(a, toks[:127], []), StepEntry(b, toks[:5], [])])
    got = eng.step([StepEntry(a, toks[127:128], [0])])  # the 128th token still fits
    assert rel_err(got[0], ref.forward(toks[:128])[127]) < TOL
    with pytest.raises(SequenceTooLong, match=f"slot {a}: 128 tokens held"):
        eng.step([StepEntry(b, [1], []), StepEntry(a, [1], [0])])
    assert eng.length(a) == 128 and eng.length(b) == 5  # the refused step changed nothing
    eng2, _ = make(tmp_path, TINY_A, max_sequence_tokens=10)
    s = eng2.new_sequence()
    with pytest.raises(SequenceTooLong):
        eng2.step([StepEntry(s, toks[:11], [])])
    with pytest.raises(ValueError):
        make(tmp_path, TINY_A, max_sequence_tokens=0)


def test_toy_parts_register_build_and_step_without_touching_the_framework(tmp_path):
    toy_parts.register_toys()
    try:
        cfg = toy_parts.ToyConfig.from_dict(toy_parts.TOY)
        eng = random_engine(cfg, seed=3, dtype="float32", max_tokens=512, device="cpu", kernels=CpuKernels(), std=0.2)
        assert not eng.graph_safe  # parts written with another library's operators are never captured
        assert len(eng.cache.state_groups) == 1 and len(eng.cache.kv_groups) == 1 and len(eng.cache.groups) == 3
        assert sorted(eng.cache.kv_groups[0].layers) == [1, 3]  # runs 1 and 3 own keys; run 2 reads run 1's
        latent = [g for g in eng.cache.groups if isinstance(g, toy_parts.LatentGroup)]
        assert len(latent) == 1 and latent[0].layers == [4]  # a kind of cache the framework does not know
        tensors = random_tensors(eng.model.tensor_specs(), 3, torch.float32, 0.2)
        a, b = random_tokens(40, 53, 1), random_tokens(9, 53, 2)
        wa, wb = (toy_parts.plain_toy(toy_parts.TOY, tensors, t) for t in (a, b))
        sa, sb = eng.new_sequence(), eng.new_sequence()
        out = eng.step([StepEntry(sa, a[:17], range(17)), StepEntry(sb, b[:8], range(8))])
        assert rel_err(out[:17], wa[:17]) < TOL and rel_err(out[17:], wb[:8]) < TOL
        # what a captured step is keyed by is the mixers' answer: the toy's own rule (steps of 500 tokens, uneven
        # beyond three to one) beside attention's default
        assert eng.length_bound(5) == 500 and eng.length_bound(501) == 1000
        assert eng.lengths_uneven([40, 10]) and not eng.lengths_uneven([30, 10])
        del toy_parts.DecayMixer.seen[:]
        out = eng.step([StepEntry(sa, a[17:18], [0]), StepEntry(sb, b[8:], [0])])
        assert rel_err(out[0], wa[17]) < TOL and rel_err(out[1], wb[8]) < TOL
        assert toy_parts.DecayMixer.seen == [(18, False)]  # a direct step: the longest length itself, 18 to 9
        eng.release(sb)
        out = eng.step([StepEntry(sa, a[18:], range(22))])
        assert rel_err(out, wa[18:]) < TOL
        eng.release(sa)
        assert latent[0].blocks.taken_count == 0  # the third kind's blocks came back with the slots
        s = eng.new_sequence()  # the state of a reused slot starts from zero
        assert rel_err(eng.step([StepEntry(s, b, range(9))]), wb) < TOL
        assert eng.max_sequence_tokens == toy_parts.TOY["positions"]
    finally:
        toy_parts.unregister_toys()


def _replayed_graphs():
    """Stand-ins for captured graphs on the CPU: a launch runs the step's body from the graph's own
    arrays, as a replay does, so arrays that were not written anew give the wrong tokens here too."""
    from longbow_quarrel_amd.engine.decode import DecodeGraph, DecodeGraphs

    log = []

    class ReplayedGraph(DecodeGraph):
        def load(self, slots, tokens, starts):
            log.append(("load", self.batch, tuple(slots)))
            super().load(slots, tokens, starts)

        def capture(self, sampler):
            log.append(("capture", self.batch))
            self._sampler = sampler
            self.handle = 1

        def launch(self):
            log.append(("launch", self.batch))
            self.run_body(self._sampler)

        def destroy(self):
            self.handle = None

    class ReplayedGraphs(DecodeGraphs):
        graph_cls = ReplayedGraph

    return ReplayedGraphs, log


@pytest.mark.parametrize("n_prompts,max_batch", [(6, 3), (2, 1), (5, 2)])
def test_a_batch_after_another_of_the_same_size_loads_its_graph_anew(tmp_path, n_prompts, max_batch):
    """Several batches of one size in one call: the second finds a graph of its size, on the same slots,
    whose arrays still hold the first batch's last tokens and positions.  Its first decoding step must
    write them anew.  Greedy tokens with graphs equal those of direct steps and of the plain model."""
    from longbow_quarrel_amd.engine.generate import EngineBackend, GenerationLoop

    eng, ref = make(tmp_path, TINY_A)
    assert eng.graph_safe
    prompts = [random_tokens(3 + 2 * i, 256, 40 + i) for i in range(n_prompts)]
    expect = []
    for p in prompts:
        seq, out = list(p), []
        for _ in range(4):
            out.append(plain.arg_max(ref.forward(seq)[-1]))
            seq.append(out[-1])
        expect.append(out)
    graphs_cls, log = _replayed_graphs()
    for use_graphs in (False, True):
        be = EngineBackend(eng, lq.SamplingParams(), use_graphs=use_graphs, graphs_cls=graphs_cls)
        assert be.use_graphs == use_graphs
        res = GenerationLoop(be, max_batch=max_batch).run(prompts, 4, stop_ids=[])
        be.close()
        assert res.tokens == expect, use_graphs
    batches = -(-n_prompts // max_batch)
    loads = [e for e in log if e[0] == "load"]
    assert len(loads) == batches  # once a batch: no sequence ended early, so nothing else asks for one
    assert eng.cache.slots.taken_count == 0


def test_steps_queued_ahead_give_the_same_tokens_and_none_is_wasted_at_a_known_end(tmp_path):
    """A replayed step takes its tokens from where the last one left them, so the backend queues the next
    step before the host has read this one's tokens.  The tokens are those of direct steps, also when a
    sequence ends on a stop id in the middle (the step queued ahead then ran for a batch with one sequence
    too many: the others' tokens are taken from it) and when a batch ends and another follows on the same
    slots.  Where every sequence ends by its limit the loop says so, and no step is queued in vain."""
    from longbow_quarrel_amd.engine.generate import EngineBackend, GenerationLoop

    eng, ref = make(tmp_path, TINY_A)
    prompts = [random_tokens(3 + 2 * i, 256, 70 + i) for i in range(5)]
    direct = lq.generate(eng, prompts, 6, stop_ids=[], use_graphs=False)
    stop = direct.tokens[1][2]  # request 1 ends on its third token; whoever else samples it ends there too
    expect = lq.generate(eng, prompts, 6, stop_ids=[stop], use_graphs=False)
    assert expect.finish[1] == "stop" and "length" in expect.finish
    graphs_cls, log = _replayed_graphs()
    for ahead in (True, False):
        del log[:]
        be = EngineBackend(eng, lq.SamplingParams(), graphs_cls=graphs_cls)
        be.run_ahead = ahead
        res = GenerationLoop(be, max_batch=3).run(prompts, 6, stop_ids=[stop])
        assert res.tokens == expect.tokens and res.finish == expect.finish, ahead
        assert (be.steps_ahead > 0) == ahead
        launches = sum(1 for e in log if e[0] == "launch")
        assert launches >= res.decode_steps and (ahead or launches == res.decode_steps)
        del log[:]
        res = GenerationLoop(be, max_batch=3).run(prompts, 6, stop_ids=[])
        assert res.tokens == direct.tokens
        assert sum(1 for e in log if e[0] == "launch") == res.decode_steps  # every sequence ends by its limit
        be.close()
        assert be.ahead is None and eng.cache.slots.taken_count == 0


def test_a_freed_block_goes_to_a_survivor_while_a_step_is_queued_and_a_batch_follows_one_that_stopped(tmp_path):
    eng, ref = make(tmp_path, TINY_A, max_tokens=256)
    graphs_cls, log = _replayed_graphs()
    stopping_scenarios(eng, graphs_cls)


def test_prompts_run_in_portions_of_at_most_max_prefill_rows(tmp_path):
    """A batch's prompts are fed in steps of a bounded number of rows: several sequences a step, a long
    prompt over several steps (cut at 2 tokens, at a cache block's edge, anywhere), logits only from each
    prompt's last portion.  The tokens do not depend on the cutting."""
    eng, ref = make(tmp_path, TINY_C)
    prompts = [random_tokens(n, 331, 60 + n) for n in (150, 3, 64, 1, 70)]
    whole = lq.generate(eng, prompts, 3, stop_ids=[], use_graphs=False)
    expect = []
    for p in prompts:
        seq, out = list(p), []
        for _ in range(3):
            out.append(plain.arg_max(ref.forward(seq)[-1]))
            seq.append(out[-1])
        expect.append(out)
    assert whole.tokens == expect
    from longbow_quarrel_amd.engine.generate import EngineBackend, GenerationLoop
    for rows, steps in ((2, 144), (64, 5), (100, 3), (1000, 1)):  # the 288 rows, densely packed
        be = EngineBackend(eng, lq.SamplingParams(), use_graphs=False, max_prefill_rows=rows)
        res = GenerationLoop(be).run(prompts, 3, stop_ids=[])
        assert res.tokens == expect, rows
        assert be.prefill_steps == steps, (rows, be.prefill_steps)
    with pytest.raises(ValueError):
        EngineBackend(eng, lq.SamplingParams(), max_prefill_rows=0)


def test_generation_stops_where_a_sequence_may_not_grow_further(tmp_path):
    from longbow_quarrel_amd.engine import SequenceTooLong

    eng, ref = make(tmp_path, TINY_A, max_sequence_tokens=12)
    a, b = random_tokens(10, 256, 1), random_tokens(4, 256, 2)
    res = lq.generate(eng, [a, b], 6, stop_ids=[], use_graphs=False)
    # 10 prompt tokens + 2 fed back fill the 12; the third token is sampled and never fed
    assert [len(t) for t in res.tokens] == [3, 6] and res.finish == ["length", "length"]
    with pytest.raises(SequenceTooLong, match="request 1"):
        lq.generate(eng, [b, a + a], 2, stop_ids=[], use_graphs=False)
    assert eng.cache.slots.taken_count == 0


def test_the_whole_cache_is_reachable_when_pool_and_sequence_bound_are_one_figure(tmp_path):
    """The cache's pool and the bound of a sequence are the same 128 tokens (what the facade, the replay tool
    and the command line with one prompt set up): a prompt of 10 tokens gets 119 tokens, the last of them
    sampled from position 127 (the reference accepts positions below its cache size:
    internal/engine/kv_cache.go:121-124), and a larger request is clipped there, not refused."""
    eng, ref = make(tmp_path, TINY_A, max_tokens=128, max_sequence_tokens=128)
    prompt = random_tokens(10, 256, 3)
    res = lq.generate(eng, [prompt], 119, stop_ids=[], use_graphs=False)
    assert [len(t) for t in res.tokens] == [119] and res.finish == ["length"]
    for n in (120, 500):
        more = lq.generate(eng, [prompt], n, stop_ids=[], use_graphs=False)
        assert more.tokens == res.tokens and more.finish == ["length"], n
    assert eng.cache.slots.taken_count == 0 and eng.cache.free_blocks() == 2


def test_non_finite_logits_are_reported_not_sampled(tmp_path):
    """A NaN or an infinity among a row's logits stops generation with an error that names the request
    (the reference would go on from the first finite index: internal/engine/sampler.go:72-75, 107-123)."""
    folder = write_folder(tmp_path, TINY_A, 5, dtype=torch.float32)
    c, tensors = read_folder(folder)
    eng = lq.load_engine(folder, dtype="float32", max_tokens=512, device="cpu", kernels=CpuKernels())
    assert lq.generate(eng, [[1, 2, 3], [4, 5]], 3, stop_ids=[], use_graphs=False).finish == ["length"] * 2
    eng.model.head[17, :] = float("inf")  # token 17's logit overflows for every row
    with pytest.raises(lq.NonFiniteLogits, match="request 0") as caught:
        lq.generate(eng, [[1, 2, 3], [4, 5]], 3, stop_ids=[], use_graphs=False)
    assert caught.value.result.finish == ["error", "error"] and caught.value.result.tokens == [[], []]
    assert eng.cache.slots.taken_count == 0  # the failed call gave its slots back


def test_one_faulty_request_ends_alone_and_the_others_keep_their_tokens(tmp_path):
    """Only the request whose logits are not finite ends (finish "error"); the others of its batch and the
    batch after it run to their ends with the tokens they get without it, and the error that is raised at the
    end carries all of them."""
    folder = write_folder(tmp_path, TINY_A, 5, dtype=torch.float32)
    eng = lq.load_engine(folder, dtype="float32", max_tokens=512, device="cpu", kernels=CpuKernels())
    prompts = [[1, 2, 3], [4, 5], [9, 8, 7, 6], [11]]
    good = lq.generate(eng, prompts, 4, stop_ids=[], use_graphs=False, max_batch=3)
    # request 1 alone goes wrong, from its second token on: the embedding row of its first token is not finite
    first = good.tokens[1][0]
    assert all(first not in t for i, t in enumerate(good.tokens) if i != 1) and first not in sum(prompts, [])
    eng.model.embedding.table[first, 0] = float("nan")
    with pytest.raises(lq.NonFiniteLogits, match=r"request 1 \(slot") as caught:
        lq.generate(eng, prompts, 4, stop_ids=[], use_graphs=False, max_batch=3)
    res = caught.value.result
    assert res.finish == ["length", "error", "length", "length"] and res.batches == 2
    assert res.tokens == [good.tokens[0], [first], good.tokens[2], good.tokens[3]]
    assert eng.cache.slots.taken_count == 0


def test_workspace_lifetimes():
    """A plain buffer lasts until the end of the next run of the schedule and its memory comes again two
    runs later; a kept one lasts the whole step; a step's footprint is that of two runs, however many run."""
    from longbow_quarrel_amd.parts.base import Workspace

    ws = Workspace(torch.device("cpu"), 1 << 16)
    ws.reset()
    kept = ws.alloc((100,), torch.float32, keep=True)
    kept.fill_(7.0)
    seen = []
    for run in range(6):
        ws.next_run()
        t = ws.alloc((1000,), torch.float32)
        t.fill_(float(run))
        if seen:
            assert float(seen[-1][0]) == run - 1  # the run before still holds its values
        seen.append(t)
    assert seen[0].data_ptr() == seen[2].data_ptr() == seen[4].data_ptr()
    assert seen[1].data_ptr() == seen[3].data_ptr() != seen[0].data_ptr()
    assert float(kept[0]) == 7.0 and ws.high < 3 * 4096
    # a step that outgrows the buffers still runs (from the allocator), and the next step has room
    ws.next_run()
    big = ws.alloc((1 << 16,), torch.float32)
    big.zero_()
    ws.reset()
    ws.next_run()
    again = ws.alloc((1 << 16,), torch.float32)
    assert again.data_ptr() == ws.runs[ws.cur].buf.data_ptr()
    # a captured graph's buffers must not move
    ws.frozen = True
    ws.reset()
    ws.next_run()
    with pytest.raises(RuntimeError, match="too small"):
        ws.alloc((1 << 20,), torch.float32)
