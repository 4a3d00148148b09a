"""The generation loop's decisions with a scripted backend (no GPU): which requests run together,
stop tokens, sequences that end earlier, batches one after another, slots given back."""
import pytest

from longbow_quarrel_amd.cache import CacheFull
from longbow_quarrel_amd.engine.generate import GenerationLoop
from longbow_quarrel_amd.sampling import SamplingParams, sequence_key


class ScriptedBackend:
    """Every sequence emits prompt[0] + 1, + 2, ...; records what the loop asks for."""

    def __init__(self, blocks=100, slots=8):
        self.free = blocks
        self.slot_free = list(range(slots))
        self.live = {}
        self.log = []
        self.held = {}

    def free_blocks(self):
        return self.free

    def blocks_needed(self, tokens):
        return (tokens + 63) // 64

    def new_sequence(self, request_index, prompt):
        slot = self.slot_free.pop(0)
        self.live[slot] = {"req": request_index, "next": prompt[0] + 1}
        need = 1
        self.held[slot] = need
        self.free -= need
        self.log.append(("new", request_index, slot))
        return slot

    def release(self, slot):
        assert slot in self.live, "released twice"
        del self.live[slot]
        self.free += self.held.pop(slot)
        self.slot_free.insert(0, slot)
        self.log.append(("release", slot))

    def _emit(self, slots):
        out = []
        for s in slots:
            out.append(self.live[s]["next"])
            self.live[s]["next"] += 1
        return out

    def prefill(self, slots, prompts):
        self.log.append(("prefill", tuple(slots), tuple(len(p) for p in prompts)))
        return self._emit(slots)

    def decode(self, slots, last_tokens, changed):
        for s, t in zip(slots, last_tokens):
            assert t == self.live[s]["next"] - 1  # the loop feeds back what was sampled
        self.log.append(("decode", tuple(slots), changed))
        return self._emit(slots)


def test_unequal_prompts_stop_tokens_and_early_ends():
    be = ScriptedBackend()
    loop = GenerationLoop(be, max_batch=8)
    prompts = [[10, 1, 1], [20], [30, 2], [40] * 7]
    res = loop.run(prompts, max_new_tokens=5, stop_ids=[13, 21, 99])
    # request 0 emits 11 12 [13 stops]; 1 stops on its very first token; 2 and 3 run to the limit
    assert res.tokens == [[11, 12], [], [31, 32, 33, 34, 35], [41, 42, 43, 44, 45]]
    assert res.finish == ["stop", "stop", "length", "length"]
    assert res.batches == 1 and res.prefill_tokens == 13
    prefill = [e for e in be.log if e[0] == "prefill"]
    assert prefill == [("prefill", (0, 1, 2, 3), (3, 1, 2, 7))]
    decodes = [e for e in be.log if e[0] == "decode"]
    assert [len(d[1]) for d in decodes] == [3, 3, 2, 2]  # the batch shrinks as sequences end
    assert [d[2] for d in decodes] == [True, False, True, False]  # composition changes are announced
    assert not be.live and be.free == 100  # every slot was given back exactly once


def test_stop_token_can_be_returned_and_callback_sees_every_token():
    be = ScriptedBackend()
    seen = []
    res = GenerationLoop(be).run([[5], [7]], 4, stop_ids=[7], include_stop=True,
                                 callback=lambda r, t: seen.append((r, t)))
    assert res.tokens == [[6, 7], [8, 9, 10, 11]] and res.finish == ["stop", "length"]
    assert seen == [(0, 6), (1, 8), (0, 7), (1, 9), (1, 10), (1, 11)]


def test_as_many_batches_as_the_requests_need_on_the_same_slots():
    be = ScriptedBackend(slots=3)
    prompts = [[i * 10] for i in range(7)]
    res = GenerationLoop(be, max_batch=3).run(prompts, 2, stop_ids=[])
    assert res.batches == 3 and res.tokens == [[i * 10 + 1, i * 10 + 2] for i in range(7)]
    news = [e for e in be.log if e[0] == "new"]
    assert [e[1] for e in news] == list(range(7))  # in the order of the requests
    assert {e[2] for e in news} == {0, 1, 2}  # slots are used again


def test_batches_are_cut_by_what_the_cache_can_hold():
    be = ScriptedBackend(blocks=4)
    prompts = [[1] * 100, [2] * 60, [3] * 10, [4] * 200]
    res = GenerationLoop(be, max_batch=8).run(prompts, 28, stop_ids=[])
    # 128 -> 2 blocks, 88 -> 2 blocks: the first batch is requests 0 and 1; then 2 (1 block) alone
    # with 3 (228 -> 4 blocks) waiting for a batch of its own
    prefills = [e[1] for e in be.log if e[0] == "prefill"]
    assert [len(p) for p in prefills] == [2, 1, 1] and res.batches == 3
    with pytest.raises(CacheFull):
        GenerationLoop(ScriptedBackend(blocks=2), max_batch=8).run([[1] * 200], 10)


def test_the_last_sampled_token_takes_no_room_in_the_cache():
    """A request caches its prompt and all its tokens but the last (sampled, never fed back): a prompt of
    10 tokens with 119 to come fills exactly two blocks of 64, and one with 120 to come needs a third."""
    be = ScriptedBackend(blocks=2)
    res = GenerationLoop(be, max_batch=8).run([[1] * 10], 119, stop_ids=[])
    assert len(res.tokens[0]) == 119
    with pytest.raises(CacheFull, match="129 tokens"):
        GenerationLoop(ScriptedBackend(blocks=2), max_batch=8).run([[1] * 10], 120, stop_ids=[])


def test_degenerate_requests():
    be = ScriptedBackend()
    assert GenerationLoop(be).run([], 5).tokens == []
    assert GenerationLoop(be).run([[1]], 0).tokens == [[]] and not be.log
    with pytest.raises(ValueError):
        GenerationLoop(be).run([[1], []], 3)
    with pytest.raises(ValueError):
        GenerationLoop(be, max_batch=0)


def test_a_failing_step_still_gives_the_slots_back():
    be = ScriptedBackend()

    def boom(slots, last, changed):
        raise RuntimeError("step failed")

    be.decode = boom
    with pytest.raises(RuntimeError):
        GenerationLoop(be).run([[1], [2]], 3)
    assert not be.live and be.free == 100


def test_sampling_params_and_sequence_keys():
    assert SamplingParams().greedy and not SamplingParams(temperature=0.7).greedy
    with pytest.raises(ValueError):
        SamplingParams(temperature=-1)
    with pytest.raises(ValueError):
        SamplingParams(repetition_penalty=0)
    keys = {sequence_key(s, i) for s in range(3) for i in range(50)}
    assert len(keys) == 150 and all(-(1 << 63) <= k < (1 << 63) for k in keys)
    assert sequence_key(1, 2) == sequence_key(1, 2)


def test_when_a_step_calls_its_lengths_uneven():
    """The hint to the attention kernel is the kernel library's own function of the lengths alone (a host
    function, callable without a GPU): the longest at least half again the mean, two sequences or more, and
    something to share out (512 tokens).  The bound of the lengths is the longest rounded up to the library's
    bucket.  The engine asks its model, the model its mixers, and a mixer without a rule gives a power of two."""
    import ctypes

    from longbow_quarrel_amd import build
    from longbow_quarrel_amd.parts.base import Mixer

    lib = ctypes.CDLL(build.ensure_built())

    def lengths_uneven(lengths):
        return bool(lib.lq_attention_lengths_uneven((ctypes.c_int * max(1, len(lengths)))(*lengths), len(lengths)))

    assert lengths_uneven([3000, 1000]) and lengths_uneven([1401, 61, 26, 301]) and lengths_uneven([600, 200, 100])
    assert not lengths_uneven([530] * 8) and not lengths_uneven([4000]) and not lengths_uneven([])
    assert not lengths_uneven([1000, 985, 300])      # 1.31 times the mean
    assert not lengths_uneven([500, 20, 30])         # nothing long enough to share out
    assert lengths_uneven([1500, 1000, 500]) and not lengths_uneven([1499, 1000, 501])  # the bound itself: 1.5
    assert lengths_uneven([5000] + [4000] * 63) is False and lengths_uneven([8000] + [100] * 63)
    assert lib.lq_attention_length_bucket() > 0 and lib.lq_attention_length_bucket() % 64 == 0
    plain_mixer = Mixer()
    assert [plain_mixer.length_bound(None, n) for n in (1, 64, 65, 1000, 1025)] == [64, 64, 128, 1024, 2048]
    assert plain_mixer.lengths_uneven(None, [3000, 1000]) is False


def test_command_line_options_have_the_reference_names_and_a_few_more():
    """cmd/quarrel/main_metal.go:24-36 and cmd/generate_text/main.go:18-26 name the options; the count of
    tokens also answers to -len and -max-new-tokens, stop ids may be given several times."""
    from longbow_quarrel_amd.cli import build_parser

    ap = build_parser()
    a = ap.parse_args(["-model", "m", "-prompt", "1 2", "-n", "7", "-kv-cache-size", "99", "-temp", "0.5", "-topk", "3",
                       "-topp", "0.9", "-penalty", "1.2", "-stream"])
    assert (a.model, a.prompt, a.n, a.kv_cache_size, a.temp, a.topk, a.topp, a.penalty, a.stream) == \
        ("m", "1 2", 7, 99, 0.5, 3, 0.9, 1.2, True)
    d = ap.parse_args(["-model", "m"])
    assert (d.prompt_file, d.prompt_ids, d.stop_ids, d.n, d.kv_cache_size, d.temp, d.topk, d.topp, d.penalty) == \
        ("", "", [], 20, 2048, 0.7, 40, 0.95, 1.1)
    for spelling in ("-len", "--len", "-max-new-tokens", "--max-new-tokens", "--n"):
        assert ap.parse_args(["-model", "m", spelling, "5"]).n == 5
    b = ap.parse_args(["--model", "m", "--stop-id", "4", "-stop-id", "9", "--prompt-file", "p.txt", "--prompt-ids", "1,2"])
    assert b.stop_ids == [4, 9] and b.prompt_file == "p.txt" and b.prompt_ids == "1,2"
