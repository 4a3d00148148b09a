"""The engine's own code (step function, cache, block tables, schedule) driven on the CPU through
a stand-in for the kernel library, against the plain implementation.  The GPU tests repeat the
comparisons with the real kernels; these catch faults of the batching and the cache without one."""
import pytest
import torch

import longbow_quarrel_amd as lq
import plain
import toy_parts
from cpu_kernels import CpuKernels
from helpers import TINY_A, TINY_B, TINY_C, random_tokens, read_folder, rel_err, write_folder
from longbow_quarrel_amd.cache import CacheFull
from longbow_quarrel_amd.engine import StepEntry
from longbow_quarrel_amd.loading import random_engine
from longbow_quarrel_amd.weights import random_tensors

TOL = 2e-5


def make(tmp_path, cfg, seed=7, max_tokens=1024):
    folder = write_folder(tmp_path, cfg, seed, dtype=torch.float32)
    eng = lq.load_engine(folder, dtype="float32", max_tokens=max_tokens, device="cpu", kernels=CpuKernels())
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


def test_toy_parts_register_build_and_step_without_touching_the_framework(tmp_path):
    toy_parts.register_toys()
    try:
        cfg = toy_parts.ToyConfig.from_dict(toy_parts.TOY)
        eng = random_engine(cfg, seed=3, dtype="float32", max_tokens=512, device="cpu", kernels=CpuKernels(), std=0.2)
        assert not eng.graph_safe  # parts written with another library's operators are never captured
        assert len(eng.cache.state_groups) == 1 and len(eng.cache.kv_groups) == 1
        assert sorted(eng.cache.kv_groups[0].layers) == [1, 3]  # runs 1 and 3 own keys; run 2 reads run 1's
        tensors = random_tensors(eng.model.tensor_specs(), 3, torch.float32, 0.2)
        a, b = random_tokens(40, 53, 1), random_tokens(9, 53, 2)
        wa, wb = (toy_parts.plain_toy(toy_parts.TOY, tensors, t) for t in (a, b))
        sa, sb = eng.new_sequence(), eng.new_sequence()
        out = eng.step([StepEntry(sa, a[:17], range(17)), StepEntry(sb, b[:8], range(8))])
        assert rel_err(out[:17], wa[:17]) < TOL and rel_err(out[17:], wb[:8]) < TOL
        out = eng.step([StepEntry(sa, a[17:18], [0]), StepEntry(sb, b[8:], [0])])
        assert rel_err(out[0], wa[17]) < TOL and rel_err(out[1], wb[8]) < TOL
        eng.release(sb)
        out = eng.step([StepEntry(sa, a[18:], range(22))])
        assert rel_err(out, wa[18:]) < TOL
        eng.release(sa)
        s = eng.new_sequence()  # the state of a reused slot starts from zero
        assert rel_err(eng.step([StepEntry(s, b, range(9))]), wb) < TOL
    finally:
        toy_parts.unregister_toys()


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
