"""The sampling kernels against the plain sampler: the reference's own vectors, kept sets of
top-k and top-p, the law of the draw, the penalty ring, and independence from the batch."""
import math

import pytest
import torch

import plain
from longbow_quarrel_amd.sampling import RECENT, Sampler, SamplerState, SamplingParams, sequence_key

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
MASK = (1 << 64) - 1


@pytest.fixture(scope="module")
def kn():
    from longbow_quarrel_amd.kernels.hip import HipKernels

    return HipKernels()


def uniform_of(key, counter):
    """The n-th uniform of a sequence: splitmix64 of key + golden * (n + 1), top 53 bits."""
    z = (key + 0x9E3779B97F4A7C15 * (counter + 1)) & MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & MASK
    z ^= z >> 31
    return (z >> 11) / float(1 << 53)


def draw_in_index_order(dist, u):
    """The kernel's draw: running sum over the kept candidates in index order (the reference walks
    them in order of probability; the law of the drawn token is the same)."""
    r = u * sum(dist.values())
    acc, last = 0.0, None
    for i in sorted(dist):
        acc += dist[i]
        last = i
        if r < acc:
            return i
    return last


def run(kn, logits, params, slots=None, state=None, history=None, parts=False):
    rows, vocab = logits.shape
    slots = slots or list(range(rows))
    state = state or SamplerState(max(slots) + 1, DEV)
    if history is not None:
        for s, h in zip(slots, history):
            state.start(s, sequence_key(params.seed, s), h)
    out = torch.full((rows,), -1, dtype=torch.int32, device=DEV)
    kept = torch.zeros(rows, dtype=torch.int32, device=DEV)
    mass = torch.zeros(rows, dtype=torch.float64, device=DEV)
    seq_slot = torch.tensor(slots, dtype=torch.int32, device=DEV)
    lg = logits.clone().to(DEV)
    if params.repetition_penalty > 1:
        kn.apply_penalty(lg, seq_slot, state.recent, state.recent_n, params.repetition_penalty)
    if params.greedy:
        kn.argmax(lg, out, state.argmax_scratch, seq_slot, state.recent, state.recent_n)
    else:
        scratch = torch.empty(kn.sample_scratch_bytes(rows), dtype=torch.uint8, device=DEV) if parts else None
        kn.sample(lg, out, seq_slot, params.temperature, params.top_k, params.top_p, state.rng_key, state.rng_ctr,
                  state.recent, state.recent_n, kept, mass, scratch=scratch)
    return out.cpu().tolist(), kept.cpu().tolist(), mass.cpu().tolist(), state, lg.cpu()


def test_reference_vectors(kn):
    """internal/engine/sampler_test.go:9-106."""
    tok, *_ = run(kn, torch.tensor([[1.0, 5.0, 2.0, 0.5]]), SamplingParams())
    assert tok == [1]
    tok, *_ = run(kn, torch.tensor([[2.0, 7.0, 7.0, 7.0]]), SamplingParams())
    assert tok == [1]  # first maximal index
    wide = torch.zeros((3, 128256))
    wide[0, [99999, 500, 128255]] = 4.0   # equal maxima in different slices of the vocabulary
    wide[1, 128255] = 1.0
    wide[2] = -1.0
    tok, *_ = run(kn, wide, SamplingParams())
    assert tok == [500, 128255, 0]
    wider = torch.zeros((2, 262147))  # beyond every vocabulary that a kernel here is tuned for
    wider[0, [262146, 131072]] = 2.0
    wider[1, 262146] = 1.0
    tok, *_ = run(kn, wider, SamplingParams())
    assert tok == [131072, 262146]
    for seed in range(30):
        h = [[0]] 
        tok, kept, *_ = run(kn, torch.tensor([[2.0, 10.0, 5.0, 1.0]]), SamplingParams(temperature=1.0, top_k=1, seed=seed), history=h)
        assert tok == [1] and kept == [1]
        tok, kept, *_ = run(kn, torch.tensor([[2.0, 10.0, 5.0, 1.0]]), SamplingParams(temperature=1.0, top_k=2, seed=seed), history=h)
        assert tok[0] in (1, 2) and kept == [2]
        tok, kept, *_ = run(kn, torch.tensor([[-0.91, -1.20, -1.61, -2.30]]), SamplingParams(temperature=1.0, top_p=0.5, seed=seed), history=h)
        assert tok[0] in (0, 1) and kept == [2]
    tok, _, _, _, lg = run(kn, torch.tensor([[0.8, 1.0, 0.8]]), SamplingParams(repetition_penalty=2.0), history=[[1]])
    assert tok == [0] and lg[0].tolist() == [0.800000011920929, 0.5, 0.800000011920929]


@pytest.mark.parametrize("vocab", [331, 4096, 128256, 262147])
@pytest.mark.parametrize("temperature,top_k,top_p", [(0.8, 0, 1.0), (1.0, 40, 1.0), (0.7, 0, 0.9), (0.7, 40, 0.95),
                                                    (1.3, 5, 0.5), (0.5, 1000, 0.999)])
def test_kept_set_and_draw_follow_the_plain_sampler(kn, vocab, temperature, top_k, top_p):
    g = torch.Generator().manual_seed(vocab + top_k)
    logits = torch.randn((4, vocab), generator=g) * 3.0
    params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, seed=11)
    slots = [3, 0, 2, 5]
    tok, kept, mass, state, _ = run(kn, logits, params, slots=slots, history=[[1]] * 4)
    for r in range(4):
        dist = plain.candidate_distribution(logits[r], temperature, top_k, top_p)
        assert kept[r] == len(dist)
        u = uniform_of(sequence_key(11, slots[r]) & MASK, 0)
        assert tok[r] == draw_in_index_order(dist, u)
        assert tok[r] in dist
    assert state.rng_ctr.cpu().tolist()[:6] == [1, 0, 1, 1, 0, 1]  # each sampled sequence moved on by one draw


@pytest.mark.parametrize("vocab", [8192, 50021, 128256, 131072, 200003])
@pytest.mark.parametrize("temperature,top_k,top_p", [(1.0, 40, 1.0), (0.7, 40, 0.95), (1.3, 5, 0.5), (0.8, 1, 1.0),
                                                    (0.5, 64, 0.999), (2.0, 17, 0.3)])
def test_a_small_top_k_worked_on_in_parts_gives_what_the_one_block_kernel_and_the_plain_sampler_give(
        kn, vocab, temperature, top_k, top_p):
    """With scratch memory and top_k <= 64 the row is cut into 32 slices that leave their k largest; the
    kept set, the draw and the generator's counter are those of the kernel that walks the row alone."""
    g = torch.Generator().manual_seed(vocab + top_k)
    logits = torch.randn((5, vocab), generator=g) * 3.0
    logits[3] = (logits[3] * 2).round() / 2  # half-integer logits: many ties, in every slice
    logits[4, :] = -5.0
    logits[4, [3, vocab // 2, vocab - 1]] = torch.tensor([1.0, 1.5, 0.5])  # a peaked row: fewer candidates than k
    params = SamplingParams(temperature=temperature, top_k=top_k, top_p=top_p, seed=11)
    slots = [3, 0, 2, 5, 1]
    alone = run(kn, logits, params, slots=slots, history=[[1]] * 5)
    parts = run(kn, logits, params, slots=slots, history=[[1]] * 5, parts=True)
    assert parts[0] == alone[0] and parts[1] == alone[1]
    assert max(abs(a - b) for a, b in zip(parts[2], alone[2])) < 1e-6
    assert parts[3].rng_ctr.cpu().tolist() == alone[3].rng_ctr.cpu().tolist()
    assert parts[3].recent_n.cpu().tolist() == alone[3].recent_n.cpu().tolist()
    for r in (0, 1, 2, 4):
        dist = plain.candidate_distribution(logits[r], temperature, top_k, top_p)
        assert parts[1][r] == len(dist) and parts[0][r] in dist
        u = uniform_of(sequence_key(11, slots[r]) & MASK, 0)
        assert parts[0][r] == draw_in_index_order(dist, u)


def test_rows_with_more_ties_than_a_part_holds_go_the_long_way(kn):
    """A row of equal logits: every slice's k-th value ties with thousands, no part can hold them, and the
    row is sampled by the kernel that walks it alone; the row beside it goes through the parts."""
    vocab = 128256
    g = torch.Generator().manual_seed(9)
    logits = torch.randn((3, vocab), generator=g)
    logits[1] = 0.25
    logits[2, 1000:] = float("nan")
    params = SamplingParams(temperature=0.9, top_k=40, top_p=0.9, seed=4)
    alone = run(kn, logits, params, history=[[1]] * 3)
    parts = run(kn, logits, params, history=[[1]] * 3, parts=True)
    assert parts[0] == alone[0] and parts[1] == alone[1] and parts[0][2] == -1
    assert parts[1][1] == 40 and 0 <= parts[0][1] < 40  # the first 40 indices of the tie, in index order
    assert parts[3].rng_ctr.cpu().tolist() == alone[3].rng_ctr.cpu().tolist() == [1, 1, 0]


def test_ties_are_kept_in_index_order(kn):
    logits = torch.zeros((1, 50))
    logits[0, [7, 20, 33, 41]] = 2.0  # four equal maxima
    for k in (1, 2, 3):
        tok, kept, *_ = run(kn, logits, SamplingParams(temperature=1.0, top_k=k, seed=k), history=[[0]])
        assert kept == [k] and tok[0] in [7, 20, 33][:k]
    dist = plain.candidate_distribution(logits[0], 1.0, 3, 1.0)
    assert sorted(dist) == [7, 20, 33]


def test_draws_follow_the_law(kn):
    """20 000 draws from one distribution: chi-square against the plain sampler's probabilities."""
    logits = torch.tensor([[0.0, 1.0, 2.0, 0.5, -1.0, 3.0, -30.0, 1.5]])
    params = SamplingParams(temperature=0.9, top_k=6, top_p=0.97, seed=5)
    dist = plain.candidate_distribution(logits[0], 0.9, 6, 0.97)
    n = 20000
    rows = 500
    state = SamplerState(rows, DEV)
    for s in range(rows):
        pass
    state.rng_key.copy_(torch.tensor([sequence_key(5, s) for s in range(rows)], dtype=torch.int64))
    counts = {}
    lg = logits.expand(rows, -1).contiguous().to(DEV)
    out = torch.empty(rows, dtype=torch.int32, device=DEV)
    seq_slot = torch.arange(rows, dtype=torch.int32, device=DEV)
    for _ in range(n // rows):
        kn.sample(lg, out, seq_slot, 0.9, 6, 0.97, state.rng_key, state.rng_ctr)
        for t in out.cpu().tolist():
            counts[t] = counts.get(t, 0) + 1
    assert set(counts) <= set(dist)
    chi2 = sum((counts.get(i, 0) - n * p) ** 2 / (n * p) for i, p in dist.items())
    assert chi2 < 30.0  # 5 degrees of freedom: 30 is far in the tail (p < 2e-5)


def test_same_seed_same_draws_and_the_batch_does_not_matter(kn):
    """Two samplers with one seed give the same 20 draws (internal/engine/logit_analysis_test.go:374-398);
    a sequence's draws do not depend on which other sequences are sampled with it."""
    g = torch.Generator().manual_seed(1)
    logits = torch.randn((3, 1000), generator=g)
    p = SamplingParams(temperature=1.0, seed=12345)

    def draws(rows, slots):
        state = SamplerState(8, DEV)
        for s in slots:
            state.start(s, sequence_key(12345, 0), [1])
        seq = []
        for _ in range(20):
            tok, *_ = run(kn, logits[rows], p, slots=slots, state=state)
            seq.append(tok[0])
        return seq

    a = draws([0, 1, 2], [0, 1, 2])
    assert a == draws([0, 1, 2], [0, 1, 2]) == draws([0], [5])
    assert len(set(a)) > 10  # and they are not all the same token


def test_penalty_ring_holds_the_last_64_ids(kn):
    vocab = 200
    hist = list(range(100))  # ids 36..99 are the last 64
    logits = torch.ones((1, vocab))
    logits[0, 150] = -2.0
    tok, _, _, state, lg = run(kn, logits, SamplingParams(repetition_penalty=2.0), history=[hist + [150, 150]])
    want = plain.apply_repetition_penalty(logits[0], hist + [150, 150], 2.0)
    assert torch.equal(lg[0], want) and float(lg[0, 150]) == -4.0 and float(lg[0, 37]) == 1.0 and float(lg[0, 38]) == 0.5
    # the sampled token joins the ring
    assert int(state.recent_n[0]) == 103 and tok[0] in state.recent[0].cpu().tolist()


# --------------------------------------------------------------------------- rows that cannot be sampled from

@pytest.mark.parametrize("params", [SamplingParams(), SamplingParams(temperature=0.8, seed=3),
                                    SamplingParams(temperature=0.7, top_k=40, top_p=0.95, repetition_penalty=1.1, seed=3)])
@pytest.mark.parametrize("vocab", [331, 128256])
def test_a_row_with_a_nan_or_an_infinity_gives_no_token_and_leaves_its_state_alone(kn, params, vocab):
    """The reference scans the logits for NaN and infinities before anything else
    (internal/engine/sampler.go:72-75, 107-123) and then falls back; here such a row yields NO_TOKEN, its
    generator and its ring stay as they were, and the clean rows beside it come out as if it were not there."""
    from longbow_quarrel_amd.sampling import NonFiniteLogits

    g = torch.Generator().manual_seed(vocab)
    clean = torch.randn((5, vocab), generator=g) * 3
    history = [[1, 2, 3]] * 5

    def sample(logits):
        state = SamplerState(5, DEV)
        for s in range(5):
            state.start(s, sequence_key(params.seed, s), history[s])
        sampler = Sampler(kn, state, params)
        out = torch.full((5,), -7, dtype=torch.int32, device=DEV)
        sampler.sample(logits.clone().to(DEV), torch.arange(5, dtype=torch.int32, device=DEV), out)
        return sampler, out, state

    _, want, clean_state = sample(clean)
    assert Sampler.read_tokens(want) == want.tolist() and min(want.tolist()) >= 0
    bad = clean.clone()
    bad[1, vocab - 1] = float("nan")  # the very last entry, the row's unaligned tail
    bad[3, 5] = float("inf")
    bad[4, 0] = float("-inf")
    sampler, out, state = sample(bad)
    assert out.tolist() == [want[0].item(), -1, want[2].item(), -1, -1]
    with pytest.raises(NonFiniteLogits, match=r"row\(s\) \[1, 3, 4\]"):
        Sampler.read_tokens(out)
    # the rows that were refused: no draw taken, nothing pushed into the ring
    assert state.rng_ctr.tolist()[1] == 0 and state.recent_n.tolist()[1] == 3
    assert state.rng_ctr.tolist()[0] == clean_state.rng_ctr.tolist()[0]
    assert state.recent_n.tolist()[0] == 4 and state.recent_n.tolist()[3] == 3
