"""Shared by the tests: tiny configurations that differ in every size and option,
model folders written into temporary places, and the comparison rule."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence

import torch

import longbow_quarrel_amd as lq

# Two tiny Llama configurations that share no size or option.
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 64, "intermediate_size": 128,
    "num_hidden_layers": 2, "num_attention_heads": 4, "num_key_value_heads": 2, "head_dim": 16,
    "vocab_size": 256, "max_position_embeddings": 128, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
    "rope_scaling": None, "tie_word_embeddings": False, "torch_dtype": "float32",
    "bos_token_id": 1, "eos_token_id": 2,
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 96, "intermediate_size": 320,
    "num_hidden_layers": 3, "num_attention_heads": 3, "num_key_value_heads": 1, "head_dim": 32,
    "vocab_size": 384, "max_position_embeddings": 256, "rms_norm_eps": 1e-6, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                     "high_freq_factor": 4.0, "original_max_position_embeddings": 64},
    "tie_word_embeddings": True, "torch_dtype": "bfloat16", "bos_token_id": 0, "eos_token_id": [5, 7],
}
# head_dim is not hidden/heads, sizes are no powers of two, 6 heads over 3 groups
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 80, "intermediate_size": 208,
    "num_hidden_layers": 4, "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 48,
    "vocab_size": 331, "max_position_embeddings": 512, "rms_norm_eps": 3e-6, "rope_theta": 25000.0,
    "rope_scaling": None, "tie_word_embeddings": False, "torch_dtype": "bfloat16",
    "bos_token_id": 3, "eos_token_id": 4,
}


def write_folder(tmp_path, cfg: Dict, seed: int, dtype=None, std: float = 0.02) -> str:
    config = lq.LlamaConfig.from_dict(cfg)
    folder = os.path.join(str(tmp_path), f"model_{seed}_{cfg['hidden_size']}")
    lq.write_model_folder(folder, config, seed, dtype=dtype, std=std, gain_spread=0.3)
    return folder


def read_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    # read with the container format's own package, not with the library's reader: a fault of that reader
    # (an offset, a byte order) must not reach the plain implementation and the engine alike
    from safetensors.torch import load_file

    tensors = load_file(os.path.join(folder, "model.safetensors"))
    return cfg, tensors


def random_tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest absolute difference over the largest magnitude of the expected values."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


# Tolerances, fixed once: float32 against float64 arithmetic; bfloat16 against the plain
# implementation that rounds activations to bfloat16 at the same places.
# Measured on the GPU, float32 engine against the float64 plain implementation, whole prompts of 1 to 400
# tokens: 2.2e-7 to 7.8e-7 on the tiny configurations with weights of standard deviation 0.02 to 0.1, 3.3e-6
# with the peaked attention of standard deviation 0.15.  One case is harsher by construction (weights of 0.1,
# norm gains 1 +- 0.4, head size 144): its worst single row reads 1.3e-5 and keeps the limit that it always
# had, TOL_F32_HARSH.
TOL_F32 = 1e-5
TOL_F32_HARSH = 2e-5
TOL_BF16 = 1.5e-2


def stopping_scenarios(eng, graphs_cls=None):
    """Two orders of events around a step that is queued ahead, through captured steps against direct ones.

    (1) The cache is as full as it may be (4 blocks).  C holds block 0 and ends on its fourth token; the step
    queued ahead still ran for C and wrote into block 0.  In the very next step A passes 64 tokens and is
    handed block 0, the only free one.  (2) Every sequence of a batch ends on a stop id while a step is queued
    ahead, and the next batch starts on the same slots and blocks."""
    import longbow_quarrel_amd as lq
    from longbow_quarrel_amd.engine.generate import EngineBackend, GenerationLoop

    def run(prompts, n, stops, graphs, max_batch=3):
        kw = {} if graphs_cls is None else {"graphs_cls": graphs_cls}
        be = EngineBackend(eng, lq.SamplingParams(), use_graphs=graphs, **kw)
        try:
            return GenerationLoop(be, max_batch=max_batch).run(prompts, n, stop_ids=stops), be.steps_ahead
        finally:
            be.close()

    vocab = eng.vocab_size
    for seed in range(31, 31 + 3 * 20, 3):  # (the first prompts with which the events fall as the scenario wants)
        c, a, b = random_tokens(5, vocab, seed), random_tokens(60, vocab, seed + 1), random_tokens(10, vocab, seed + 2)
        free, _ = run([c, a, b], 10, [], False)
        stop = free.tokens[0][3]
        if stop not in free.tokens[0][:3] and stop not in free.tokens[1] and stop not in free.tokens[2]:
            break
    else:
        raise AssertionError("no prompts found whose first request alone meets its stop id")
    direct, _ = run([c, a, b], 10, [stop], False)
    assert direct.finish == ["stop", "length", "length"] and len(direct.tokens[0]) == 3
    table = eng.cache.kv_groups[0]
    seen = []
    ensure = table.ensure

    def watch(slot, new_len):
        before = list(table.owned[slot])
        ensure(slot, new_len)
        if len(table.owned[slot]) > len(before) and before:
            seen.append((new_len, table.owned[slot][len(before):]))

    table.ensure = watch
    try:
        got, ahead = run([c, a, b], 10, [stop], True)
    finally:
        table.ensure = ensure
    assert got.tokens == direct.tokens and got.finish == direct.finish and ahead > 0
    assert seen == [(65, [0])]  # A's 65th token went into the block that C had just given back
    # (2) all of a batch stop at once, a step is queued, the next batch takes over slots and blocks
    for seed in range(50, 50 + 7 * 20, 7):
        prompts = [random_tokens(3 + i, vocab, seed + i) for i in range(6)]
        free, _ = run(prompts, 8, [], False)
        stops = sorted({t[2] for t in free.tokens[:3]})
        direct, _ = run(prompts, 8, stops, False)
        if direct.finish[:3] == ["stop"] * 3 and direct.batches == 2 and "length" in direct.finish:
            break
    else:
        raise AssertionError("no prompts found whose first batch ends on stop ids alone")
    got, ahead = run(prompts, 8, stops, True)
    assert got.tokens == direct.tokens and got.finish == direct.finish and ahead > 0
    assert eng.cache.slots.taken_count == 0 and eng.cache.free_blocks() == eng.cache.n_blocks
