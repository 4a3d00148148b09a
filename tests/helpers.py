"""Shared by the tests: tiny configurations that differ in every size and option,
model folders written into temporary places, and the comparison rule."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Sequence

import torch

import longbow_quarrel_amd as lq
from longbow_quarrel_amd.weights.safetensors_io import SafetensorsFile

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
    sf = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {n: sf.tensor(n) for n in sf.names()}
    sf.close()
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
TOL_F32 = 2e-5
TOL_BF16 = 1.5e-2
