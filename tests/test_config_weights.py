"""Configuration, registry, the safetensors container and weight errors (no GPU)."""
import json
import os
import struct

import pytest
import torch

import longbow_quarrel_amd as lq
from longbow_quarrel_amd.config import ConfigError, LlamaConfig, read_config_json
from longbow_quarrel_amd.model import DecoderModel
from longbow_quarrel_amd.parts.base import MATRIX, TABLE, VECTOR32, TensorSpec
from longbow_quarrel_amd.registry import (config_from_dict, lookup, register_architecture,
                                          registered_architectures, spec_from_config, unregister_architecture)
from longbow_quarrel_amd.weights import (SafetensorsFile, WeightError, WeightFileError, load_tensors,
                                         storage_dtype, write_safetensors)
from helpers import TINY_A, TINY_B, TINY_C, read_folder, write_folder


# --------------------------------------------------------------------------- configuration

def test_the_tiny_configurations_differ_in_every_size_and_option():
    keys = ["hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
            "head_dim", "vocab_size", "max_position_embeddings", "rms_norm_eps", "rope_theta",
            "tie_word_embeddings", "torch_dtype"]
    for k in keys:
        assert TINY_A[k] != TINY_B[k], k
    assert TINY_A["rope_scaling"] is None and TINY_B["rope_scaling"] is not None
    assert TINY_A["num_attention_heads"] // TINY_A["num_key_value_heads"] != \
        TINY_B["num_attention_heads"] // TINY_B["num_key_value_heads"]
    c = LlamaConfig.from_dict(TINY_C)
    assert c.head_dim * c.num_attention_heads != c.hidden_size  # head_dim given explicitly


def test_config_reads_every_key_and_round_trips():
    c = LlamaConfig.from_dict(TINY_B)
    assert (c.hidden_size, c.intermediate_size, c.num_hidden_layers) == (96, 320, 3)
    assert (c.num_attention_heads, c.num_key_value_heads, c.head_dim, c.vocab_size) == (3, 1, 32, 384)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and c.tie_word_embeddings
    assert c.rope_scaling.factor == 8.0 and c.rope_scaling.original_max_position_embeddings == 64
    assert c.eos_token_ids == (5, 7) and c.bos_token_id == 0
    assert LlamaConfig.from_dict(c.to_dict()) == c
    a = LlamaConfig.from_dict(TINY_A)
    assert a.eos_token_ids == (2,) and LlamaConfig.from_dict(a.to_dict()) == a


def test_config_defaults_follow_the_reference():
    """kv heads default to heads, head size to width / heads, rope base 10000, eps 1e-5
    (internal/engine/engine.go:482-542)."""
    c = LlamaConfig.from_dict({"hidden_size": 32, "num_attention_heads": 4, "intermediate_size": 64,
                               "num_hidden_layers": 1, "vocab_size": 10})
    assert c.num_key_value_heads == 4 and c.head_dim == 8 and c.rope_theta == 10000.0 and c.rms_norm_eps == 1e-5
    assert c.rope_scaling is None and not c.tie_word_embeddings and c.eos_token_ids == ()


def test_other_ways_to_write_the_rotation():
    d = dict(TINY_A)
    d["rope_scaling"] = {"rope_type": "default"}
    assert LlamaConfig.from_dict(d).rope_scaling is None
    d["rope_scaling"] = {"type": "linear", "factor": 4}
    c = LlamaConfig.from_dict(d)
    assert c.rope_scaling.rope_type == "linear" and c.rope_scaling.factor == 4.0
    assert c.to_dict()["rope_scaling"] == {"rope_type": "linear", "factor": 4.0}
    assert LlamaConfig.from_dict(c.to_dict()) == c
    # base and scaling together under `rope_parameters`
    d = {k: v for k, v in TINY_B.items() if k not in ("rope_scaling", "rope_theta")}
    d["rope_parameters"] = dict(TINY_B["rope_scaling"], rope_theta=TINY_B["rope_theta"])
    assert LlamaConfig.from_dict(d) == LlamaConfig.from_dict(TINY_B)
    d["rope_parameters"] = {"rope_type": "default", "rope_theta": 1234.0}
    c = LlamaConfig.from_dict(d)
    assert c.rope_scaling is None and c.rope_theta == 1234.0


@pytest.mark.parametrize("change,needle", [
    ({"num_attention_heads": None}, "num_attention_heads"),
    ({"intermediate_size": None}, "intermediate_size"),
    ({"vocab_size": None}, "vocab_size"),
    ({"num_key_value_heads": 3}, "not a multiple"),
    ({"num_key_value_heads": 8}, "exceeds"),
    ({"head_dim": 15}, "even"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"rope_theta": -1.0}, "rope_theta"),
    ({"hidden_size": 0}, "hidden_size"),
    ({"num_hidden_layers": 2.5}, "integer"),
    ({"attention_bias": True}, "bias"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                       "original_max_position_embeddings": 64}}, "high_freq_factor"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 4.0, "high_freq_factor": 1.0,
                       "original_max_position_embeddings": 64}}, "exceed"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 0.5, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                       "original_max_position_embeddings": 64}}, "factor"),
    ({"torch_dtype": "int8"}, "torch_dtype"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"rope_type": "linear"}}, "factor"),
])
def test_config_errors_name_the_key(change, needle):
    d = dict(TINY_A)
    d.update(change)
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(d)
    assert needle in str(e.value)


def test_head_dim_needs_a_divisible_width_only_when_it_is_not_given():
    d = dict(TINY_A, hidden_size=66)
    d.pop("head_dim")
    with pytest.raises(ConfigError):
        LlamaConfig.from_dict(d)
    assert LlamaConfig.from_dict(dict(TINY_A, hidden_size=66)).head_dim == 16


def test_registry_maps_the_architecture_name_and_lists_known_names_on_failure(tmp_path):
    assert "LlamaForCausalLM" in registered_architectures()
    assert lookup("LlamaForCausalLM")[0] is LlamaConfig
    with pytest.raises(ConfigError) as e:
        config_from_dict({"architectures": ["MambaForCausalLM"]})
    assert "MambaForCausalLM" in str(e.value) and "LlamaForCausalLM" in str(e.value)
    with pytest.raises(ConfigError):
        config_from_dict({"hidden_size": 8})
    with pytest.raises(ConfigError):
        read_config_json(str(tmp_path))
    register_architecture("Alias", LlamaConfig, lookup("LlamaForCausalLM")[1])
    try:
        assert isinstance(config_from_dict(dict(TINY_A, architectures=["Alias"])), LlamaConfig)
    finally:
        unregister_architecture("Alias")


def test_model_spec_is_built_from_the_configuration_alone():
    for cfg in (TINY_A, TINY_B, TINY_C):
        c = LlamaConfig.from_dict(cfg)
        spec = spec_from_config(c)
        assert len(spec.layers) == c.num_hidden_layers and [r.layer for r in spec.schedule] == list(range(c.num_hidden_layers))
        model = DecoderModel(spec)
        names = {s.name: s for s in model.tensor_specs()}
        assert ("lm_head.weight" in names) == (not c.tie_word_embeddings)
        assert names["model.layers.0.self_attn.k_proj.weight"].shape == (c.num_key_value_heads * c.head_dim, c.hidden_size)
        assert names["model.layers.0.self_attn.o_proj.weight"].shape == (c.hidden_size, c.num_attention_heads * c.head_dim)
        assert names["model.layers.0.mlp.down_proj.weight"].shape == (c.hidden_size, c.intermediate_size)
        assert names["model.norm.weight"].kind == VECTOR32
        att = model.blocks[0].mixer
        assert att.scale == 1.0 / (c.head_dim ** 0.5) and model.blocks[0].mixer_norm.eps == c.rms_norm_eps


# --------------------------------------------------------------------------- container and loader

def test_safetensors_round_trip_and_layout(tmp_path):
    path = str(tmp_path / "t.safetensors")
    tensors = {"a": torch.arange(6, dtype=torch.float32).view(2, 3), "b": torch.randn(5).bfloat16(),
               "c": torch.tensor([1, 2, 3], dtype=torch.int32)}
    write_safetensors(path, tensors, {"format": "pt"})
    with open(path, "rb") as f:
        (hlen,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(hlen))
    assert header["a"] == {"dtype": "F32", "shape": [2, 3], "data_offsets": [0, 24]}
    assert header["b"]["dtype"] == "BF16" and header["__metadata__"] == {"format": "pt"}
    sf = SafetensorsFile(path)
    for n, t in tensors.items():
        assert torch.equal(sf.tensor(n), t) and sf.info(n) == (t.dtype, tuple(t.shape))
    sf.close()
    # the installed reference reader of the format agrees
    from safetensors.torch import load_file
    for n, t in load_file(path).items():
        assert torch.equal(t, tensors[n])


def test_truncated_and_malformed_files_are_refused(tmp_path):
    path = str(tmp_path / "t.safetensors")
    write_safetensors(path, {"a": torch.zeros(100)})
    data = open(path, "rb").read()
    open(path, "wb").write(data[:-40])
    with pytest.raises(WeightFileError) as e:
        SafetensorsFile(path)
    assert "truncated" in str(e.value) and "'a'" in str(e.value)
    open(path, "wb").write(b"\x05")
    with pytest.raises(WeightFileError):
        SafetensorsFile(path)
    open(path, "wb").write(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(WeightFileError):
        SafetensorsFile(path)


def test_rejected_files_leave_no_open_handle_and_malformed_entries_are_weight_errors(tmp_path):
    def open_files():
        return len(os.listdir("/proc/self/fd"))

    def write_raw(path, header):
        blob = json.dumps(header).encode()
        open(path, "wb").write(struct.pack("<Q", len(blob)) + blob + b"\0" * 64)

    path = str(tmp_path / "m.safetensors")
    before = open_files()
    for header in ({"a": {"dtype": "F32", "data_offsets": [0, 4]}},  # no shape
                   {"a": {"dtype": "F32", "shape": [1], "data_offsets": [0]}},  # one offset
                   {"a": {"dtype": "F32", "shape": ["x"], "data_offsets": [0, 4]}},
                   {"a": "F32"}, ["a"]):
        write_raw(path, header)
        with pytest.raises(WeightFileError):
            SafetensorsFile(path)
    assert open_files() == before
    # a folder whose second shard is refused: the first shard is closed again
    folder = tmp_path / "sharded"
    folder.mkdir()
    write_safetensors(str(folder / "a.safetensors"), {"x": torch.zeros(3)})
    write_raw(str(folder / "b.safetensors"), {"y": {"dtype": "F32"}})
    (folder / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": "a.safetensors", "y": "b.safetensors"}}))
    from longbow_quarrel_amd.weights.safetensors_io import open_model_files
    with pytest.raises(WeightFileError, match="b.safetensors"):
        open_model_files(str(folder))
    assert open_files() == before
    (folder / "model.safetensors.index.json").write_text("{}")
    with pytest.raises(WeightFileError, match="weight_map"):
        open_model_files(str(folder))


def _shard(folder, parts):
    """Rewrites a model folder as shards with an index; `parts` maps shard file -> predicate on names."""
    cfg, tensors = read_folder(folder)
    os.remove(os.path.join(folder, "model.safetensors"))
    weight_map = {}
    for fname, take in parts.items():
        mine = {n: t for n, t in tensors.items() if take(n)}
        write_safetensors(os.path.join(folder, fname), mine)
        weight_map.update({n: fname for n in mine})
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f)
    return tensors


def test_a_sharded_folder_loads_to_the_same_tensors_and_a_name_in_two_shards_is_an_error(tmp_path):
    folder = write_folder(tmp_path, TINY_B, 4)
    model = DecoderModel(spec_from_config(config_from_dict(read_config_json(folder))))
    whole = load_tensors(folder, model.tensor_specs(), torch.bfloat16, torch.device("cpu"))
    first = lambda n: "layers.0." in n or "embed" in n
    _shard(folder, {"model-00001-of-00002.safetensors": first,
                    "model-00002-of-00002.safetensors": lambda n: not first(n)})
    sharded = load_tensors(folder, model.tensor_specs(), torch.bfloat16, torch.device("cpu"))
    assert sharded.keys() == whole.keys() and all(torch.equal(sharded[n], whole[n]) for n in whole)
    # the same name in both shards
    _, t = read_folder_shard(folder, "model-00001-of-00002.safetensors")
    dup = "model.layers.0.mlp.up_proj.weight"
    _, second = read_folder_shard(folder, "model-00002-of-00002.safetensors")
    second[dup] = t[dup]
    write_safetensors(os.path.join(folder, "model-00002-of-00002.safetensors"), second)
    with pytest.raises(WeightError) as e:
        load_tensors(folder, model.tensor_specs(), torch.bfloat16, torch.device("cpu"))
    assert dup in str(e.value) and "in both" in str(e.value)
    # a shard that lacks a tensor: the one error names it, as for a single file
    del second[dup], second["model.norm.weight"]
    write_safetensors(os.path.join(folder, "model-00002-of-00002.safetensors"), second)
    with pytest.raises(WeightError) as e:
        load_tensors(folder, model.tensor_specs(), torch.bfloat16, torch.device("cpu"))
    assert e.value.missing == ["model.norm.weight"]


def read_folder_shard(folder, fname):
    sf = SafetensorsFile(os.path.join(folder, fname))
    tensors = {n: sf.tensor(n) for n in sf.names()}
    sf.close()
    return None, tensors


def test_storage_dtype_rule():
    m, v, t = TensorSpec("m", (1,)), TensorSpec("v", (1,), kind=VECTOR32), TensorSpec("t", (1,), kind=TABLE)
    bf, f32, f16 = torch.bfloat16, torch.float32, torch.float16
    assert storage_dtype(m, bf, bf) == bf and storage_dtype(m, f16, bf) == bf
    assert storage_dtype(m, f32, bf) == f32  # a tensor stored in 32-bit stays so
    assert storage_dtype(m, bf, f32) == f32 and storage_dtype(v, bf, bf) == f32
    assert storage_dtype(t, torch.int64, bf) == torch.int32


def _rewrite(folder, change):
    cfg, tensors = read_folder(folder)
    change(tensors)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = write_folder(tmp_path, TINY_A, 1)

    def change(t):
        del t["model.layers.1.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(64)
        t["extra.weight"] = torch.zeros(3)
        t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64)
        t["lm_head.weight"] = torch.zeros(256, 32)

    _rewrite(folder, change)
    model = DecoderModel(spec_from_config(LlamaConfig.from_dict(TINY_A)))
    with pytest.raises(WeightError) as e:
        load_tensors(folder, model.tensor_specs(), torch.float32, torch.device("cpu"))
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["extra.weight", "model.layers.0.self_attn.q_proj.bias"]
    assert len(err.wrong_shape) == 2 and "expected [32, 64], found [64, 64]" in str(err)
    for name in err.missing + err.unexpected:
        assert name in str(err)


def test_a_head_in_a_tied_model_is_unexpected_and_a_missing_head_is_missing(tmp_path):
    folder = write_folder(tmp_path, TINY_B, 2)
    _rewrite(folder, lambda t: t.__setitem__("lm_head.weight", torch.zeros(384, 96)))
    model = DecoderModel(spec_from_config(LlamaConfig.from_dict(TINY_B)))
    with pytest.raises(WeightError) as e:
        load_tensors(folder, model.tensor_specs(), torch.bfloat16, torch.device("cpu"))
    assert e.value.unexpected == ["lm_head.weight"]
    folder = write_folder(tmp_path, TINY_A, 3)
    _rewrite(folder, lambda t: t.pop("lm_head.weight"))
    model = DecoderModel(spec_from_config(LlamaConfig.from_dict(TINY_A)))
    with pytest.raises(WeightError) as e:
        load_tensors(folder, model.tensor_specs(), torch.float32, torch.device("cpu"))
    assert e.value.missing == ["lm_head.weight"]


def test_loaded_dtypes_follow_the_rule(tmp_path):
    folder = write_folder(tmp_path, TINY_B, 4)  # stored in bfloat16
    model = DecoderModel(spec_from_config(LlamaConfig.from_dict(TINY_B)))
    got = load_tensors(folder, model.tensor_specs(), torch.bfloat16, torch.device("cpu"))
    assert got["model.embed_tokens.weight"].dtype == torch.bfloat16 and got["model.norm.weight"].dtype == torch.float32
    got32 = load_tensors(folder, model.tensor_specs(), torch.float32, torch.device("cpu"))
    assert all(t.dtype == torch.float32 for t in got32.values())
    assert torch.equal(got32["model.embed_tokens.weight"], got["model.embed_tokens.weight"].float())
    folder = write_folder(tmp_path, TINY_A, 5)  # stored in float32: stays so in the bfloat16 mode
    model = DecoderModel(spec_from_config(LlamaConfig.from_dict(TINY_A)))
    got = load_tensors(folder, model.tensor_specs(), torch.bfloat16, torch.device("cpu"))
    assert got["model.layers.0.mlp.down_proj.weight"].dtype == torch.float32


def test_random_weights_depend_on_seed_and_name_only(tmp_path):
    a = read_folder(write_folder(tmp_path / "x", TINY_A, 7))[1]
    b = read_folder(write_folder(tmp_path / "y", TINY_A, 7))[1]
    c = read_folder(write_folder(tmp_path / "z", TINY_A, 8))[1]
    assert all(torch.equal(a[n], b[n]) for n in a)
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    gain = a["model.norm.weight"].float()  # around one, and not one: a gain that is left out must show
    assert abs(float(gain.mean()) - 1.0) < 0.2 and float(gain.std()) > 0.1
    w = a["model.layers.0.mlp.gate_proj.weight"]
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    assert not torch.equal(w, a["model.layers.1.mlp.gate_proj.weight"])
    cfg = json.load(open(os.path.join(str(tmp_path / "x"), "model_7_64", "config.json")))
    assert cfg["architectures"] == ["LlamaForCausalLM"] and cfg["hidden_size"] == 64
