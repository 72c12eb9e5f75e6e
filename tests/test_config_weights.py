"""Configuration and registry, safetensors reading, weight errors, random-weights mode."""
import json
import os
import struct

import pytest
import torch

from helpers import TINY_A, TINY_B, TINY_C, make_folder, read_folder
from reinfer_amd.config import (ConfigError, Qwen3Config, UnknownArchitecture, config_from_dict, load_config,
                                register_architecture, registered_architectures)
from reinfer_amd.models import declare_params
from reinfer_amd.weights import (ParamDecl, SafetensorsError, SafetensorsFile, WeightError, load_weights,
                                 random_tensors, write_model_folder, write_safetensors)


# ------------------------------------------------------------------ config
def test_every_field_of_a_real_qwen3_config():
    """The reference's fixture: Qwen3-0.6B (crates/arch/tests/hf_config.rs:19-41)."""
    raw = {"architectures": ["Qwen3ForCausalLM"], "model_type": "qwen3", "hidden_size": 1024,
           "num_hidden_layers": 28, "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 128,
           "intermediate_size": 3072, "vocab_size": 151936, "max_position_embeddings": 40960,
           "rope_theta": 1000000, "rms_norm_eps": 1e-06, "tie_word_embeddings": True,
           "use_sliding_window": False, "sliding_window": None, "max_window_layers": 28,
           "bos_token_id": 151643, "eos_token_id": 151645, "attention_bias": False, "rope_scaling": None,
           "torch_dtype": "bfloat16"}
    c = config_from_dict(raw)
    assert isinstance(c, Qwen3Config)
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads, c.head_dim) == \
        (1024, 28, 16, 8, 128)
    assert (c.intermediate_size, c.vocab_size, c.max_position_embeddings) == (3072, 151936, 40960)
    assert c.rope_theta == 1e6 and c.rms_norm_eps == 1e-6 and c.tie_word_embeddings
    assert c.eos_token_ids == (151645,) and c.bos_token_id == 151643
    assert c.layer_windows == (0,) * 28
    spec = c.to_spec()
    assert len(spec.blocks) == 28 and [e.block for e in spec.run_order] == list(range(28))
    m = spec.blocks[0].mixer
    assert m.qk_norm and m.position.kind == "rope_neox" and m.position.rotary_dim == 128
    assert abs(m.scale - 128 ** -0.5) < 1e-12 and not m.bias


def test_defaults_and_derived():
    raw = {"model_type": "qwen3", "hidden_size": 64, "num_hidden_layers": 1, "num_attention_heads": 4,
           "intermediate_size": 8, "vocab_size": 10, "max_position_embeddings": 32}
    c = config_from_dict(raw)
    # kv heads default to the query heads, head_dim to hidden/heads, theta 1e6, eps 1e-5
    # (crates/arch/src/llama.rs:338-372)
    assert (c.num_key_value_heads, c.head_dim, c.rope_theta, c.rms_norm_eps) == (4, 16, 1e6, 1e-5)
    assert not c.tie_word_embeddings


@pytest.mark.parametrize("key", ["max_position_embeddings", "num_hidden_layers", "hidden_size",
                                 "intermediate_size", "vocab_size", "num_attention_heads"])
def test_missing_key_names_the_key(key):
    raw = dict(TINY_A)
    del raw[key]
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert e.value.key == key and key in str(e.value)


@pytest.mark.parametrize("patch,key", [
    ({"num_key_value_heads": 0}, "num_key_value_heads"), ({"num_key_value_heads": 5}, "num_key_value_heads"),
    ({"num_key_value_heads": 3}, "num_key_value_heads"), ({"num_attention_heads": 0}, "num_attention_heads"),
    ({"rope_theta": float("inf")}, "rope_theta"), ({"rope_theta": -1.0}, "rope_theta"),
    ({"attention_bias": True}, "attention_bias"), ({"rope_scaling": {"rope_type": "yarn", "factor": 4}}, "rope_scaling"),
    ({"head_dim": 15}, "head_dim"), ({"hidden_size": "64"}, "hidden_size"),
    ({"use_sliding_window": True}, "sliding_window"), ({"layer_types": ["full_attention"]}, "layer_types"),
    ({"tie_word_embeddings": "yes"}, "tie_word_embeddings"),
    ({"hidden_act": "gelu"}, "hidden_act"), ({"hidden_act": 3}, "hidden_act"),
])
def test_bad_values_are_refused(patch, key):
    raw = dict(TINY_A)
    raw.update(patch)
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert e.value.key == key


def test_head_dim_cannot_be_derived():
    raw = dict(TINY_A, hidden_size=66)
    del raw["head_dim"]
    with pytest.raises(ConfigError) as e:
        config_from_dict(raw)
    assert e.value.key == "head_dim"


def test_unknown_architecture():
    with pytest.raises(UnknownArchitecture) as e:
        config_from_dict({"architectures": ["MambaForCausalLM"]})
    assert "MambaForCausalLM" in str(e.value)
    with pytest.raises(ConfigError):
        config_from_dict({"hidden_size": 4})
    assert "Qwen3ForCausalLM" in registered_architectures() and "qwen3" in registered_architectures()


def test_windows_per_layer():
    c = config_from_dict(TINY_C)
    assert c.layer_windows == (21, 0, 21)
    assert [b.mixer.window for b in c.to_spec().blocks] == [21, 0, 21]
    raw = dict(TINY_A, use_sliding_window=True, sliding_window=8, max_window_layers=1)
    assert config_from_dict(raw).layer_windows == (0, 8)
    # the dictionary written for a folder reads back to the same configuration
    assert config_from_dict(c.to_dict()) == c


def test_eos_list_and_generation_config(tmp_path):
    raw = dict(TINY_A, eos_token_id=[7, 9])
    assert config_from_dict(raw).eos_token_ids == (7, 9)
    d = tmp_path / "m"
    d.mkdir()
    (d / "config.json").write_text(json.dumps(dict(TINY_A, eos_token_id=3)))
    (d / "generation_config.json").write_text(json.dumps({"eos_token_id": [11, 12]}))
    assert load_config(str(d)).eos_token_ids == (11, 12)      # generation_config wins (llama.rs:406-432)


def test_registering_another_architecture():
    class Other:
        @classmethod
        def from_dict(cls, cfg):
            return "made"
    register_architecture("OtherForCausalLM", Other)
    assert config_from_dict({"architectures": ["OtherForCausalLM"]}) == "made"


# ------------------------------------------------------------- safetensors
def test_safetensors_round_trip_and_truncation(tmp_path):
    p = str(tmp_path / "x.safetensors")
    t = {"a": torch.arange(6, dtype=torch.float32).reshape(2, 3), "b": torch.randn(4).to(torch.bfloat16),
         "c": torch.tensor([1, 2, 3], dtype=torch.int64)}
    write_safetensors(p, t)
    with SafetensorsFile(p) as f:
        assert sorted(f.names()) == ["a", "b", "c"]
        for k in t:
            assert torch.equal(f.tensor(k), t[k]) and f.tensor(k).dtype == t[k].dtype
        with pytest.raises(KeyError):
            f.tensor("zz")
    raw = open(p, "rb").read()
    bad = str(tmp_path / "bad.safetensors")
    open(bad, "wb").write(raw[:5])
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(bad)
    open(bad, "wb").write(struct.pack("<Q", 10 ** 9) + raw[8:])
    with pytest.raises(SafetensorsError, match="truncated header"):
        SafetensorsFile(bad)
    open(bad, "wb").write(raw[:-4])
    with pytest.raises(SafetensorsError, match="outside the data section"):
        SafetensorsFile(bad)


# ------------------------------------------------------------------ weights
def test_random_folder_loads_and_is_reproducible(tmp_path):
    a = make_folder(tmp_path / "1", "B", "bfloat16")
    b = make_folder(tmp_path / "2", "B", "bfloat16")
    _, wa = read_folder(a)
    _, wb = read_folder(b)
    assert wa.keys() == wb.keys() and all(torch.equal(wa[k], wb[k]) for k in wa)
    cfg = load_config(a)
    decls = declare_params(cfg.to_spec())
    w = load_weights(a, decls, torch.bfloat16, torch.device("cpu"))
    assert w["model.layers.0.self_attn.q_proj.weight"].dtype == torch.bfloat16
    assert w["model.layers.0.self_attn.q_proj.weight"].shape == (256, 96)
    std = w["model.embed_tokens.weight"].float().std().item()
    assert 0.018 < std < 0.022
    n = w["model.norm.weight"].float()
    assert 0.8 <= n.min() and n.max() <= 1.2
    # a 32-bit path widens; a vector stored in 32-bit stays so under bfloat16
    w32 = load_weights(a, decls, torch.float32, torch.device("cpu"))
    assert all(t.dtype == torch.float32 for t in w32.values())
    f32 = make_folder(tmp_path / "3", "B", "float32")
    wmix = load_weights(f32, decls, torch.bfloat16, torch.device("cpu"))
    assert wmix["model.norm.weight"].dtype == torch.float32
    assert wmix["model.layers.1.mlp.down_proj.weight"].dtype == torch.bfloat16
    # another seed, other values
    other = write_model_folder(cfg, 99, str(tmp_path / "4"))
    assert not torch.equal(read_folder(other)[1]["lm_head.weight"], wa["lm_head.weight"])


def test_one_error_lists_everything(tmp_path):
    folder = make_folder(tmp_path, "A", "bfloat16")
    raw, w = read_folder(folder)
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.0.self_attn.extra.weight"] = torch.zeros(2)
    w["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64, dtype=torch.bfloat16)
    w["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)      # ignorable
    write_safetensors(os.path.join(folder, "model.safetensors"), w)
    decls = declare_params(load_config(folder).to_spec())
    with pytest.raises(WeightError) as e:
        load_weights(folder, decls, torch.bfloat16, torch.device("cpu"))
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.extra.weight"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (16, 64))]
    for s in ("model.norm.weight", "extra.weight", "expected [32, 64] got [16, 64]"):
        assert s in str(err)


def test_tied_and_untied_heads(tmp_path):
    a = make_folder(tmp_path, "A", "bfloat16")          # tied: no head tensor written or needed
    assert "lm_head.weight" not in read_folder(a)[1]
    b = make_folder(tmp_path, "B", "bfloat16")
    raw, w = read_folder(b)
    w = {k: v.to(torch.bfloat16) for k, v in w.items() if k != "lm_head.weight"}
    write_safetensors(os.path.join(b, "model.safetensors"), w)
    with pytest.raises(WeightError) as e:
        load_weights(b, declare_params(load_config(b).to_spec()), torch.bfloat16, torch.device("cpu"))
    assert e.value.missing == ["lm_head.weight"]


def test_sharded_folder(tmp_path):
    folder = make_folder(tmp_path, "A", "bfloat16")
    _, w = read_folder(folder)
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    names = sorted(w)
    half = len(names) // 2
    write_safetensors(os.path.join(folder, "s1.safetensors"), {k: w[k] for k in names[:half]})
    write_safetensors(os.path.join(folder, "s2.safetensors"), {k: w[k] for k in names[half:]})
    os.remove(os.path.join(folder, "model.safetensors"))
    index = {"weight_map": {k: ("s1.safetensors" if i < half else "s2.safetensors") for i, k in enumerate(names)}}
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as f:
        json.dump(index, f)
    got = load_weights(folder, declare_params(load_config(folder).to_spec()), torch.bfloat16, torch.device("cpu"))
    assert all(torch.equal(got[k], w[k]) for k in names)


def test_no_size_stands_in_code():
    """Parameter shapes follow the configuration, whatever it says."""
    raw = dict(TINY_B, hidden_size=40, num_attention_heads=5, num_key_value_heads=5, head_dim=24,
               intermediate_size=56, vocab_size=123, num_hidden_layers=1)
    decls = {d.name: d.shape for d in declare_params(config_from_dict(raw).to_spec())}
    assert decls["model.layers.0.self_attn.q_proj.weight"] == (120, 40)
    assert decls["model.layers.0.self_attn.o_proj.weight"] == (40, 120)
    assert decls["model.layers.0.self_attn.k_norm.weight"] == (24,)
    assert decls["model.layers.0.mlp.down_proj.weight"] == (40, 56)
    assert decls["lm_head.weight"] == (123, 40)


def test_unexpected_tensors_are_refused_unless_allowed(tmp_path):
    """A tensor that no part declares is listed in the one error; with ``allow_unexpected`` it is left
    unread and named in the report (the reference reads what it asks for and no more,
    crates/cuda/src/engine.rs:3216-3235)."""
    import torch
    from reinfer_amd.models import declare_params
    from reinfer_amd.weights import WeightError, load_weights, random_tensors, write_safetensors
    cfg = config_from_dict(TINY_A)
    decls = declare_params(cfg.to_spec())
    tensors = random_tensors(decls, 0, torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)      # a known exporter's extra: always let through
    tensors["model.extra_head.weight"] = torch.zeros(3, 3)
    os.makedirs(tmp_path / "m")
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), tensors)
    with pytest.raises(WeightError) as e:
        load_weights(str(tmp_path / "m"), decls, torch.bfloat16, torch.device("cpu"))
    assert e.value.unexpected == ["model.extra_head.weight"] and not e.value.missing
    report = {}
    got = load_weights(str(tmp_path / "m"), decls, torch.bfloat16, torch.device("cpu"), allow_unexpected=True,
                       report=report)
    assert report["unexpected"] == ["model.extra_head.weight"]
    assert "model.extra_head.weight" not in got and len(got) == len([d for d in decls if not d.optional])
    # what is missing or misshapen is still refused
    del tensors["model.norm.weight"]
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), tensors)
    with pytest.raises(WeightError) as e:
        load_weights(str(tmp_path / "m"), decls, torch.bfloat16, torch.device("cpu"), allow_unexpected=True)
    assert e.value.missing == ["model.norm.weight"] and not e.value.unexpected


def test_random_weights_are_a_function_of_seed_name_and_index():
    """A tensor's values do not depend on what else is drawn, on how the drawing is cut into pieces, or
    (checked on the GPU box) on the device; they have the asked deviation and range."""
    import torch
    import reinfer_amd.weights.random_init as ri
    from reinfer_amd.weights import ParamDecl, random_tensor, random_tensors
    a = ParamDecl("a.weight", (300, 257))
    n = ParamDecl("n.weight", (1000,), init="norm", role="vector")
    one = random_tensor(a, 5, torch.float32)
    both = random_tensors([n, a], 5, torch.float32)
    assert torch.equal(one, both["a.weight"])
    assert not torch.equal(one, random_tensor(a, 6, torch.float32))
    assert not torch.equal(one, random_tensor(ParamDecl("b.weight", (300, 257)), 5, torch.float32))
    chunk = ri._CHUNK
    try:
        ri._CHUNK = 1000
        assert torch.equal(one, random_tensor(a, 5, torch.float32))
    finally:
        ri._CHUNK = chunk
    assert abs(one.std().item() - 0.02) < 5e-4 and abs(one.mean().item()) < 3e-4
    assert one.abs().max().item() < 0.02 * 4.9
    u = both["n.weight"]
    assert 0.8 <= u.min().item() and u.max().item() < 1.2 and abs(u.mean().item() - 1.0) < 0.02
    # rounded once: the bfloat16 tensor is the rounding of the float32 one
    assert torch.equal(random_tensor(a, 5, torch.bfloat16), one.to(torch.bfloat16))
