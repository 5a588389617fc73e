"""Configuration, registry, safetensors reading and writing, and the loader's one error."""
import json
import os
import struct

import pytest
import torch

import nanoinfer_amd  # noqa: F401
from nanoinfer_amd.config.model_config import ConfigError, LlamaConfig, read_config_json
from nanoinfer_amd.registry import RegistryError, architecture_of, get_architecture, get_part
from nanoinfer_amd.weights.loader import (WeightMismatchError, expected_tensors, load_tensors, make_random_model,
                                          read_model_folder, write_model_folder)
from nanoinfer_amd.weights.safetensors_io import SafetensorsFile, WeightFileError, write_safetensors
from tiny_configs import ALL, TINY_A, TINY_B, TINY_C


# ------------------------------------------------------------------ configuration

def test_config_reads_every_key():
    c = LlamaConfig.from_dict(TINY_B)
    assert (c.hidden_size, c.num_hidden_layers, c.num_attention_heads, c.num_key_value_heads) == (192, 3, 6, 1)
    assert (c.head_dim, c.intermediate_size, c.vocab_size) == (32, 512, 1000)
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 500000.0 and c.max_position_embeddings == 512
    assert c.tie_word_embeddings is False and c.eos_token_ids == (998, 999) and c.bos_token_id == 0
    s = c.rope_scaling
    assert (s.rope_type, s.factor, s.low_freq_factor, s.high_freq_factor, s.original_max_position_embeddings) == \
        ("llama3", 4.0, 1.0, 4.0, 64)
    a = LlamaConfig.from_dict(TINY_A)
    assert a.rope_scaling is None and a.tie_word_embeddings is True and a.eos_token_ids == (2,)


def test_config_defaults_and_derived():
    d = dict(TINY_A)
    del d["head_dim"], d["num_key_value_heads"], d["rope_theta"]
    d.pop("tie_word_embeddings")
    c = LlamaConfig.from_dict(d)
    assert c.head_dim == 16 and c.num_key_value_heads == 4 and c.rope_theta == 10000.0 and not c.tie_word_embeddings
    # head_dim need not be hidden / heads
    assert LlamaConfig.from_dict(TINY_C).head_dim == 48
    # "default" scaling means none
    assert LlamaConfig.from_dict(dict(TINY_A, rope_scaling={"rope_type": "default"})).rope_scaling is None


def test_config_round_trip():
    for raw in ALL.values():
        c = LlamaConfig.from_dict(raw)
        assert LlamaConfig.from_dict(c.to_dict()) == c


@pytest.mark.parametrize("change, word", [
    ({"hidden_size": None}, "hidden_size"),
    ({"rms_norm_eps": None}, "rms_norm_eps"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"head_dim": 15}, "odd"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 2.0}}, "yarn"),
    ({"rope_scaling": {"rope_type": "llama3", "factor": 2.0}}, "low_freq_factor"),
    ({"hidden_act": "gelu"}, "gelu"),
    ({"attention_bias": True}, "bias"),
    ({"vocab_size": 0}, "vocab_size"),
    ({"architectures": []}, "architectures"),
])
def test_config_errors_name_the_fault(change, word):
    d = dict(TINY_A)
    for k, v in change.items():
        if v is None:
            del d[k]
        else:
            d[k] = v
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(d)
    assert word in str(e.value)


def test_registry_selects_by_architecture_name(tmp_path):
    assert get_architecture("LlamaForCausalLM").name == "LlamaForCausalLM"
    with pytest.raises(RegistryError) as e:
        architecture_of({"architectures": ["MambaForCausalLM"]})
    assert "MambaForCausalLM" in str(e.value) and "LlamaForCausalLM" in str(e.value)
    with pytest.raises(RegistryError):
        get_part("mixer", "hyena")
    for family, kind in [("mixer", "attention"), ("feed_forward", "swiglu"), ("norm", "rmsnorm"),
                         ("position", "rope"), ("position", "none"), ("block", "prenorm"), ("embedding", "table"),
                         ("head", "linear")]:
        assert get_part(family, kind).kind == kind
    with pytest.raises(ConfigError):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        read_config_json(str(tmp_path))


def test_spec_has_no_constant_of_its_own():
    """Every number of the spec comes from the configuration: change each key, see it arrive."""
    arch = get_architecture("LlamaForCausalLM")
    spec = arch.build_spec(arch.config_from_dict(TINY_B))
    assert len(spec.blocks) == 3 and [r.block for r in spec.order] == [0, 1, 2] and [r.cache for r in spec.order] == [0, 1, 2]
    m = spec.blocks[1].mixer
    assert m.kind == "attention" and m.params["num_heads"] == 6 and m.params["num_kv_heads"] == 1 and m.params["head_dim"] == 32
    pos = m.params["position"]
    assert pos.kind == "rope" and pos.params["theta"] == 500000.0 and pos.params["scaling"]["factor"] == 4.0
    assert pos.params["max_positions"] == 512 and pos.params["rotary_dim"] == 32
    assert spec.blocks[0].mixer_norm.params["eps"] == 1e-6 and spec.final_norm.params["eps"] == 1e-6
    assert spec.blocks[2].ffn.params["intermediate_size"] == 512
    assert spec.head.weights["weight"] == "lm_head.weight"
    tied = arch.build_spec(arch.config_from_dict(TINY_A))
    assert tied.head.weights["weight"] == tied.embedding.weights["weight"] == "model.embed_tokens.weight"
    assert m.weights["q"] == "model.layers.1.self_attn.q_proj.weight"


# ------------------------------------------------------------------ safetensors container

def test_safetensors_round_trip_and_foreign_reader(tmp_path):
    g = torch.Generator().manual_seed(0)
    tensors = {"a": torch.randn(3, 5, generator=g), "b": torch.randn(7, generator=g).to(torch.bfloat16),
               "c": torch.arange(6, dtype=torch.int64).reshape(2, 3), "d": torch.randn(2, 2, generator=g).to(torch.float16)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors, {"format": "pt"})
    f = SafetensorsFile(path)
    assert sorted(f.names()) == ["a", "b", "c", "d"] and f.shape("a") == (3, 5) and f.dtype("b") == torch.bfloat16
    for n, t in tensors.items():
        assert torch.equal(f.tensor(n), t)
    from safetensors import safe_open           # the container is the public format: another reader agrees
    with safe_open(path, framework="pt") as other:
        for n, t in tensors.items():
            assert torch.equal(other.get_tensor(n), t)
    from safetensors.torch import save_file     # ... and we read what another writer wrote
    save_file({k: v.contiguous() for k, v in tensors.items()}, str(tmp_path / "y.safetensors"))
    f2 = SafetensorsFile(str(tmp_path / "y.safetensors"))
    for n, t in tensors.items():
        assert torch.equal(f2.tensor(n), t)


def test_safetensors_damaged_files(tmp_path):
    with pytest.raises(WeightFileError):
        SafetensorsFile(str(tmp_path / "absent.safetensors"))
    p = tmp_path / "short.safetensors"
    p.write_bytes(b"\x01\x02")
    with pytest.raises(WeightFileError):
        SafetensorsFile(str(p))
    p = tmp_path / "liar.safetensors"
    p.write_bytes(struct.pack("<Q", 10 ** 9) + b"{}")
    with pytest.raises(WeightFileError):
        SafetensorsFile(str(p))
    good = str(tmp_path / "good.safetensors")
    write_safetensors(good, {"w": torch.zeros(100, 10)})
    data = open(good, "rb").read()
    trunc = tmp_path / "trunc.safetensors"
    trunc.write_bytes(data[:-500])
    with pytest.raises(WeightFileError) as e:
        SafetensorsFile(str(trunc))
    assert "'w'" in str(e.value)
    hdr = json.dumps({"w": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}).encode()
    odd = tmp_path / "odd.safetensors"
    odd.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0")
    with pytest.raises(WeightFileError) as e:
        SafetensorsFile(str(odd))
    assert "F8_E4M3" in str(e.value)


# ------------------------------------------------------------------ the loader

def test_random_model_folder_is_reproducible_and_typed(tmp_path):
    a = make_random_model(str(tmp_path / "a"), TINY_A, seed=3, dtype="bfloat16")
    b = make_random_model(str(tmp_path / "b"), TINY_A, seed=3, dtype="bfloat16")
    c = make_random_model(str(tmp_path / "c"), TINY_A, seed=4, dtype="bfloat16")
    fa, fb, fc = (SafetensorsFile(os.path.join(x, "model.safetensors")) for x in (a, b, c))
    assert sorted(fa.names()) == sorted(fb.names())
    assert "lm_head.weight" not in fa.names()                       # tied: stored once
    for n in fa.names():
        assert fa.dtype(n) == torch.bfloat16 and torch.equal(fa.tensor(n), fb.tensor(n))
    assert not torch.equal(fa.tensor("model.norm.weight"), fc.tensor("model.norm.weight"))
    w = fa.tensor("model.layers.0.mlp.down_proj.weight").float()
    assert w.shape == (64, 160) and abs(float(w.std()) - 0.02) < 0.002
    nw = fa.tensor("model.norm.weight").float()
    assert abs(float(nw.mean()) - 1.0) < 0.05
    arch, cfg, spec = read_model_folder(a)
    assert cfg == LlamaConfig.from_dict(dict(TINY_A, torch_dtype="bfloat16"))
    d32 = make_random_model(str(tmp_path / "d"), TINY_B, seed=3, dtype="float32")
    f32 = SafetensorsFile(os.path.join(d32, "model.safetensors"))
    assert "lm_head.weight" in f32.names() and all(f32.dtype(n) == torch.float32 for n in f32.names())


def test_loader_keeps_stored_types(tmp_path):
    d = make_random_model(str(tmp_path / "m"), TINY_A, seed=1, dtype="bfloat16")
    _, _, spec = read_model_folder(d)
    tensors = load_tensors(d, spec)
    assert set(tensors) == set(expected_tensors(spec))
    assert all(t.dtype == torch.bfloat16 for t in tensors.values())
    # a tensor stored in 32 bits stays so
    f = SafetensorsFile(os.path.join(d, "model.safetensors"))
    mixed = {n: (t.float() if n.endswith("norm.weight") else t) for n, t in f.items()}
    write_model_folder(str(tmp_path / "mixed"), json.load(open(os.path.join(d, "config.json"))), mixed)
    tensors = load_tensors(str(tmp_path / "mixed"), spec)
    assert tensors["model.norm.weight"].dtype == torch.float32
    assert tensors["model.layers.0.self_attn.q_proj.weight"].dtype == torch.bfloat16


def test_loader_reports_everything_in_one_error(tmp_path):
    d = make_random_model(str(tmp_path / "m"), TINY_B, seed=1, dtype="float32")
    cfg_json = json.load(open(os.path.join(d, "config.json")))
    f = SafetensorsFile(os.path.join(d, "model.safetensors"))
    tensors = dict(f.items())
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.7.extra.weight"] = torch.zeros(2)
    tensors["lm_head.weight"] = torch.zeros(999, 192)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 192)
    bad = write_model_folder(str(tmp_path / "bad"), cfg_json, tensors)
    _, _, spec = read_model_folder(bad)
    with pytest.raises(WeightMismatchError) as e:
        load_tensors(bad, spec)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.extra.weight"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["lm_head.weight", "model.layers.0.self_attn.k_proj.weight"]
    msg = str(err)
    for word in ("missing (2)", "unexpected (1)", "wrong shape (2)", "model.norm.weight", "extra.weight",
                 "[64, 192]", "[32, 192]"):
        assert word in msg, word


def test_tied_head_stored_twice_is_accepted_only_if_equal(tmp_path):
    d = make_random_model(str(tmp_path / "m"), TINY_A, seed=1, dtype="float32")
    cfg_json = json.load(open(os.path.join(d, "config.json")))
    tensors = dict(SafetensorsFile(os.path.join(d, "model.safetensors")).items())
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    ok = write_model_folder(str(tmp_path / "ok"), cfg_json, tensors)
    _, _, spec = read_model_folder(ok)
    assert "lm_head.weight" not in load_tensors(ok, spec)
    tensors["lm_head.weight"] = tensors["lm_head.weight"] + 1
    bad = write_model_folder(str(tmp_path / "bad"), cfg_json, tensors)
    with pytest.raises(WeightMismatchError) as e:
        load_tensors(bad, spec)
    assert e.value.unexpected == ["lm_head.weight"]


def test_sharded_checkpoint_is_read_through_its_index(tmp_path):
    one = make_random_model(str(tmp_path / "one"), TINY_B, seed=4, dtype="bfloat16")
    three = make_random_model(str(tmp_path / "three"), TINY_B, seed=4, dtype="bfloat16", shards=3)
    assert not os.path.exists(os.path.join(three, "model.safetensors"))
    index = json.load(open(os.path.join(three, "model.safetensors.index.json")))
    assert len(set(index["weight_map"].values())) == 3
    _, _, spec = read_model_folder(three)
    a, b = load_tensors(one, spec), load_tensors(three, spec)
    assert sorted(a) == sorted(b) and all(torch.equal(a[n], b[n]) for n in a)
    # the same single error over all shards: a tensor gone from its shard's index entry, an extra one in a shard
    del index["weight_map"]["model.norm.weight"]
    shard = os.path.join(three, index["weight_map"]["model.layers.0.mlp.up_proj.weight"])
    tensors = dict(SafetensorsFile(shard).items())
    del tensors["model.layers.0.mlp.up_proj.weight"]
    tensors["stray.weight"] = torch.zeros(3)
    from nanoinfer_amd.weights.safetensors_io import write_safetensors
    write_safetensors(shard, tensors, {"format": "pt"})
    del index["weight_map"]["model.layers.0.mlp.up_proj.weight"]
    json.dump(index, open(os.path.join(three, "model.safetensors.index.json"), "w"))
    with pytest.raises(WeightMismatchError) as e:
        load_tensors(three, spec)
    assert e.value.missing == ["model.layers.0.mlp.up_proj.weight"] and e.value.unexpected == ["stray.weight"]
    # an index that names a tensor its shard does not hold, and an index that is no index
    index["weight_map"]["model.layers.0.mlp.up_proj.weight"] = os.path.basename(shard)
    json.dump(index, open(os.path.join(three, "model.safetensors.index.json"), "w"))
    with pytest.raises(Exception) as e:
        load_tensors(three, spec)
    assert "not in their shards" in str(e.value)
    open(os.path.join(three, "model.safetensors.index.json"), "w").write("{}")
    with pytest.raises(Exception) as e:
        load_tensors(three, spec)
    assert "weight_map" in str(e.value)


# ------------------------------------------------------------------ random weights: the generator and the streamed file

def test_random_elements_depend_on_seed_name_and_index_only():
    from nanoinfer_amd.weights import random_init as R
    key = R.tensor_key(3, "model.embed_tokens.weight")
    whole = R.standard_normal(key, 0, 70000)                     # more than one block of the routine
    assert whole.dtype.name == "float32"
    cut = [R.standard_normal(key, s, n) for s, n in ((0, 1), (1, 4999), (5000, 32768), (37768, 32232))]
    assert (torch.from_numpy(whole) == torch.cat([torch.from_numpy(c) for c in cut])).all()
    far = R.standard_normal(key, (1 << 33) + 5, 100)             # indices beyond 32 bits
    assert (far != whole[:100]).any() and abs(float(far.mean())) < 0.5
    other = R.standard_normal(R.tensor_key(3, "model.norm.weight"), 0, 1000)
    again = R.standard_normal(R.tensor_key(4, "model.embed_tokens.weight"), 0, 1000)
    assert (other != whole[:1000]).any() and (again != whole[:1000]).any()
    # a standard normal: moments, tails, no trace of the neighbour
    x = torch.from_numpy(R.standard_normal(key, 0, 400000)).double()
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01
    assert abs(float((x ** 4).mean() / x.var() ** 2) - 3.0) < 0.05
    assert abs(float((x.abs() > 1.959964).double().mean()) - 0.05) < 0.003
    assert abs(float((x[:-1] * x[1:]).mean())) < 0.01
    assert float(x.abs().max()) < 6.0


def test_random_model_follows_the_architecture_s_rule_and_its_parts(tmp_path):
    from nanoinfer_amd.weights import random_init as R
    d = make_random_model(str(tmp_path / "m"), TINY_B, seed=9, dtype="float32", matrix_std=0.5, vector_mean=-2.0)
    f = SafetensorsFile(os.path.join(d, "model.safetensors"))
    _, _, spec = read_model_folder(d)
    assert set(f.names()) == set(expected_tensors(spec))
    w = f.tensor("model.layers.2.mlp.up_proj.weight")
    assert abs(float(w.std()) - 0.5) < 0.01
    assert abs(float(f.tensor("model.layers.1.input_layernorm.weight").mean()) + 2.0) < 0.05
    # an element is what the generator says for (seed, name, index), whatever the piece it was written in
    want = R.random_tensor(9, "model.layers.2.mlp.up_proj.weight", tuple(w.shape), 0.0, 0.5)
    assert torch.equal(w, want)
    with pytest.raises(TypeError):
        make_random_model(str(tmp_path / "n"), TINY_B, seed=9, dtype="float32", no_such_field=1.0)


def test_streamed_file_equals_the_file_written_whole(tmp_path, monkeypatch):
    from nanoinfer_amd.weights import random_init as R
    from nanoinfer_amd.weights.safetensors_io import write_safetensors_streamed
    whole = make_random_model(str(tmp_path / "whole"), TINY_A, seed=2, dtype="bfloat16")
    monkeypatch.setattr(R, "PIECE", 1000)                       # every matrix now comes in many pieces
    pieces = make_random_model(str(tmp_path / "pieces"), TINY_A, seed=2, dtype="bfloat16")
    a, b = (open(os.path.join(x, "model.safetensors"), "rb").read() for x in (whole, pieces))
    assert a == b
    # pieces that do not add up to the tensor, or are of another type, are an error, not a damaged file
    with pytest.raises(WeightFileError, match="pieces gave"):
        write_safetensors_streamed(str(tmp_path / "short.safetensors"),
                                   [("t", torch.float32, (4, 4), lambda: iter([torch.zeros(10)]))])
    with pytest.raises(WeightFileError, match="piece of type"):
        write_safetensors_streamed(str(tmp_path / "typed.safetensors"),
                                   [("t", torch.float32, (4,), lambda: iter([torch.zeros(4, dtype=torch.bfloat16)]))])
    assert not os.path.exists(str(tmp_path / "short.safetensors"))


def test_buffers_that_exporters_write_along_are_ignored_other_extras_are_not(tmp_path):
    d = make_random_model(str(tmp_path / "m"), TINY_A, seed=1, dtype="float32")
    cfg_json = json.load(open(os.path.join(d, "config.json")))
    tensors = dict(SafetensorsFile(os.path.join(d, "model.safetensors")).items())
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    ok = write_model_folder(str(tmp_path / "ok"), cfg_json, tensors)
    _, _, spec = read_model_folder(ok)
    assert set(load_tensors(ok, spec)) == set(expected_tensors(spec))
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.ones(64)
    bad = write_model_folder(str(tmp_path / "bad"), cfg_json, tensors)
    with pytest.raises(WeightMismatchError) as e:
        load_tensors(bad, spec)
    assert e.value.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
