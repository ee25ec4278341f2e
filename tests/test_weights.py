"""Weights: the safetensors reader and writer, the one error that lists everything wrong with
a checkpoint, storage rules, and the random-weights mode."""
import json
import os
import struct

import pytest
import torch

from axon_amd.config import config_from_dict
from axon_amd.models import build_model_description
from axon_amd.weights import (Checkpoint, CheckpointSource, RandomSource, SafetensorsError, SafetensorsFile,
                              WeightError, WeightStore, check_tensors, write_random_model, write_safetensors)
from helpers import TINY


def test_writer_and_reader_agree_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file
    t = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16), "c": torch.arange(6, dtype=torch.int32).view(2, 3),
         "d": torch.randn(2, 2, 2).to(torch.float16)}
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, t.items())
    back = load_file(ours)                                # their reader, our file
    for k in t:
        assert back[k].dtype == t[k].dtype and torch.equal(back[k], t[k])
    theirs = str(tmp_path / "theirs.safetensors")
    save_file(t, theirs)
    f = SafetensorsFile(theirs)                           # our reader, their file
    for k in t:
        assert f.dtype(k) == t[k].dtype and f.shape(k) == tuple(t[k].shape) and torch.equal(f.tensor(k), t[k])


def _raw(path, header: bytes, data: bytes, length=None):
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(header) if length is None else length) + header + data)


@pytest.mark.parametrize("case,fragment", [
    ("short", "too short"), ("length", "does not fit"), ("json", "not JSON"), ("object", "not a JSON object"),
    ("dtype", "unknown dtype"), ("dims", "bad shape"), ("outside", "outside the data"), ("bytes", "needs 16"),
    ("gap", "gap or overlap"), ("tail", "bytes after the last tensor"),
])
def test_bad_headers_are_clean_errors(tmp_path, case, fragment):
    p = str(tmp_path / "x.safetensors")
    good = {"a": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}
    data = b"\0" * 16
    if case == "short":
        open(p, "wb").write(b"abc")
    elif case == "length":
        _raw(p, json.dumps(good).encode(), data, length=1 << 40)
    elif case == "json":
        _raw(p, b"{not json", data)
    elif case == "object":
        _raw(p, b"[1, 2]", data)
    else:
        h = json.loads(json.dumps(good))
        if case == "dtype":
            h["a"]["dtype"] = "F8_E4M3X"
        elif case == "dims":
            h["a"]["shape"] = [1, 1, 1, 1, 4]
        elif case == "outside":
            h["a"]["data_offsets"] = [0, 64]
        elif case == "bytes":
            h["a"]["data_offsets"] = [0, 12]
        elif case == "gap":
            h["a"]["data_offsets"] = [4, 20]
            data = b"\0" * 20
        elif case == "tail":
            data = b"\0" * 24
        _raw(p, json.dumps(h).encode(), data)
    with pytest.raises(SafetensorsError) as e:
        SafetensorsFile(p)
    assert fragment in str(e.value)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(model_dirs, tmp_path):
    src = Checkpoint(model_dirs("A"))
    tensors = {n: src.tensor(n).clone() for n in src.names()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(64)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)       # skipped, not an error
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(32, 63)
    tensors["model.layers.1.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    d = tmp_path / "bad"
    d.mkdir()
    write_safetensors(str(d / "model.safetensors"), tensors.items())
    config = config_from_dict(TINY["A"]["config"])
    model = build_model_description(config)
    with pytest.raises(WeightError) as e:
        check_tensors(model.tensors(), CheckpointSource(Checkpoint(str(d))), config.ignores_tensor)
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.o_proj.bias"]
    assert len(err.wrong) == 2 and "[32, 63]" in str(err) and "[32, 64]" in str(err) and "int32" in str(err)
    for name in err.missing + err.unexpected:
        assert name in str(err)


def test_untied_model_needs_its_head_and_tied_may_have_one(model_dirs, tmp_path):
    src = Checkpoint(model_dirs("B"))
    tensors = {n: src.tensor(n).clone() for n in src.names() if n != "lm_head.weight"}
    d = tmp_path / "nohead"
    d.mkdir()
    write_safetensors(str(d / "model.safetensors"), tensors.items())
    model = build_model_description(config_from_dict(TINY["B"]["config"]))
    with pytest.raises(WeightError) as e:
        check_tensors(model.tensors(), CheckpointSource(Checkpoint(str(d))))
    assert e.value.missing == ["lm_head.weight"]
    tied = build_model_description(config_from_dict(dict(TINY["B"]["config"], tie_word_embeddings=True)))
    check_tensors(tied.tensors(), CheckpointSource(Checkpoint(str(d))))           # fine without
    check_tensors(tied.tensors(), CheckpointSource(src))                          # and with


def test_sharded_checkpoints(model_dirs, tmp_path):
    src = Checkpoint(model_dirs("A"))
    names = src.names()
    d = tmp_path / "sharded"
    d.mkdir()
    shards = [names[0::3], names[1::3], names[2::3]]
    weight_map = {}
    for i, part in enumerate(shards):
        fn = f"model-{i + 1:05d}-of-00003.safetensors"
        write_safetensors(str(d / fn), [(n, src.tensor(n)) for n in part])
        weight_map.update({n: fn for n in part})
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    ck = Checkpoint(str(d))
    assert sorted(ck.names()) == sorted(names)
    for n in names:
        assert torch.equal(ck.tensor(n), src.tensor(n))
    weight_map[names[0]] = "model-00002-of-00003.safetensors"                      # index names the wrong shard
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    with pytest.raises(SafetensorsError):
        Checkpoint(str(d))
    weight_map[names[0]] = "../escape.safetensors"
    (d / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    with pytest.raises(SafetensorsError) as e:
        Checkpoint(str(d))
    assert "plain file name" in str(e.value)


def test_storage_rules_on_cpu(model_dirs):
    """Matrices take the compute dtype; a vector stored in 32-bit stays so; on the 32-bit path a
    bfloat16 checkpoint is widened exactly."""
    f32_dir, bf16_dir = model_dirs("A", "float32"), model_dirs("A", "bfloat16")
    name_m, name_v = "model.layers.0.mlp.down_proj.weight", "model.layers.0.input_layernorm.weight"
    store = WeightStore(CheckpointSource(Checkpoint(f32_dir)), "cpu", torch.bfloat16)
    assert store.matrix(name_m).dtype == torch.bfloat16 and store.vector(name_v).dtype == torch.float32
    store = WeightStore(CheckpointSource(Checkpoint(bf16_dir)), "cpu", torch.bfloat16)
    assert store.matrix(name_m).dtype == torch.bfloat16 and store.vector(name_v).dtype == torch.bfloat16
    store = WeightStore(CheckpointSource(Checkpoint(bf16_dir)), "cpu", torch.float32)
    raw = Checkpoint(bf16_dir).tensor(name_m)
    assert store.matrix(name_m).dtype == torch.float32 and torch.equal(store.matrix(name_m), raw.float())
    assert store.vector(name_v).dtype == torch.float32
    fused = store.fused_matrix(["model.layers.0.mlp.gate_proj.weight", "model.layers.0.mlp.up_proj.weight"])
    assert fused.shape == (352, 64)
    assert torch.equal(fused[176:], Checkpoint(bf16_dir).tensor("model.layers.0.mlp.up_proj.weight").float())


def test_random_weights_mode(tmp_path):
    cfg = config_from_dict(TINY["B"]["config"])
    a, b, c = (str(tmp_path / x) for x in "abc")
    write_random_model(cfg, a, seed=4, std=0.05)
    write_random_model(cfg, b, seed=4, std=0.05)
    write_random_model(cfg, c, seed=5, std=0.05)
    ca, cb, cc = Checkpoint(a), Checkpoint(b), Checkpoint(c)
    assert json.load(open(os.path.join(a, "config.json")))["hidden_size"] == 96
    assert config_from_dict(json.load(open(os.path.join(a, "config.json")))) == cfg
    for n in ca.names():
        assert torch.equal(ca.tensor(n), cb.tensor(n))                     # the seed decides
    assert not torch.equal(ca.tensor("lm_head.weight"), cc.tensor("lm_head.weight"))
    w = ca.tensor("model.layers.0.mlp.gate_proj.weight")
    assert abs(w.std().item() - 0.05) < 0.005 and abs(w.mean().item()) < 0.005
    g = ca.tensor("model.norm.weight")
    assert abs(g.mean().item() - 1.0) < 0.05 and 0.05 < g.std().item() < 0.15
    assert ca.tensor("model.layers.2.self_attn.k_proj.bias").abs().max() > 0   # biases are not trivial
    check_tensors(build_model_description(cfg).tensors(), CheckpointSource(ca))
    rs = RandomSource(build_model_description(cfg).tensors(), 4, std=0.05, storage=torch.float32)
    assert torch.equal(rs.tensor("lm_head.weight"), ca.tensor("lm_head.weight"))   # same draw, not written
