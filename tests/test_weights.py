"""Weights: the safetensors container, binding by name with one error for everything that is
wrong, which dtypes are kept, and the random-weights mode."""
import json
import os
import struct

import numpy as np
import pytest
import torch

import configs
import plain_qwen3
from lucciola_amd import models  # noqa: F401
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.engine.loading import load_model
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.weights.loader import (DictSource, FolderSource, ParamDecl, WeightsError, precision_notices,
                                         load_declared)
from lucciola_amd.weights.random_init import random_tensors, write_model_folder
from lucciola_amd.weights.safetensors_io import SafetensorsError, SafetensorsFile, write_safetensors


def some_tensors():
    g = torch.Generator().manual_seed(0)
    return {"a.weight": torch.randn(5, 7, generator=g).bfloat16(),
            "b": torch.randn(3, generator=g),
            "c.half": torch.randn(2, 2, generator=g).half(),
            "ids": torch.arange(6, dtype=torch.int64).view(2, 3),
            "scalar": torch.tensor(3.5)}


def test_round_trip(tmp_path):
    path = str(tmp_path / "x.safetensors")
    tensors = some_tensors()
    write_safetensors(path, tensors.items())
    with SafetensorsFile(path) as f:
        assert set(f.names()) == set(tensors)
        for name, t in tensors.items():
            got = f.get(name)
            assert got.dtype == t.dtype and got.shape == t.shape and torch.equal(got, t)


def test_agrees_with_the_safetensors_package(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    tensors = {k: v for k, v in some_tensors().items()}
    theirs, ours = str(tmp_path / "theirs.safetensors"), str(tmp_path / "ours.safetensors")
    st.save_file(tensors, theirs)
    with SafetensorsFile(theirs) as f:
        for name, t in tensors.items():
            assert torch.equal(f.get(name), t)
    write_safetensors(ours, tensors.items())
    loaded = st.load_file(ours)
    for name, t in tensors.items():
        assert torch.equal(loaded[name], t)


def test_container_errors(tmp_path):
    with pytest.raises(SafetensorsError, match="no such weights file"):
        SafetensorsFile(str(tmp_path / "missing.safetensors"))
    short = tmp_path / "short.safetensors"
    short.write_bytes(b"abc")
    with pytest.raises(SafetensorsError, match="too short"):
        SafetensorsFile(str(short))
    trunc = tmp_path / "trunc.safetensors"
    trunc.write_bytes(struct.pack("<Q", 10_000) + b"{}")
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(str(trunc))
    bad = tmp_path / "bad.safetensors"
    bad.write_bytes(struct.pack("<Q", 4) + b"{{{{")
    with pytest.raises(SafetensorsError, match="not valid JSON"):
        SafetensorsFile(str(bad))
    header = json.dumps({"t": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    off = tmp_path / "off.safetensors"
    off.write_bytes(struct.pack("<Q", len(header)) + header + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="needs 16 bytes"):
        SafetensorsFile(str(off))
    header = json.dumps({"t": {"dtype": "F8_E4M3", "shape": [1], "data_offsets": [0, 1]}}).encode()
    kind = tmp_path / "kind.safetensors"
    kind.write_bytes(struct.pack("<Q", len(header)) + header + b"\0")
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFile(str(kind))


def test_one_error_lists_everything():
    declared = {"w1": ParamDecl((4, 3)), "w2": ParamDecl((2, 2)), "n": ParamDecl((3,), role="vector"),
                "gone1": ParamDecl((1,)), "gone2": ParamDecl((1,))}
    source = DictSource({"w1": torch.zeros(4, 3), "w2": torch.zeros(2, 5), "n": torch.zeros(4),
                         "extra": torch.zeros(1), "w1.bias": torch.zeros(4)})
    with pytest.raises(WeightsError) as info:
        load_declared(source, declared, torch.device("cpu"))
    err = info.value
    assert err.missing == ["gone1", "gone2"]
    assert err.unexpected == ["extra", "w1.bias"]
    assert [(n, have, want) for n, have, want in err.wrong_shape] == [
        ("w2", (2, 5), (2, 2)), ("n", (4,), (3,))]
    text = str(err)
    for needle in ("gone1", "gone2", "extra", "w1.bias", "w2: file has [2, 5], model wants [2, 2]"):
        assert needle in text


def test_kept_dtypes():
    declared = {"m_bf16": ParamDecl((2, 2)), "m_f32": ParamDecl((2, 2)), "m_f16": ParamDecl((2, 2)),
                "v_bf16": ParamDecl((2,), role="vector"), "table": ParamDecl((3,), role="int")}
    source = DictSource({"m_bf16": torch.ones(2, 2).bfloat16(), "m_f32": torch.ones(2, 2),
                         "m_f16": torch.ones(2, 2).half(), "v_bf16": torch.ones(2).bfloat16(),
                         "table": torch.tensor([1, 2, 3], dtype=torch.int64)})
    out = load_declared(source, declared, torch.device("cpu"))
    assert out["m_bf16"].dtype == torch.bfloat16      # kept in bfloat16
    assert out["m_f32"].dtype == torch.float32        # stored in 32-bit: stays so
    assert out["m_f16"].dtype == torch.float32        # widened, no value changes
    assert out["v_bf16"].dtype == torch.float32       # kernels read small vectors as float32
    assert out["table"].dtype == torch.int32 and out["table"].tolist() == [1, 2, 3]
    with pytest.raises(WeightsError, match="wrong dtype"):
        load_declared(DictSource({"x": torch.zeros(2, dtype=torch.int64)}),
                      {"x": ParamDecl((2,))}, torch.device("cpu"))
    # what keeping costs is said once per class of tensor, and only where it costs something
    stored = {}
    load_declared(source, declared, torch.device("cpu"), stored_dtypes=stored)
    assert stored["m_f16"] == torch.float16 and stored["v_bf16"] == torch.bfloat16
    lines = precision_notices(stored, declared, torch.bfloat16)
    assert len(lines) == 2 and any("float32" in l and "m_f32" in l for l in lines)
    assert any("float16" in l and "m_f16" in l and "general kernel" in l for l in lines)
    assert precision_notices(stored, declared, torch.float32) == []
    only_bf16 = {"m_bf16": torch.bfloat16, "v_bf16": torch.bfloat16}
    assert precision_notices(only_bf16, declared, torch.bfloat16) == []


@pytest.mark.parametrize("key", ["A", "B", "C", "D"])
def test_random_model_folder(tmp_path, key):
    cfg, _, seed = configs.ALL[key]
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    assert json.load(open(os.path.join(folder, "config.json"))) == cfg
    arch = architecture_for(cfg)
    declared = declared_tensors(arch.model_spec(arch.read_config(cfg)))
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        assert set(f.names()) == set(declared)
        assert ("lm_head.weight" in f.names()) == (not cfg["tie_word_embeddings"])
        for name, decl in declared.items():
            t = f.get(name)
            assert t.dtype == torch.bfloat16 and tuple(t.shape) == decl.shape
            centre = 1.0 if decl.init == "ones_plus_normal" else 0.0
            assert abs(float(t.float().mean()) - centre) < 4 * cfg["initializer_range"]
            if t.numel() > 100:
                assert abs(float(t.float().std()) / cfg["initializer_range"] - 1) < 0.3
    # the same seed gives the same file, another seed another one; order does not matter
    again = dict(random_tensors(declared, seed, cfg["initializer_range"]))
    backwards = dict(random_tensors(dict(reversed(list(declared.items()))), seed, cfg["initializer_range"]))
    other = dict(random_tensors(declared, seed + 1, cfg["initializer_range"]))
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        for name in declared:
            assert torch.equal(f.get(name), again[name]) and torch.equal(again[name], backwards[name])
    assert any(not torch.equal(again[n], other[n]) for n in declared)
    model, config = load_model(folder, "float32", "cpu")
    assert len(model.layers) == cfg["num_hidden_layers"]
    assert (model.head is model.embedding) == cfg["tie_word_embeddings"]


@pytest.mark.parametrize("key", ["A", "C"])
def test_random_weights_are_a_function_of_seed_name_and_index(key):
    """Every value again from the written recipe, in numpy: bit for bit."""
    cfg, _, seed = configs.ALL[key]
    arch = architecture_for(cfg)
    declared = declared_tensors(arch.model_spec(arch.read_config(cfg)))
    std = cfg["initializer_range"]
    for name, t in random_tensors(declared, seed, std, torch.float32):
        again = plain_qwen3.random_weight(seed, name, declared[name].shape, std,
                                          plus_one=declared[name].init == "ones_plus_normal")
        assert t.dtype == torch.float32 and np.array_equal(t.numpy(), again), name
    # rounded once to bfloat16; a value does not depend on how many come before or after it
    name = "model.layers.1.mlp.down_proj.weight"
    whole = dict(random_tensors({name: declared[name]}, seed, std, torch.bfloat16))[name]
    assert torch.equal(whole, torch.from_numpy(
        plain_qwen3.random_weight(seed, name, declared[name].shape, std)).to(torch.bfloat16))
    from lucciola_amd.weights.random_init import tensor_key, unit_normal
    part = unit_normal(tensor_key(seed, name), 1000, 50, "cpu") * torch.tensor(std)
    assert torch.equal(part.to(torch.bfloat16), whole.reshape(-1)[1000:1050])
    # twelve uniform numbers less six: unit variance, nothing beyond six
    z = unit_normal(tensor_key(seed, "any"), 0, 1 << 18, "cpu")
    assert abs(float(z.mean())) < 0.01 and abs(float(z.std()) - 1) < 0.01 and float(z.abs().max()) <= 6


@pytest.mark.gpu
def test_random_weights_do_not_depend_on_the_device(tmp_path):
    """A model made on the GPU from (configuration, seed) holds the tensors of the folder
    written on the CPU from the same two."""
    from lucciola_amd.engine.loading import random_model
    cfg, _, seed = configs.ALL["B"]
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed)
    arch = architecture_for(cfg)
    declared = declared_tensors(arch.model_spec(arch.read_config(cfg)))
    on_gpu = dict(random_tensors(declared, seed, cfg["initializer_range"], torch.bfloat16, device="cuda:0"))
    as_f32 = dict(random_tensors(declared, seed, cfg["initializer_range"], torch.float32, device="cuda:0"))
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        for name in declared:
            assert torch.equal(f.get(name), on_gpu[name].cpu()), name
            assert np.array_equal(as_f32[name].cpu().numpy(), plain_qwen3.random_weight(
                seed, name, declared[name].shape, cfg["initializer_range"],
                plus_one=declared[name].init == "ones_plus_normal")), name
    made, _ = random_model(cfg, seed, "bfloat16", "cuda:0")
    loaded, _ = load_model(folder, "bfloat16", "cuda:0")
    assert torch.equal(made.embedding, loaded.embedding) and torch.equal(made.head, loaded.head)
    for a, b in zip(made.layers, loaded.layers):
        assert torch.equal(a.mixer.qkv, b.mixer.qkv) and torch.equal(a.mixer.o, b.mixer.o)
        assert torch.equal(a.feed_forward.gate_up, b.feed_forward.gate_up)
        assert torch.equal(a.feed_forward.down, b.feed_forward.down)
        assert torch.equal(a.mixer_norm.weight, b.mixer_norm.weight)


def test_folder_with_wrong_weights(tmp_path):
    cfg, _, seed = configs.ALL["A"]
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed)
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        tensors = {n: f.get(n).clone() for n in f.names()}
    del tensors["model.layers.1.mlp.up_proj.weight"]
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.ones(8).bfloat16()
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.ones(64).bfloat16()
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors.items())
    with pytest.raises(WeightsError) as info:
        load_model(folder, "float32", "cpu")
    assert info.value.missing == ["model.layers.1.mlp.up_proj.weight"]
    assert info.value.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert info.value.wrong_shape[0][0] == "model.layers.0.self_attn.q_norm.weight"
    os.remove(os.path.join(folder, "model.safetensors"))
    with pytest.raises(SafetensorsError, match="no such weights file"):
        load_model(folder, "float32", "cpu")


def test_head_follows_the_checkpoint_as_in_the_reference(tmp_path):
    # src/qwen.cc:80-84: without lm_head.weight the head is the embedding table, whatever the flag
    cfg, _, seed = configs.ALL["B"]
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed)
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        tensors = {n: f.get(n).clone() for n in f.names() if n != "lm_head.weight"}
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors.items())
    model, _ = load_model(folder, "float32", "cpu")
    assert model.head is model.embedding
    # a tied configuration may still carry a head in its checkpoint: it is not an error
    cfg_a, _, seed_a = configs.ALL["A"]
    folder_a = write_model_folder(str(tmp_path / "a"), cfg_a, seed_a)
    with SafetensorsFile(os.path.join(folder_a, "model.safetensors")) as f:
        tensors = {n: f.get(n).clone() for n in f.names()}
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    write_safetensors(os.path.join(folder_a, "model.safetensors"), tensors.items())
    model, _ = load_model(folder_a, "float32", "cpu")
    assert model.head is model.embedding


def test_sharded_checkpoint(tmp_path):
    """model.safetensors.index.json names the shard that holds each tensor."""
    cfg, _, seed = configs.ALL["B"]
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed)
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        tensors = {n: f.get(n).clone() for n in f.names()}
    os.remove(os.path.join(folder, "model.safetensors"))
    names = sorted(tensors)
    shards = {"model-00001-of-00002.safetensors": names[::2], "model-00002-of-00002.safetensors": names[1::2]}
    weight_map = {}
    for shard, members in shards.items():
        write_safetensors(os.path.join(folder, shard), [(n, tensors[n]) for n in members])
        weight_map.update({n: shard for n in members})
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as fh:
        json.dump({"metadata": {}, "weight_map": weight_map}, fh)
    source = FolderSource(folder)
    assert sorted(source.names()) == names
    assert all(torch.equal(source.get(n), tensors[n]) for n in names)
    source.close()
    model, _ = load_model(folder, "float32", "cpu")
    assert len(model.layers) == cfg["num_hidden_layers"]
    # an index that names a tensor its shard does not hold
    weight_map[names[0]] = "model-00002-of-00002.safetensors"
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as fh:
        json.dump({"weight_map": weight_map}, fh)
    with pytest.raises(WeightsError) as info:
        FolderSource(folder)
    assert info.value.missing == [names[0]]


def test_a_model_folder_is_written_without_the_kernel_library(tmp_path, monkeypatch):
    """Describing a model, declaring its tensors and writing random weights is host work: none
    of it may load (or build) the kernel library."""
    from lucciola_amd.kernels import ops

    def refuse(*args, **kwargs):
        raise AssertionError("the kernel library was asked for")
    monkeypatch.setattr(ops, "library", refuse)
    cfg, _, seed = configs.ALL["C"]
    folder = write_model_folder(str(tmp_path / "m"), cfg, seed)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
