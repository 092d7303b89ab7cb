"""Safetensors reading and writing, the one error of the loader, and the random-weights mode."""
import json
import os
import struct

import pytest
import torch

import arle_amd.models  # noqa: F401
from arle_amd.config import Qwen3Config
from arle_amd.models import expected_checkpoint_tensors
from arle_amd.models.qwen3 import qwen3_spec
from arle_amd.weights import (SafetensorsFile, WeightsError, load_weights, write_random_model,
                              write_safetensors)
from arle_amd.weights.safetensors_io import SafetensorsError
from tiny import ARCH, TINY_A, TINY_B


def test_safetensors_round_trip(tmp_path):
    tensors = {"a": torch.randn(3, 5).bfloat16(), "b": torch.arange(7, dtype=torch.int64),
               "c": torch.randn(2, 2, 2), "d": torch.randn(4).half()}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors, metadata={"k": "v"})
    f = SafetensorsFile(path)
    assert sorted(f.names()) == ["a", "b", "c", "d"] and f.metadata == {"k": "v"}
    for name, t in tensors.items():
        got = f.read(name)
        assert got.dtype == t.dtype and torch.equal(got, t)
    # the same bytes as the reference format: 8-byte little-endian header length, then JSON
    raw = open(path, "rb").read()
    (hlen,) = struct.unpack("<Q", raw[:8])
    assert json.loads(raw[8:8 + hlen])["a"]["dtype"] == "BF16"
    f.close()


def test_written_file_is_read_by_the_safetensors_package(tmp_path):
    st = pytest.importorskip("safetensors.torch")
    tensors = {"w": torch.randn(4, 3).bfloat16(), "n": torch.ones(3)}
    path = str(tmp_path / "y.safetensors")
    write_safetensors(path, tensors)
    back = st.load_file(path)
    assert all(torch.equal(back[k], v) for k, v in tensors.items())


def test_file_written_by_the_safetensors_package_is_read_by_the_own_reader(tmp_path):
    # what real checkpoints are: the package's writer (its own key order, padding of the header, alignment)
    st = pytest.importorskip("safetensors.torch")
    g = torch.Generator().manual_seed(3)
    tensors = {"model.embed_tokens.weight": torch.randn(37, 24, generator=g).bfloat16(),
               "z.norm": torch.randn(24, generator=g), "a.half": torch.randn(5, 3, generator=g).half(),
               "ids": torch.arange(11, dtype=torch.int64), "scalar": torch.tensor(2.5),
               "empty": torch.zeros(0, 4), "b.i32": torch.arange(6, dtype=torch.int32).reshape(2, 3),
               "flags": torch.tensor([1, 0, 255], dtype=torch.uint8)}
    path = str(tmp_path / "pkg.safetensors")
    st.save_file(tensors, path, metadata={"format": "pt"})
    f = SafetensorsFile(path)
    assert sorted(f.names()) == sorted(tensors) and f.metadata == {"format": "pt"}
    for name, t in tensors.items():
        dtype, shape = f.info(name)
        got = f.read(name)
        assert tuple(shape) == tuple(t.shape) and got.dtype == t.dtype and torch.equal(got, t), name
    f.close()


@pytest.mark.parametrize("entry", [None, 5, {}, {"dtype": "BF16", "shape": [2], "data_offsets": [0]},
                                   {"dtype": "BF16", "shape": [2], "data_offsets": "ab"},
                                   {"dtype": "BF16", "shape": [-2], "data_offsets": [0, 4]},
                                   {"dtype": None, "shape": [2], "data_offsets": [0, 4]},
                                   {"dtype": "BF16", "shape": [2 ** 40, 2 ** 40], "data_offsets": [0, 4]},
                                   {"dtype": "BF16", "shape": [2], "data_offsets": [-4, 0]}])
def test_a_damaged_header_entry_is_refused_with_the_tensors_name(tmp_path, entry):
    """Whatever stands where a tensor's dtype, shape and offsets belong: the reader's own error, naming the tensor,
    and not the exception of whatever tripped over it."""
    path = str(tmp_path / "bad.safetensors")
    header = json.dumps({"model.w": entry, "__metadata__": 5}).encode()
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(header)) + header + b"\0" * 8)
    with pytest.raises(SafetensorsError, match="model.w"):
        SafetensorsFile(path)


def test_data_length_mismatch_names_the_tensor(tmp_path):
    path = str(tmp_path / "bad.safetensors")
    header = json.dumps({"w": {"dtype": "BF16", "shape": [2, 3], "data_offsets": [0, 8]}}).encode()
    with open(path, "wb") as fh:
        fh.write(struct.pack("<Q", len(header)) + header + b"\0" * 8)
    with pytest.raises(ValueError, match="'w'.*data length mismatch"):
        SafetensorsFile(path)


def _spec(raw):
    return qwen3_spec(Qwen3Config.from_dict(raw))


def test_random_model_is_seeded_and_loads(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    d1 = write_random_model(str(tmp_path / "m1"), ARCH, cfg, seed=5, std=0.02, norm_std=0.02)
    d2 = write_random_model(str(tmp_path / "m2"), ARCH, cfg, seed=5, std=0.02, norm_std=0.02)
    d3 = write_random_model(str(tmp_path / "m3"), ARCH, cfg, seed=6, std=0.02, norm_std=0.02)
    expected = expected_checkpoint_tensors(_spec(TINY_A))
    w1, w2, w3 = (load_weights(d, expected, "cpu", torch.bfloat16) for d in (d1, d2, d3))
    assert "lm_head.weight" not in w1  # tied: the head is the embedding table
    assert all(torch.equal(w1[k], w2[k]) for k in w1)
    assert not torch.equal(w1["model.embed_tokens.weight"], w3["model.embed_tokens.weight"])
    assert all(t.dtype == torch.bfloat16 for t in w1.values())  # kept in bfloat16
    norm = w1["model.layers.0.input_layernorm.weight"].float()
    assert abs(float(norm.mean()) - 1.0) < 0.05 and float(norm.std()) > 0
    q = w1["model.layers.1.self_attn.q_proj.weight"].float()
    assert q.shape == (64, 64) and abs(float(q.std()) - 0.02) < 0.005
    # float32 engine: widened exactly
    w32 = load_weights(d1, expected, "cpu", torch.float32)
    assert all(torch.equal(w32[k], w1[k].float()) for k in w1)
    assert json.load(open(os.path.join(d1, "config.json")))["architectures"] == [ARCH]


def test_tensor_stored_in_32_bits_stays_so(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    d = write_random_model(str(tmp_path / "m"), ARCH, cfg, seed=1)
    f = SafetensorsFile(os.path.join(d, "model.safetensors"))
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()
    write_safetensors(os.path.join(d, "model.safetensors"), tensors)
    w = load_weights(d, expected_checkpoint_tensors(_spec(TINY_A)), "cpu", torch.bfloat16)
    assert w["model.norm.weight"].dtype == torch.float32
    assert w["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_B)
    d = write_random_model(str(tmp_path / "m"), ARCH, cfg, seed=1)
    path = os.path.join(d, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    del tensors["lm_head.weight"]
    del tensors["model.layers.2.mlp.up_proj.weight"]
    tensors["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(192).bfloat16()
    tensors["model.layers.1.self_attn.k_norm.weight"] = torch.ones(16).bfloat16()
    write_safetensors(path, tensors)
    with pytest.raises(WeightsError) as info:
        load_weights(d, expected_checkpoint_tensors(_spec(TINY_B)), "cpu", torch.bfloat16)
    err = info.value
    assert err.missing == ["lm_head.weight", "model.layers.2.mlp.up_proj.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert err.wrong_shape == [("model.layers.1.self_attn.k_norm.weight", (32,), (16,))]
    text = str(err)
    for needle in ("lm_head.weight", "q_proj.bias", "expected [32], found [16]"):
        assert needle in text


def test_tensors_the_model_does_not_know_are_ignored_with_a_warning(tmp_path):
    # a tied checkpoint that still stores lm_head.weight loads in the reference (it reads by name:
    # infer/src/model/qwen3/weights.rs:305-316, infer/src/weight_loader.rs:102-120) and must load here
    from arle_amd.weights.loader import UnexpectedTensors

    cfg = Qwen3Config.from_dict(TINY_A)
    assert cfg.tie_word_embeddings
    d = write_random_model(str(tmp_path / "m"), ARCH, cfg, seed=4)
    path = os.path.join(d, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"].clone()
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.ones(8)
    write_safetensors(path, tensors)
    expected = expected_checkpoint_tensors(_spec(TINY_A))
    with pytest.warns(UnexpectedTensors, match="lm_head.weight"):
        w = load_weights(d, expected, "cpu", torch.bfloat16)
    assert set(w) == set(expected) and "lm_head.weight" not in w
    with pytest.raises(WeightsError) as info:
        load_weights(d, expected, "cpu", torch.bfloat16, strict=True)
    assert info.value.unexpected == ["lm_head.weight", "model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert not info.value.missing and not info.value.wrong_shape


def test_sharded_folder_with_index(tmp_path):
    cfg = Qwen3Config.from_dict(TINY_A)
    d = write_random_model(str(tmp_path / "m"), ARCH, cfg, seed=2)
    f = SafetensorsFile(os.path.join(d, "model.safetensors"))
    tensors = {n: f.read(n) for n in f.names()}
    f.close()
    os.remove(os.path.join(d, "model.safetensors"))
    names = sorted(tensors)
    half = len(names) // 2
    shards = {"model-00001-of-00002.safetensors": names[:half], "model-00002-of-00002.safetensors": names[half:]}
    for fname, ns in shards.items():
        write_safetensors(os.path.join(d, fname), {n: tensors[n] for n in ns})
    index = {"weight_map": {n: fname for fname, ns in shards.items() for n in ns}}
    json.dump(index, open(os.path.join(d, "model.safetensors.index.json"), "w"))
    w = load_weights(d, expected_checkpoint_tensors(_spec(TINY_A)), "cpu", torch.bfloat16)
    assert all(torch.equal(w[n], tensors[n]) for n in names)
    json.dump({}, open(os.path.join(d, "model.safetensors.index.json"), "w"))
    with pytest.raises(WeightsError, match="missing weight_map"):
        load_weights(d, expected_checkpoint_tensors(_spec(TINY_A)), "cpu", torch.bfloat16)


def test_weight_fills_are_a_registry():
    from arle_amd.parts import WeightDecl
    from arle_amd.weights import register_init
    from arle_amd.weights.random_init import random_tensor

    z = random_tensor("any", WeightDecl((3, 2), init="zeros"), 1, 0.5, 0.1, torch.float32)
    assert torch.count_nonzero(z) == 0
    register_init("test_sevens", lambda shape, gen, std, norm_std, device: torch.full(shape, 7.0, device=device))
    assert float(random_tensor("x", WeightDecl((2,), init="test_sevens"), 1, 0.5, 0.1, torch.bfloat16).float().sum()) == 14.0
    with pytest.raises(ValueError, match="no way to fill a weight of kind 'nope'"):
        random_tensor("w", WeightDecl((2,), init="nope"), 1, 0.5, 0.1, torch.float32)
