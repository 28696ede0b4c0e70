"""Weights: the safetensors container and its errors, binding by name with one error that
lists everything wrong, dtype policy, the random-weights mode."""
import json
import struct

import pytest
import torch

import tiny
from zinfer_amd import FormatError, WeightError
from zinfer_amd.models.build import build_model, declare_tensors
from zinfer_amd.weights import (SafetensorsFile, draw_tensors, load_tensors, write_model_dir,
                                write_safetensors)


def _container(header: dict, payload: bytes = b"", raw_header: bytes = None) -> bytes:
    blob = raw_header if raw_header is not None else json.dumps(header).encode()
    return struct.pack("<Q", len(blob)) + blob + payload


def test_round_trip_and_reference_vectors(tmp_path):
    """A synthetic two-tensor file as in the reference's test (src/format/safetensors.zig:
    339-376); bfloat16 [1.0, -2.5] reads back exactly (src/tensor/storage/store.zig:525-560)."""
    p = str(tmp_path / "m.safetensors")
    t = {"a": torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]]),
         "b": torch.tensor([1.0, -2.5], dtype=torch.bfloat16),
         "ids": torch.arange(5, dtype=torch.int64)}
    write_safetensors(p, t, metadata={"format": "pt"})
    with SafetensorsFile(p) as f:
        assert f.metadata == {"format": "pt"}
        assert f.infos["a"].dtype == "F32" and f.infos["a"].shape == (2, 3)
        assert f.infos["b"].dtype == "BF16"
        for k in t:
            assert torch.equal(f.tensor(k), t[k])
    from safetensors.torch import load_file       # an independent reader agrees
    other = load_file(p)
    assert all(torch.equal(other[k], t[k]) for k in t)


@pytest.mark.parametrize("code,blob", [
    ("InvalidSafetensorsFile", b"\x01\x02"),
    ("InvalidHeaderLength", struct.pack("<Q", 100) + b"{}"),
    ("HeaderTooLarge", struct.pack("<Q", 1 << 40) + b"{}"),
    ("InvalidHeaderJson", _container({}, raw_header=b"[1]")),
    ("InvalidHeaderJson", _container({}, raw_header=b"{not json")),
    ("InvalidMetadataEntry", _container({"__metadata__": {"a": 1}})),
    ("InvalidTensorEntry", _container({"t": 5})),
    ("MissingTensorField", _container({"t": {"dtype": "F32", "shape": [1]}})),
    ("InvalidTensorField", _container({"t": {"dtype": "F32", "shape": [1], "data_offsets": [0]}})),
    ("InvalidTensorField", _container({"t": {"dtype": 3, "shape": [1], "data_offsets": [0, 4]}})),
    ("UnsupportedDType", _container({"t": {"dtype": "F128", "shape": [1], "data_offsets": [0, 4]}})),
    ("InvalidIntegerValue", _container({"t": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 4]}})),
    ("InvalidDataOffsets", _container({"t": {"dtype": "F32", "shape": [1], "data_offsets": [4, 0]}}, b"\0" * 4)),
    ("TensorOutOfBounds", _container({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, b"\0" * 4)),
    ("TensorByteSizeMismatch", _container({"t": {"dtype": "F32", "shape": [2], "data_offsets": [0, 4]}}, b"\0" * 4)),
    ("OverlappingTensorData", _container({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
                                          "b": {"dtype": "F32", "shape": [1], "data_offsets": [4, 8]}}, b"\0" * 8)),
    ("NonContiguousTensorData", _container({"a": {"dtype": "F32", "shape": [1], "data_offsets": [4, 8]}}, b"\0" * 8)),
    ("NonContiguousTensorData", _container({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}}, b"\0" * 8)),
])
def test_container_errors(tmp_path, code, blob):
    """The reference's parse and layout errors (src/format/safetensors.zig:38,139-336)."""
    p = tmp_path / "bad.safetensors"
    p.write_bytes(blob)
    with pytest.raises(FormatError) as e:
        SafetensorsFile(str(p))
    assert e.value.code == code


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = tiny.config_of("A")
    decls = declare_tensors(cfg.model_spec())
    tensors = draw_tensors(decls, 1, torch.bfloat16, tied=True)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_norm.weight"] = torch.ones(8, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.ones(16, 64, dtype=torch.bfloat16)
    tensors["model.layers.7.extra.weight"] = torch.ones(3)
    (tmp_path / "config.json").write_text(json.dumps(tiny.TINY_A))
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    with pytest.raises(WeightError) as e:
        load_tensors(str(tmp_path), decls)
    msg = str(e.value)
    for needle in ("model.layers.1.mlp.up_proj.weight", "model.norm.weight", "missing (2)",
                   "model.layers.7.extra.weight", "unexpected (1)",
                   "model.layers.0.self_attn.q_norm.weight: expected shape [16], file has [8]",
                   "model.layers.0.self_attn.k_proj.weight: expected shape [32, 64], file has [16, 64]"):
        assert needle in msg, needle
    with pytest.raises(WeightError, match="no model.safetensors"):
        load_tensors(str(tmp_path / "x"), decls)


def test_tied_head_is_optional_untied_is_not(tmp_path):
    for name, tied in (("A", True), ("B", False)):
        cfg = tiny.config_of(name)
        decls = declare_tensors(cfg.model_spec())
        assert decls["lm_head.weight"].optional == tied
        tensors = draw_tensors(decls, 1, torch.float32, tied=tied)
        assert ("lm_head.weight" in tensors) == (not tied)
    d = tmp_path / "b"
    write_model_dir(str(d), tiny.config_of("B"), 3)
    t = {}
    with SafetensorsFile(str(d / "model.safetensors")) as f:
        t = {k: f.tensor(k) for k in f.names() if k != "lm_head.weight"}
    write_safetensors(str(d / "model.safetensors"), t)
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_tensors(str(d), declare_tensors(tiny.config_of("B").model_spec()))


def test_dtypes_are_kept(tmp_path):
    """bfloat16 stays bfloat16, a tensor stored in 32-bit stays so, integers become int32."""
    cfg = tiny.config_of("A")
    decls = declare_tensors(cfg.model_spec())
    tensors = draw_tensors(decls, 1, torch.bfloat16, tied=True)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()
    tensors["model.layers.0.mlp.down_proj.weight"] = \
        tensors["model.layers.0.mlp.down_proj.weight"].float()
    (tmp_path / "config.json").write_text(json.dumps(tiny.TINY_A))
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    got = load_tensors(str(tmp_path), decls)
    assert got["model.norm.weight"].dtype == torch.float32
    assert got["model.layers.0.mlp.down_proj.weight"].dtype == torch.float32
    assert got["model.embed_tokens.weight"].dtype == torch.bfloat16
    model = build_model(cfg.model_spec(), got, "bfloat16", "cpu")
    assert model.blocks[0].feed_forward.down.weight.dtype == torch.float32
    assert model.blocks[1].feed_forward.down.weight.dtype == torch.bfloat16
    assert model.blocks[0].mixer.qkv.weight.shape == (4 * 16 + 2 * 2 * 16, 64)
    assert model.head.weight is model.embedding          # tied: the embedding is the head
    model32 = build_model(cfg.model_spec(), got, "float32", "cpu")
    assert model32.embedding.dtype == torch.float32


def test_float16_checkpoint_under_both_builds(tmp_path):
    """A float16 checkpoint: the 32-bit build holds its values exactly, the bfloat16 build
    rounds the matrices to bfloat16 (not 32-bit tensors of twice the bytes that would miss
    the bfloat16 kernels); gains are 32-bit either way."""
    cfg = tiny.config_of("A")
    decls = declare_tensors(cfg.model_spec())
    tensors = {k: t.to(torch.float16) for k, t in
               draw_tensors(decls, 3, torch.float32, tied=True).items()}
    (tmp_path / "config.json").write_text(json.dumps(tiny.TINY_A))
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    got = load_tensors(str(tmp_path), decls)
    down = "model.layers.0.mlp.down_proj.weight"
    m32 = build_model(cfg.model_spec(), got, "float32", "cpu")
    assert m32.blocks[0].feed_forward.down.weight.dtype == torch.float32
    assert torch.equal(m32.blocks[0].feed_forward.down.weight, tensors[down].float())
    assert torch.equal(m32.embedding, tensors["model.embed_tokens.weight"].float())
    m16 = build_model(cfg.model_spec(), got, "bfloat16", "cpu")
    assert m16.blocks[0].feed_forward.down.weight.dtype == torch.bfloat16
    assert torch.equal(m16.blocks[0].feed_forward.down.weight, tensors[down].to(torch.bfloat16))
    assert m16.blocks[1].mixer.qkv.weight.dtype == torch.bfloat16
    assert m16.embedding.dtype == torch.bfloat16
    for m in (m32, m16):
        assert m.final_norm.gain.dtype == torch.float32
        assert torch.equal(m.final_norm.gain, tensors["model.norm.weight"].float())


def test_random_weights_mode(tmp_path):
    a = write_model_dir(str(tmp_path / "a"), tiny.config_of("B"), seed=5, dtype=torch.bfloat16)
    b = write_model_dir(str(tmp_path / "b"), tiny.config_of("B"), seed=5, dtype=torch.bfloat16)
    c = write_model_dir(str(tmp_path / "c"), tiny.config_of("B"), seed=6, dtype=torch.bfloat16)
    decls = declare_tensors(tiny.config_of("B").model_spec())
    ta, tb, tc = (load_tensors(p, decls) for p in (a, b, c))
    assert all(torch.equal(ta[k], tb[k]) for k in ta)
    assert not torch.equal(ta["lm_head.weight"], tc["lm_head.weight"])
    w = ta["model.layers.1.mlp.gate_proj.weight"].float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.001
    g = ta["model.layers.2.self_attn.k_norm.weight"].float()
    assert float(g.min()) >= 0.9 - 1e-2 and float(g.max()) <= 1.1 + 1e-2 and g.shape == (32,)
    assert json.load(open(tmp_path / "a" / "config.json"))["torch_dtype"] == "bfloat16"


def test_counter_based_draws():
    """An element's value is a function of (seed, tensor name, index): pieces, other tensors
    and the order of drawing change nothing; the moments are those of the stated distributions."""
    import numpy as np
    from zinfer_amd.parts.base import TensorDecl
    from zinfer_amd.weights import counter_rng, draw_tensor
    key = counter_rng.tensor_key(7, "model.layers.0.mlp.up_proj.weight")
    whole = counter_rng.draw(key, 0, 50000, "normal")
    parts = np.concatenate([counter_rng.draw(key, 0, 1, "normal"),
                            counter_rng.draw(key, 1, 16383, "normal"),
                            counter_rng.draw(key, 16384, 33616, "normal")])
    assert np.array_equal(whole, parts)
    assert not np.array_equal(
        whole, counter_rng.draw(counter_rng.tensor_key(7, "model.layers.1.mlp.up_proj.weight"),
                                0, 50000, "normal"))
    assert not np.array_equal(
        whole, counter_rng.draw(counter_rng.tensor_key(8, "model.layers.0.mlp.up_proj.weight"),
                                0, 50000, "normal"))
    big = counter_rng.draw(key, 0, 400000, "normal").astype(np.float64)
    assert abs(big.mean()) < 2e-4 and abs(big.std() - 0.02) < 1e-4
    assert abs(((big / big.std()) ** 4).mean() - 3.0) < 0.05          # a normal's kurtosis
    assert abs(np.mean(np.abs(big) > 0.04) - 0.0455) < 0.002          # mass beyond two sigma
    gain = counter_rng.draw(key, 0, 100000, "gain").astype(np.float64)
    assert gain.min() >= 0.9 and gain.max() <= 1.1 and abs(gain.mean() - 1.0) < 1e-3
    assert abs(gain.std() - 0.2 / 12 ** 0.5) < 1e-3
    # through draw_tensor: bfloat16 is the nearest-even rounding of the float32 draw
    decl = TensorDecl((30, 41))
    f = draw_tensor("t", decl, 7, torch.float32)
    b = draw_tensor("t", decl, 7, torch.bfloat16)
    assert torch.equal(b, f.to(torch.bfloat16))
    assert torch.equal(f.flatten(), torch.from_numpy(
        counter_rng.draw(counter_rng.tensor_key(7, "t"), 0, 30 * 41, "normal")))
    # the library's logarithm and cosine give the same float32 values
    k = np.array([counter_rng.mix64((key + (i + 1) * counter_rng.GOLDEN) & counter_rng.MASK)
                  for i in range(3000)], dtype=np.uint64)
    k1 = (k >> np.uint64(32)).astype(np.float64)
    k2 = (k & np.uint64(0xFFFFFFFF)).astype(np.float64)
    ref = np.sqrt(-2 * np.log((k1 + 1) / 2 ** 32)) * np.cos(2 * np.pi * k2 / 2 ** 32) * 0.02
    assert np.abs(ref - whole[:3000]).max() < 1e-8


def _write_sharded(path, cfg_raw, tensors, n_shards=2):
    """A model folder whose tensors lie in several files named by model.safetensors.index.json."""
    import os
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg_raw, f)
    names = list(tensors)
    weight_map = {}
    for s in range(n_shards):
        part = names[s::n_shards]               # interleaved: a layer's tensors are split up
        fname = f"model-{s + 1:05d}-of-{n_shards:05d}.safetensors"
        write_safetensors(os.path.join(path, fname), {n: tensors[n] for n in part})
        weight_map.update({n: fname for n in part})
    with open(os.path.join(path, "model.safetensors.index.json"), "w") as f:
        json.dump({"metadata": {}, "weight_map": weight_map}, f)
    return path


def test_sharded_folder_loads_the_same_tensors(tmp_path):
    cfg = tiny.config_of("B")
    decls = declare_tensors(cfg.model_spec())
    tensors = draw_tensors(decls, 4, torch.bfloat16)
    single = write_model_dir(str(tmp_path / "one"), cfg, 4, torch.bfloat16)
    sharded = _write_sharded(str(tmp_path / "three"), tiny.TINY_B, tensors, 3)
    a, b = load_tensors(single, decls), load_tensors(sharded, decls)
    assert set(a) == set(b) == set(decls)
    assert all(torch.equal(a[k], b[k]) for k in a)
    # what is wrong is still reported in one error, whichever file it lies in
    bad = dict(tensors)
    del bad["model.layers.2.mlp.up_proj.weight"]
    bad["extra.weight"] = torch.ones(2)
    with pytest.raises(WeightError) as e:
        load_tensors(_write_sharded(str(tmp_path / "bad"), tiny.TINY_B, bad, 2), decls)
    assert "model.layers.2.mlp.up_proj.weight" in str(e.value) and "extra.weight" in str(e.value)


def test_float16_weights_widen_exactly(tmp_path):
    """A float16 tensor is handed on as stored and a 32-bit build widens it exactly (it never
    passes through bfloat16, 3 bits of mantissa fewer): the model computes with the stored
    values."""
    cfg = tiny.config_of("A")
    decls = declare_tensors(cfg.model_spec())
    tensors = {k: v.to(torch.float16) for k, v in draw_tensors(decls, 2, torch.float32, tied=True).items()}
    (tmp_path / "config.json").write_text(json.dumps(tiny.TINY_A))
    write_safetensors(str(tmp_path / "model.safetensors"), tensors)
    got = load_tensors(str(tmp_path), decls)
    for k, v in tensors.items():
        assert got[k].dtype == torch.float16 and torch.equal(got[k], v), k
    assert not torch.equal(tensors["model.embed_tokens.weight"].float(),
                           tensors["model.embed_tokens.weight"].to(torch.bfloat16).float())
    model = build_model(cfg.model_spec(), got, "float32", "cpu")
    assert torch.equal(model.embedding, tensors["model.embed_tokens.weight"].float())
    assert torch.equal(model.blocks[0].ff_norm.gain,
                       tensors["model.layers.0.post_attention_layernorm.weight"].float())
