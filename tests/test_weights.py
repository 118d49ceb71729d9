"""Safetensors by name, the one mismatch error, dtype rules and the random-weights mode (no GPU)."""

import json
import os

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINY
from somi_inference_amd.config import config_from_dict, read_config_json
from somi_inference_amd.models import collect_weight_specs, qwen2_plan
from somi_inference_amd.weights import (MATRIX, TABLE, VECTOR, RandomSource, SafetensorsError, SafetensorsSource,
                                        WeightFetcher, WeightMismatchError, WeightSpec, check_weights,
                                        device_dtype, read_header, read_tensor, write_file, write_random_model)


def test_file_format_agrees_with_the_safetensors_library(tmp_path):
    tensors = {"a": torch.randn(3, 5).bfloat16(), "b": torch.arange(7, dtype=torch.int32), "c": torch.randn(2, 2),
               "empty": torch.zeros(0, 4)}
    path = str(tmp_path / "x.safetensors")
    write_file(path, tensors)
    theirs = load_file(path)
    for name, tensor in tensors.items():
        assert torch.equal(theirs[name], tensor)
    save_file(tensors, str(tmp_path / "y.safetensors"))
    header = read_header(str(tmp_path / "y.safetensors"))
    for name, tensor in tensors.items():
        assert torch.equal(read_tensor(header[name]), tensor) and header[name].dtype == tensor.dtype


def test_broken_files_are_refused(tmp_path):
    path = tmp_path / "bad.safetensors"
    path.write_bytes(b"\x05")
    with pytest.raises(SafetensorsError, match="too short"):
        read_header(str(path))
    path.write_bytes((10**9).to_bytes(8, "little") + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        read_header(str(path))
    with pytest.raises(SafetensorsError, match="neither"):
        SafetensorsSource(str(tmp_path / "nowhere"))


def test_random_model_folder_is_reproducible_and_complete(tmp_path):
    cfg = TINY["B"]["config"]
    a = write_random_model(str(tmp_path / "a"), cfg, seed=5)
    b = write_random_model(str(tmp_path / "b"), cfg, seed=5)
    c = write_random_model(str(tmp_path / "c"), cfg, seed=6)
    wa, wb, wc = (load_file(os.path.join(d, "model.safetensors")) for d in (a, b, c))
    assert set(wa) == {s.name for s in collect_weight_specs(qwen2_plan(cfg))}
    assert all(torch.equal(wa[k], wb[k]) for k in wa)
    assert not torch.equal(wa["model.embed_tokens.weight"], wc["model.embed_tokens.weight"])
    assert all(t.dtype == torch.bfloat16 for t in wa.values())
    # N(0, 0.02) for weights and biases, 1 + N(0, 0.1) for norm scales
    big = wa["model.layers.0.mlp.gate_proj.weight"].float()
    assert abs(big.mean()) < 2e-3 and abs(big.std() - 0.02) < 2e-3
    norm = torch.cat([v.float() for k, v in wa.items() if "norm" in k])
    assert abs(norm.mean() - 1.0) < 0.05 and abs(norm.std() - 0.1) < 0.03
    # the folder's config.json builds the same typed configuration
    assert config_from_dict(read_config_json(a))[1] == cfg
    # a tensor depends on (seed, name) only, not on the others: a smaller model shares its first layer
    small = type(cfg)(**{**cfg.__dict__, "num_hidden_layers": 1})
    ws = load_file(os.path.join(write_random_model(str(tmp_path / "s"), small, seed=5), "model.safetensors"))
    assert torch.equal(ws["model.layers.0.self_attn.q_proj.weight"], wa["model.layers.0.self_attn.q_proj.weight"])


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    cfg = TINY["A"]["config"]
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=1)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 63, dtype=torch.bfloat16)
    tensors["model.layers.0.extra.weight"] = torch.zeros(2, dtype=torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)     # ignored buffer (reference :164-166)
    tensors["lm_head.weight"] = torch.zeros(256, 64, dtype=torch.bfloat16)       # tied model: tolerated (reference :161-162)
    save_file(tensors, path)
    plan = qwen2_plan(cfg)
    with pytest.raises(WeightMismatchError) as err:
        check_weights(collect_weight_specs(plan), SafetensorsSource(folder), plan.ignore_weights)
    assert err.value.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.value.unexpected == ["model.layers.0.extra.weight"]
    assert err.value.wrong_shape == [("model.layers.0.self_attn.q_proj.weight", (64, 63), (64, 64))]
    text = str(err.value)
    for word in ("missing", "unexpected", "wrong shapes", "up_proj", "extra", "(64, 63)"):
        assert word in text


def test_untied_model_needs_its_head(tmp_path):
    cfg = TINY["B"]["config"]
    folder = write_random_model(str(tmp_path / "m"), cfg, seed=1)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["lm_head.weight"]
    save_file(tensors, path)
    plan = qwen2_plan(cfg)
    with pytest.raises(WeightMismatchError, match="lm_head.weight"):
        check_weights(collect_weight_specs(plan), SafetensorsSource(folder), plan.ignore_weights)


def test_integer_and_float_kinds_are_checked(tmp_path):
    write_file(str(tmp_path / "model.safetensors"), {"t": torch.zeros(4), "w": torch.zeros(4, dtype=torch.int64)})
    specs = [WeightSpec("t", (4,), TABLE), WeightSpec("w", (4,), VECTOR)]
    with pytest.raises(WeightMismatchError, match="wrong dtypes"):
        check_weights(specs, SafetensorsSource(str(tmp_path)))


def test_dtype_rules_on_the_device():
    assert device_dtype(MATRIX, torch.bfloat16) == torch.bfloat16 and device_dtype(MATRIX, torch.float32) == torch.float32
    assert device_dtype(VECTOR, torch.bfloat16) == torch.float32      # scales and biases stay 32-bit
    assert device_dtype(TABLE, torch.bfloat16) == torch.int32


def test_fetcher_casts_by_role(tmp_path):
    write_file(str(tmp_path / "model.safetensors"),
               {"m": torch.randn(4, 4).bfloat16(), "v": torch.randn(4), "t": torch.arange(4, dtype=torch.int64)})
    specs = [WeightSpec("m", (4, 4), MATRIX), WeightSpec("v", (4,), VECTOR), WeightSpec("t", (4,), TABLE)]
    source = SafetensorsSource(str(tmp_path))
    check_weights(specs, source)
    for compute in (torch.bfloat16, torch.float32):
        fetch = WeightFetcher(specs, source, compute, "cpu")
        assert fetch("m").dtype == compute and fetch("v").dtype == torch.float32 and fetch("t").dtype == torch.int32
    # widening a bfloat16 checkpoint to float32 is exact
    assert torch.equal(WeightFetcher(specs, source, torch.float32, "cpu")("m"), source.read("m", "cpu").float())


def test_sharded_folder_with_index(tmp_path):
    write_file(str(tmp_path / "s1.safetensors"), {"a": torch.ones(2)})
    write_file(str(tmp_path / "s2.safetensors"), {"b": torch.zeros(3)})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    source = SafetensorsSource(str(tmp_path))
    assert sorted(source.names()) == ["a", "b"] and source.shape("b") == (3,)


def test_random_source_answers_like_a_file():
    specs = collect_weight_specs(qwen2_plan(TINY["A"]["config"]))
    source = RandomSource(specs, seed=3)
    check_weights(specs, source)
    one = source.read("model.layers.0.self_attn.k_proj.weight", "cpu")
    assert one.dtype == torch.bfloat16 and tuple(one.shape) == (32, 64)
    assert torch.equal(one, RandomSource(specs, seed=3).read("model.layers.0.self_attn.k_proj.weight", "cpu"))
