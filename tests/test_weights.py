"""Weights: names on disk, one error that lists everything wrong, kept dtypes, random mode."""
import json
import os

import pytest
import torch

from helpers import TINY_A, TINY_B, make_weights, tensor_shapes, write_model_dir
from minivllm_amd.models import config_from_dict, expected_tensors, load_config
from minivllm_amd.weights import (DeviceTensors, DictSource, WeightError, check_tensors, open_model_folder,
                                  storage_dtype, write_model_folder)


@pytest.mark.parametrize("raw", [TINY_A, TINY_B])
def test_expected_names_are_the_checkpoint_names(raw):
    """The engine's name map against the names spelled out in the tests' own table."""
    arch, cfg = config_from_dict(dict(raw))
    exp = expected_tensors(arch, cfg)
    assert {k: tuple(v.shape) for k, v in exp.items()} == tensor_shapes(raw)
    assert ("lm_head.weight" in exp) == (not raw["tie_word_embeddings"])


def test_good_folder_passes_and_tied_head_copy_is_ignored(tmp_path):
    w = make_weights(TINY_A, 0)
    w["lm_head.weight"] = w["model.embed_tokens.weight"].clone()   # the reference skips it (qwen3.py:231-232)
    d = write_model_dir(str(tmp_path / "m"), TINY_A, w)
    arch, cfg = load_config(d)
    check_tensors(open_model_folder(d), expected_tensors(arch, cfg), arch.ignorable(cfg), d)


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    w = make_weights(TINY_B, 0)
    del w["model.layers.1.mlp.up_proj.weight"]
    del w["model.norm.weight"]
    w["model.layers.7.mlp.up_proj.weight"] = torch.zeros(2, 2)
    w["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(31)
    w["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(64, 95)
    w["model.layers.0.self_attn.o_proj.bias"] = torch.zeros(96, dtype=torch.int32)
    d = write_model_dir(str(tmp_path / "m"), TINY_B, w)
    arch, cfg = load_config(d)
    with pytest.raises(WeightError) as ei:
        check_tensors(open_model_folder(d), expected_tensors(arch, cfg), arch.ignorable(cfg), d)
    e = ei.value
    assert e.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert e.unexpected == ["model.layers.7.mlp.up_proj.weight"]
    assert ("model.layers.0.self_attn.q_norm.weight", (31,), (32,)) in e.wrong_shape
    assert ("model.layers.2.self_attn.k_proj.weight", (64, 95), (64, 96)) in e.wrong_shape
    assert e.wrong_type and e.wrong_type[0][0] == "model.layers.0.self_attn.o_proj.bias"
    text = str(e)
    for needle in ("missing tensors (2)", "unexpected tensors (1)", "wrong shapes (2)", "found [31], expected [32]",
                   "model.norm.weight", "model.layers.7.mlp.up_proj.weight"):
        assert needle in text


def test_untied_model_needs_its_head(tmp_path):
    w = make_weights(TINY_B, 0)
    del w["lm_head.weight"]
    arch, cfg = config_from_dict(dict(TINY_B))
    with pytest.raises(WeightError, match="lm_head.weight"):
        check_tensors(DictSource(w), expected_tensors(arch, cfg), arch.ignorable(cfg))


def test_kept_dtypes():
    assert storage_dtype(torch.zeros(1, dtype=torch.bfloat16)) == torch.bfloat16
    with pytest.raises(TypeError, match="float16"):                                  # never converted silently
        storage_dtype(torch.zeros(1, dtype=torch.float16))
    assert storage_dtype(torch.zeros(1, dtype=torch.float32)) == torch.float32      # 32-bit stays 32-bit
    assert storage_dtype(torch.zeros(1, dtype=torch.float64)) == torch.float32
    assert storage_dtype(torch.zeros(1, dtype=torch.int64)) == torch.int32           # integer tables
    src = DictSource({"a": torch.ones(3, dtype=torch.bfloat16), "b": torch.ones(3), "c": torch.arange(3)})
    dev = DeviceTensors(src, torch.device("cpu"))
    assert dev.get("a").dtype == torch.bfloat16 and dev.get("b").dtype == torch.float32
    assert dev.get("c").dtype == torch.int32
    first = dev.get("b")
    assert dev.get("b") is first                       # one object per name: tied tensors share memory
    assert first.data_ptr() != src.read("b").data_ptr()


@pytest.mark.parametrize("raw,stored", [(TINY_A, "float32"), (TINY_B, "bfloat16")])
def test_random_model_folder(tmp_path, raw, stored):
    arch, cfg = config_from_dict(dict(raw))
    d = write_model_folder(str(tmp_path / "rand"), cfg, seed=3, dtype=stored)
    assert sorted(os.listdir(d)) == ["config.json", "model.safetensors"]
    arch2, cfg2 = load_config(d)
    assert cfg2 == type(cfg).from_dict({**cfg.to_dict(), "torch_dtype": stored})
    src = open_model_folder(d)
    check_tensors(src, expected_tensors(arch2, cfg2), arch2.ignorable(cfg2), d)
    q = src.read("model.layers.0.self_attn.q_proj.weight")
    n = src.read("model.layers.0.input_layernorm.weight")
    assert q.dtype == getattr(torch, stored)
    assert abs(float(q.float().std()) - 0.02) < 0.004 and abs(float(q.float().mean())) < 0.004
    assert abs(float(n.float().mean()) - 1.0) < 0.02
    # the same seed gives the same tensors, another seed others; a tensor does not depend on the rest
    d2 = write_model_folder(str(tmp_path / "rand2"), cfg, seed=3, dtype=stored)
    d3 = write_model_folder(str(tmp_path / "rand3"), cfg, seed=4, dtype=stored)
    assert torch.equal(open_model_folder(d2).read("model.norm.weight"), src.read("model.norm.weight"))
    assert not torch.equal(open_model_folder(d3).read("model.norm.weight"), src.read("model.norm.weight"))


def test_float16_tensors_are_refused_not_converted(tmp_path):
    """A tensor stored in float16 is named in the one error; nothing is converted silently."""
    w = make_weights(TINY_A, 0, stored=torch.bfloat16)
    w["model.layers.1.mlp.down_proj.weight"] = w["model.layers.1.mlp.down_proj.weight"].to(torch.float16)
    w["model.norm.weight"] = w["model.norm.weight"].to(torch.float16)
    del w["model.layers.0.mlp.up_proj.weight"]
    d = write_model_dir(str(tmp_path / "m"), TINY_A, w)
    arch, cfg = load_config(d)
    with pytest.raises(WeightError) as ei:
        check_tensors(open_model_folder(d), expected_tensors(arch, cfg), arch.ignorable(cfg), d)
    e = ei.value
    assert e.unsupported_dtype == [("model.layers.1.mlp.down_proj.weight", "F16"), ("model.norm.weight", "F16")]
    assert e.missing == ["model.layers.0.mlp.up_proj.weight"]
    assert "unsupported dtype F16 (2 tensors" in str(e)
    with pytest.raises(TypeError, match="float16"):
        storage_dtype(torch.zeros(2, dtype=torch.float16))
    # the same through a dictionary of tensors
    with pytest.raises(WeightError, match="unsupported dtype F16"):
        check_tensors(DictSource({**make_weights(TINY_A, 0), "model.norm.weight": torch.ones(64, dtype=torch.float16)}),
                      expected_tensors(arch, cfg), arch.ignorable(cfg))
