"""Weights by tensor name: stored precisions, the one error that lists everything wrong, random folders.  CPU only."""

import json

import pytest
import torch
from safetensors.torch import save_file

import plain_llama as pl
from nanospec_amd.config import LlamaConfig
from nanospec_amd.parts import wanted_tensors
from nanospec_amd.weights import DictSource, SafetensorsSource, WeightError, check, random_tensors, write_model_folder
from tiny import TINY


def _wanted(name):
    spec = LlamaConfig.from_hf(TINY[name]["cfg"]).model_spec()
    return spec, {k: v[0] for k, v in wanted_tensors(spec).items()}


def test_names_and_shapes_are_the_checkpoints_own():
    """Tensor names of the reference (model/llama.py:3,168-171,190-192,203-204,214-216,262)."""
    spec, wanted = _wanted("B")
    assert wanted["model.embed_tokens.weight"] == (1000, 192)
    assert wanted["model.layers.2.self_attn.q_proj.weight"] == (6 * 32, 192)
    assert wanted["model.layers.2.self_attn.k_proj.weight"] == (32, 192)
    assert wanted["model.layers.0.self_attn.o_proj.weight"] == (192, 192)
    assert wanted["model.layers.1.mlp.gate_proj.weight"] == (512, 192)
    assert wanted["model.layers.1.mlp.down_proj.weight"] == (192, 512)
    assert wanted["model.layers.1.post_attention_layernorm.weight"] == (192,)
    assert wanted["model.norm.weight"] == (192,) and wanted["lm_head.weight"] == (1000, 192)
    assert len(wanted) == 3 + 3 * 9


def test_one_error_lists_missing_unexpected_and_wrong_shapes():
    spec, wanted = _wanted("A")
    tensors = {k: torch.zeros(v) for k, v in wanted.items() if k != "lm_head.weight"}
    check(DictSource(tensors), wanted, optional={"lm_head.weight"})  # tied: the head may be absent
    del tensors["model.norm.weight"]
    del tensors["model.layers.1.mlp.up_proj.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(16, 64)
    with pytest.raises(WeightError) as e:
        check(DictSource(tensors, "somewhere"), wanted, optional={"lm_head.weight"})
    err = e.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert err.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (16, 64), (32, 64))]
    text = str(err)
    for piece in ("somewhere", "missing tensors (2)", "unexpected tensors (1)", "is [16, 64], the model wants [32, 64]"):
        assert piece in text
    with pytest.raises(WeightError):  # an untied model must bring its head (reference: model/loader.py:63-64)
        check(DictSource({k: torch.zeros(v) for k, v in wanted.items() if k != "lm_head.weight"}), wanted)


def test_stored_precisions_are_kept(tmp_path):
    save_file({"a": torch.ones(2, 2, dtype=torch.bfloat16), "b": torch.ones(3, dtype=torch.float32),
               "c": torch.arange(4, dtype=torch.int64)}, str(tmp_path / "model.safetensors"))
    src = SafetensorsSource(tmp_path)
    assert src.get("a").dtype == torch.bfloat16 and src.get("b").dtype == torch.float32 and src.get("c").dtype == torch.int32
    assert src.shape("a") == (2, 2) and sorted(src.names()) == ["a", "b", "c"]
    with pytest.raises(FileNotFoundError):
        SafetensorsSource(tmp_path / "empty")


def test_random_weights_follow_the_law_and_the_seed(tmp_path):
    config = LlamaConfig.from_hf(TINY["B"]["cfg"])
    folder = write_model_folder(tmp_path / "m", config, seed=1)
    assert json.loads((folder / "config.json").read_text())["architectures"] == ["LlamaForCausalLM"]
    w = pl.read_safetensors(folder / "model.safetensors")  # read back by the plain implementation's own reader
    spec, wanted = _wanted("B")
    assert set(w) == set(wanted)
    lin = w["model.layers.0.mlp.gate_proj.weight"]
    assert abs(float(lin.std()) - 0.02) < 2e-3 and abs(float(lin.mean())) < 1e-3
    norm = w["model.layers.0.input_layernorm.weight"]
    assert abs(float(norm.mean()) - 1.0) < 0.01 and 0.005 < float(norm.std()) < 0.04
    again = random_tensors(wanted_tensors(spec), seed=1)
    assert all(torch.equal(w[k], again[k]) for k in w)
    other = random_tensors(wanted_tensors(spec), seed=2)
    assert not torch.equal(w["model.norm.weight"], other["model.norm.weight"])
    # tied configuration: the head is left out of the file
    tied = write_model_folder(tmp_path / "t", LlamaConfig.from_hf(TINY["A"]["cfg"]), seed=0)
    assert "lm_head.weight" not in pl.read_safetensors(tied / "model.safetensors")
