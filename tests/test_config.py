"""Typed configuration, registry and the model spec built from config.json keys.  CPU only."""

import json

import pytest

from nanospec_amd.config import LlamaConfig, architectures, load_config, register_architecture, resolve
from nanospec_amd.config.spec import LayerCall, ModelSpec, RMSNormSpec
from tiny import TINY


def test_llama_keys_and_defaults():
    """Defaults of the reference (model/llama.py:57-77): kv heads = heads, head_dim = hidden // heads, eps 1e-5,
    theta 10000, untied head."""
    raw = dict(model_type="llama", vocab_size=50, hidden_size=48, intermediate_size=100, num_hidden_layers=2,
               num_attention_heads=6, max_position_embeddings=64)
    c = LlamaConfig.from_hf(raw)
    assert (c.num_key_value_heads, c.head_dim, c.rms_norm_eps, c.rope_theta) == (6, 8, 1e-5, 10000.0)
    assert c.rope_scaling is None and c.tie_word_embeddings is False and c.eos_token_ids == ()
    c = LlamaConfig.from_hf(dict(raw, head_dim=None))  # a falsy head_dim falls back, model/llama.py:70
    assert c.head_dim == 8


def test_rope_spellings_and_eos():
    """Old (rope_theta + rope_scaling with 'type') and new (rope_parameters with 'rope_type') spellings parse alike
    (model/llama.py:46-55); generation_config's eos wins and a list becomes a tuple (:58-61)."""
    base = dict(TINY["B"]["cfg"])
    scaling = dict(base.pop("rope_scaling"))
    theta = base.pop("rope_theta")
    scaling.pop("rope_type")
    old = LlamaConfig.from_hf(dict(base, rope_theta=theta, rope_scaling=dict(type="llama3", **scaling), eos_token_id=7))
    new = LlamaConfig.from_hf(dict(base, rope_parameters=dict(rope_type="llama3", rope_theta=theta, **scaling)), {"eos_token_id": [3, 4]})
    assert old.rope_scaling == new.rope_scaling and old.rope_theta == new.rope_theta == 500000.0
    assert old.eos_token_ids == (7,) and new.eos_token_ids == (3, 4)


@pytest.mark.parametrize("bad, exc", [
    (dict(model_type="mistral"), ValueError),
    (dict(attention_bias=True), ValueError),
    (dict(mlp_bias=True), ValueError),
    (dict(rope_scaling=dict(rope_type="yarn", factor=2.0)), ValueError),
    (dict(rope_scaling=dict(rope_type="llama3", factor=2.0)), KeyError),
    (dict(num_key_value_heads=3), ValueError),
])
def test_refusals(bad, exc):
    with pytest.raises(exc):
        LlamaConfig.from_hf(dict(TINY["A"]["cfg"], **bad))


def test_missing_required_key():
    cfg = dict(TINY["A"]["cfg"])
    del cfg["max_position_embeddings"]
    with pytest.raises(KeyError):
        LlamaConfig.from_hf(cfg)


def test_registry_by_name_and_model_type(tmp_path):
    assert "LlamaForCausalLM" in architectures()
    config, spec = resolve(dict(TINY["A"]["cfg"]))
    assert isinstance(config, LlamaConfig) and len(spec.layers) == 2
    no_arch = {k: v for k, v in TINY["A"]["cfg"].items() if k != "architectures"}
    assert resolve(no_arch)[0] == config  # falls back to model_type
    with pytest.raises(ValueError, match="unknown architecture"):
        resolve(dict(TINY["A"]["cfg"], architectures=["GPT2LMHeadModel"]))
    (tmp_path / "config.json").write_text(json.dumps(TINY["B"]["cfg"]))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": 9}))
    assert load_config(tmp_path)[0].eos_token_ids == (9,)
    with pytest.raises(FileNotFoundError):
        load_config(tmp_path / "nowhere")


def test_register_another_architecture():
    def build(cfg, gen):
        c = LlamaConfig.from_hf(dict(cfg, model_type="llama"), gen)
        return c, c.model_spec()

    register_architecture("ToyForCausalLM", build, model_type="toy")
    config, spec = resolve(dict(TINY["A"]["cfg"], architectures=["ToyForCausalLM"], model_type="toy"))
    assert spec.vocab_size == 256


def test_model_spec_carries_every_size_of_the_config():
    for name in TINY:
        c = LlamaConfig.from_hf(TINY[name]["cfg"])
        spec = c.model_spec()
        assert (spec.vocab_size, spec.hidden, len(spec.layers)) == (c.vocab_size, c.hidden_size, c.num_hidden_layers)
        assert [call.layer for call in spec.run_order] == list(range(c.num_hidden_layers))
        for i, layer in enumerate(spec.layers):
            assert layer.prefix == f"model.layers.{i}."
            a, f = layer.mixer, layer.ffn
            assert (a.heads, a.kv_heads, a.head_dim, a.window) == (c.num_attention_heads, c.num_key_value_heads, c.head_dim, 0)
            assert a.softmax_scale == pytest.approx(c.head_dim ** -0.5)
            assert (a.position.theta, a.position.rotary_dim, a.position.max_positions) == (c.rope_theta, c.head_dim, c.max_position_embeddings)
            assert (f.hidden, f.intermediate) == (c.hidden_size, c.intermediate_size)
            assert layer.mixer_norm.eps == layer.ffn_norm.eps == c.rms_norm_eps
        assert spec.tie_head == c.tie_word_embeddings
        assert LlamaConfig.from_hf(c.to_hf()) == c  # config.json round trip


def test_run_order_is_checked():
    norm = RMSNormSpec(8, 1e-5)
    kw = dict(vocab_size=4, hidden=8, embed_name="e", layers=(object(),), final_norm=norm, final_norm_name="n", head_name="h", tie_head=True)
    ModelSpec(run_order=(LayerCall(0), LayerCall(0), LayerCall(0, cache_from=0)), **kw)  # a layer twice, a borrowed cache
    with pytest.raises(ValueError):
        ModelSpec(run_order=(LayerCall(1),), **kw)
    with pytest.raises(ValueError):
        ModelSpec(run_order=(LayerCall(0, cache_from=0),), **kw)  # not an earlier entry
    with pytest.raises(ValueError):
        ModelSpec(run_order=(LayerCall(0), LayerCall(0, cache_from=0), LayerCall(0, cache_from=1)), **kw)  # borrows from a borrower
