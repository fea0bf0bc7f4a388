"""The Llama 3 dense decoder's configuration, read from its own config.json keys.

Keys, defaults and refusals follow ved1beta/nanospec model/llama.py:22-78.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

from .registry import register_architecture
from .spec import AttentionSpec, LayerCall, ModelSpec, PreNormBlockSpec, RMSNormSpec, RopeSpec, SwiGLUSpec

_LLAMA3_KEYS = ("factor", "low_freq_factor", "high_freq_factor", "original_max_position_embeddings")


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    max_position_embeddings: int
    rope_scaling: dict | None = None  # llama3 parameters, None for unscaled frequencies
    tie_word_embeddings: bool = False
    bos_token_id: int | None = None
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)

    architecture = "LlamaForCausalLM"

    @classmethod
    def from_hf(cls, cfg: dict, generation_cfg: dict | None = None) -> "LlamaConfig":
        """config.json (and generation_config.json, whose ``eos_token_id`` wins) -> LlamaConfig.

        Reference: model/llama.py:39-78.  Accepts ``rope_theta`` + ``rope_scaling`` as well as the
        newer ``rope_parameters`` dictionary, and ``rope_type`` as well as ``type``.  Refuses
        another ``model_type``, biased projections and rope kinds other than default / llama3."""
        if cfg.get("model_type") != "llama":
            raise ValueError(f"not a llama configuration: model_type={cfg.get('model_type')!r}")
        if cfg.get("attention_bias") or cfg.get("mlp_bias"):
            raise ValueError("llama configurations with biased projections are not supported")
        rope = dict(cfg.get("rope_parameters") or cfg.get("rope_scaling") or {})
        theta = float(rope.pop("rope_theta", cfg.get("rope_theta", 10000.0)))
        kind = rope.pop("rope_type", rope.pop("type", "default"))
        if kind == "default":
            scaling = None
        elif kind == "llama3":
            missing = [k for k in _LLAMA3_KEYS if k not in rope]
            if missing:
                raise KeyError(f"llama3 rope scaling lacks {missing}")
            scaling = {k: rope[k] for k in _LLAMA3_KEYS}
        else:
            raise ValueError(f"unsupported rope_type {kind!r} (supported: 'default', 'llama3')")
        heads = cfg["num_attention_heads"]
        eos = cfg.get("eos_token_id")
        if generation_cfg and generation_cfg.get("eos_token_id") is not None:
            eos = generation_cfg["eos_token_id"]
        if eos is None:
            eos_ids: tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)
        out = cls(
            vocab_size=cfg["vocab_size"],
            hidden_size=cfg["hidden_size"],
            intermediate_size=cfg["intermediate_size"],
            num_hidden_layers=cfg["num_hidden_layers"],
            num_attention_heads=heads,
            num_key_value_heads=cfg.get("num_key_value_heads", heads),
            head_dim=cfg.get("head_dim") or cfg["hidden_size"] // heads,
            rms_norm_eps=cfg.get("rms_norm_eps", 1e-5),
            rope_theta=theta,
            max_position_embeddings=cfg["max_position_embeddings"],
            rope_scaling=scaling,
            tie_word_embeddings=bool(cfg.get("tie_word_embeddings", False)),
            bos_token_id=cfg.get("bos_token_id"),
            eos_token_ids=eos_ids,
        )
        out.validate()
        return out

    def validate(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads:
            raise ValueError(
                f"num_attention_heads={self.num_attention_heads} is not a multiple of "
                f"num_key_value_heads={self.num_key_value_heads}"
            )
        if self.head_dim % 2:
            raise ValueError(f"head_dim={self.head_dim} must be even for the rotary encoding")
        for name in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "head_dim"):
            if getattr(self, name) <= 0:
                raise ValueError(f"{name} must be positive, got {getattr(self, name)}")

    def to_hf(self) -> dict:
        """The config.json this configuration is read back from."""
        out = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "mlp_bias": False,
        }
        if self.rope_scaling is not None:
            out["rope_scaling"] = {"rope_type": "llama3", **self.rope_scaling}
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return out

    def model_spec(self) -> ModelSpec:
        """The decoder as parts (reference model/llama.py:161-266): every layer is a pre-norm block of
        grouped-query attention with rotary positions and a SwiGLU feed-forward; tensor names are
        the checkpoint's own (model/llama.py:3)."""
        scaling = None
        if self.rope_scaling is not None:
            s = self.rope_scaling
            scaling = (float(s["factor"]), float(s["low_freq_factor"]), float(s["high_freq_factor"]),
                       int(s["original_max_position_embeddings"]))
        rope = RopeSpec(rotary_dim=self.head_dim, theta=self.rope_theta, scaling=scaling,
                        max_positions=self.max_position_embeddings)
        norm = RMSNormSpec(dim=self.hidden_size, eps=self.rms_norm_eps)
        attn = AttentionSpec(hidden=self.hidden_size, heads=self.num_attention_heads, kv_heads=self.num_key_value_heads,
                             head_dim=self.head_dim, position=rope, softmax_scale=1.0 / math.sqrt(self.head_dim))
        ffn = SwiGLUSpec(hidden=self.hidden_size, intermediate=self.intermediate_size)
        layers = tuple(
            PreNormBlockSpec(prefix=f"model.layers.{i}.", mixer_norm=norm, mixer=attn, ffn_norm=norm, ffn=ffn,
                             mixer_norm_name="input_layernorm.weight", mixer_prefix="self_attn.",
                             ffn_norm_name="post_attention_layernorm.weight", ffn_prefix="mlp.")
            for i in range(self.num_hidden_layers)
        )
        return ModelSpec(
            vocab_size=self.vocab_size,
            hidden=self.hidden_size,
            embed_name="model.embed_tokens.weight",
            layers=layers,
            run_order=tuple(LayerCall(i) for i in range(self.num_hidden_layers)),
            final_norm=norm,
            final_norm_name="model.norm.weight",
            head_name="lm_head.weight",
            tie_head=self.tie_word_embeddings,
            eos_token_ids=self.eos_token_ids,
        )


def _build(cfg: dict, generation_cfg: dict | None):
    config = LlamaConfig.from_hf(cfg, generation_cfg)
    return config, config.model_spec()


register_architecture("LlamaForCausalLM", _build, model_type="llama")
