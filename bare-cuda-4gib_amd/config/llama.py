"""Configuration of the Llama dense decoder.

Keys and defaults follow what the reference's converter reads from a
HuggingFace config (tools/convert/convert_weights.py:35-46):
``num_key_value_heads`` defaults to ``num_attention_heads``,
``max_position_embeddings`` to 2048, ``rope_theta`` to 10000.0,
``rms_norm_eps`` to 1e-5.  The reference always derives
``head_dim = hidden_size // num_attention_heads``; an explicit ``head_dim`` key
is honoured here as well.  The reference has no tie flag (it always requires
lm_head.weight, engine/src/model.cpp:365-366); ``tie_word_embeddings`` is read
so that a model without lm_head.weight can share the embedding table.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, Optional

from ..errors import ConfigError
from .base import ModelConfig, field_from_json
from .registry import Architecture, register_architecture


@dataclasses.dataclass
class LlamaConfig(ModelConfig):
    vocab_size: int = field_from_json("vocab_size")
    hidden_size: int = field_from_json("hidden_size")
    num_layers: int = field_from_json("num_hidden_layers")
    num_heads: int = field_from_json("num_attention_heads")
    intermediate_size: int = field_from_json("intermediate_size")
    num_kv_heads: int = field_from_json("num_key_value_heads", 0)
    head_dim: int = field_from_json("head_dim", 0)
    max_seq_len: int = field_from_json("max_position_embeddings", 2048)
    rope_theta: float = field_from_json("rope_theta", 10000.0)
    rms_norm_eps: float = field_from_json("rms_norm_eps", 1e-5)
    tie_word_embeddings: bool = field_from_json("tie_word_embeddings", False)
    hidden_act: str = field_from_json("hidden_act", "silu")
    attention_bias: bool = field_from_json("attention_bias", False)
    mlp_bias: bool = field_from_json("mlp_bias", False)
    rope_scaling: Optional[Dict[str, Any]] = field_from_json("rope_scaling", None)

    def derive(self, raw: Dict[str, Any]) -> None:
        if self.num_kv_heads == 0:
            self.num_kv_heads = self.num_heads
        if self.head_dim == 0:
            if self.num_heads <= 0 or self.hidden_size % self.num_heads:
                raise ConfigError(
                    f"config.json: hidden_size {self.hidden_size} is not a multiple of "
                    f"num_attention_heads {self.num_heads} and no head_dim is given")
            self.head_dim = self.hidden_size // self.num_heads

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "num_layers", "num_heads", "num_kv_heads",
                     "head_dim", "intermediate_size", "max_seq_len"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"config.json: {name} must be positive, got {getattr(self, name)}")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {self.num_heads} is not a multiple of "
                f"num_key_value_heads {self.num_kv_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even for rotary positions")
        if self.rope_theta <= 0:
            raise ConfigError(f"config.json: rope_theta must be positive, got {self.rope_theta}")
        if self.rms_norm_eps < 0:
            raise ConfigError(f"config.json: rms_norm_eps must not be negative, got {self.rms_norm_eps}")
        if self.hidden_act != "silu":
            raise ConfigError(f"config.json: hidden_act '{self.hidden_act}' is not supported (only 'silu')")
        if self.attention_bias or self.mlp_bias:
            raise ConfigError("config.json: attention_bias / mlp_bias are not supported (no biases)")
        if self.rope_scaling is not None:
            raise ConfigError("config.json: rope_scaling is not supported")

    def to_dict(self) -> Dict[str, Any]:
        out = super().to_dict()
        out["architectures"] = ["LlamaForCausalLM"]
        out["model_type"] = "llama"
        return out


def describe_llama(cfg: LlamaConfig):
    """The Llama layer stack as data (engine/src/model.cpp:526-615): L identical
    pre-norm blocks of grouped-query attention with rotary positions and a
    SwiGLU feed-forward, then a final RMSNorm and the output projection."""
    from ..engine.spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

    norm = {"eps": cfg.rms_norm_eps, "size": cfg.hidden_size}
    layers = []
    for i in range(cfg.num_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(
            block="prenorm",
            mixer=PartSpec("attention", dict(
                hidden_size=cfg.hidden_size, num_heads=cfg.num_heads,
                num_kv_heads=cfg.num_kv_heads, head_dim=cfg.head_dim, window=0,
                position=PartSpec("rotary", dict(theta=cfg.rope_theta, dim=cfg.head_dim))),
                prefix=p + "self_attn."),
            ffn=PartSpec("swiglu", dict(hidden_size=cfg.hidden_size,
                                        intermediate_size=cfg.intermediate_size),
                         prefix=p + "mlp."),
            mixer_norm=PartSpec("rmsnorm", dict(norm), prefix=p + "input_layernorm."),
            ffn_norm=PartSpec("rmsnorm", dict(norm), prefix=p + "post_attention_layernorm."),
        ))
    return ModelSpec(
        vocab_size=cfg.vocab_size,
        hidden_size=cfg.hidden_size,
        max_seq_len=cfg.max_seq_len,
        embedding=PartSpec("embedding", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size),
                           prefix="model.embed_tokens."),
        layers=layers,
        schedule=[ScheduleEntry(layer=i, cache=i, writes=True) for i in range(cfg.num_layers)],
        final_norm=PartSpec("rmsnorm", dict(norm), prefix="model.norm."),
        head=PartSpec("lm_head", dict(vocab_size=cfg.vocab_size, hidden_size=cfg.hidden_size,
                                      tied_to="model.embed_tokens.weight" if cfg.tie_word_embeddings else None),
                      prefix="lm_head."),
    )


LLAMA = register_architecture(Architecture(
    name="LlamaForCausalLM", model_type="llama",
    config_class=LlamaConfig, describe=describe_llama,
    ignored_tensors=("*.rotary_emb.inv_freq",)))      # a buffer some checkpoints carry; the angles are computed here
