"""Typed configuration of the Llama dense decoder, read from config.json.

Counterpart of `Config` / `parse_config` in the reference
(src/arch/llama.rs:11-22, :104-126): required keys raise, optional ones take the
reference's defaults (`num_key_value_heads` = heads, `head_dim` = hidden/heads,
`rms_norm_eps` = 1e-5, `rope_theta` = 10000: llama.rs:118-123).  The reference
reads GGUF metadata; the keys here are the ones a Llama config.json holds.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict
from typing import Any, Dict, Optional, Tuple

from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec


class ConfigError(ValueError):
    pass


@dataclass(frozen=True)
class RopeScaling:
    """`rope_scaling` of type "llama3": wavelengths longer than
    original/low_freq_factor are stretched by `factor`, those shorter than
    original/high_freq_factor are kept, the band between is blended."""
    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    @classmethod
    def from_dict(cls, d: Optional[Dict[str, Any]]) -> Optional["RopeScaling"]:
        if d is None:
            return None
        kind = d.get("rope_type", d.get("type"))
        if kind in (None, "default"):
            return None
        if kind != "llama3":
            raise ConfigError(f"unsupported rope_scaling type: {kind!r} (supported: llama3)")
        try:
            return cls("llama3", float(d["factor"]), float(d["low_freq_factor"]),
                       float(d["high_freq_factor"]), int(d["original_max_position_embeddings"]))
        except KeyError as e:
            raise ConfigError(f"missing config key: rope_scaling.{e.args[0]}") from None


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    max_position_embeddings: int
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    bos_token_id: Optional[int] = None
    eos_token_id: Tuple[int, ...] = ()
    torch_dtype: str = "bfloat16"
    architecture: str = "LlamaForCausalLM"

    REQUIRED = ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                "num_attention_heads", "max_position_embeddings")

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        for key in cls.REQUIRED:
            if d.get(key) is None:
                raise ConfigError(f"missing config key: {key}")
        heads = int(d["num_attention_heads"])
        hidden = int(d["hidden_size"])
        kv_heads = d.get("num_key_value_heads")
        kv_heads = heads if kv_heads is None else int(kv_heads)
        head_dim = d.get("head_dim")
        if head_dim is None:
            if heads <= 0 or hidden % heads:
                raise ConfigError(f"hidden_size {hidden} is no multiple of num_attention_heads {heads} and head_dim is not given")
            head_dim = hidden // heads
        if d.get("hidden_act", "silu") != "silu":
            raise ConfigError(f"unsupported hidden_act: {d['hidden_act']!r} (supported: silu)")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"unsupported: {key}=true")
        eos = d.get("eos_token_id")
        eos = () if eos is None else (tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),))
        archs = d.get("architectures") or ["LlamaForCausalLM"]
        cfg = cls(
            vocab_size=int(d["vocab_size"]), hidden_size=hidden,
            intermediate_size=int(d["intermediate_size"]),
            num_hidden_layers=int(d["num_hidden_layers"]),
            num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=int(head_dim),
            max_position_embeddings=int(d["max_position_embeddings"]),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-5)),
            rope_theta=float(d.get("rope_theta", 10000.0)),
            rope_scaling=RopeScaling.from_dict(d.get("rope_scaling")),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            bos_token_id=d.get("bos_token_id"), eos_token_id=eos,
            torch_dtype=str(d.get("torch_dtype", d.get("dtype", "bfloat16"))),
            architecture=str(archs[0]))
        cfg.validate()
        return cfg

    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"num_attention_heads {self.num_attention_heads} is no multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"head_dim must be even for rotary pairs, got {self.head_dim}")
        if not self.rms_norm_eps > 0:
            raise ConfigError(f"rms_norm_eps must be positive, got {self.rms_norm_eps}")

    def to_dict(self) -> Dict[str, Any]:
        d = asdict(self)
        d["architectures"] = [d.pop("architecture")]
        d["model_type"] = "llama"
        d["hidden_act"] = "silu"
        d["attention_bias"] = False
        d["mlp_bias"] = False
        d["eos_token_id"] = list(self.eos_token_id) if len(self.eos_token_id) != 1 else self.eos_token_id[0]
        if not self.eos_token_id:
            d["eos_token_id"] = None
        if self.rope_scaling is None:
            d["rope_scaling"] = None
        return d

    # -- what the engine builds from ---------------------------------------
    def model_spec(self) -> ModelSpec:
        """Llama as parts: every layer is pre-norm {RMSNorm, rotary GQA attention},
        {RMSNorm, SwiGLU}; layers run once each, in order (src/arch/llama.rs:151-171)."""
        rope = {"kind": "rope", "head_dim": self.head_dim, "rotary_dim": self.head_dim,
                "theta": self.rope_theta, "layout": "split_half",
                "scaling": None if self.rope_scaling is None else asdict(self.rope_scaling)}
        layers = []
        for i in range(self.num_hidden_layers):
            p = f"model.layers.{i}"
            layers.append(LayerSpec(
                block="prenorm",
                mixer=PartSpec("attention", f"{p}.self_attn", {
                    "hidden_size": self.hidden_size, "num_heads": self.num_attention_heads,
                    "num_kv_heads": self.num_key_value_heads, "head_dim": self.head_dim,
                    "window": None, "position": rope}),
                feed_forward=PartSpec("swiglu", f"{p}.mlp", {
                    "hidden_size": self.hidden_size, "intermediate_size": self.intermediate_size}),
                mixer_norm=PartSpec("rmsnorm", f"{p}.input_layernorm",
                                    {"size": self.hidden_size, "eps": self.rms_norm_eps}),
                feed_forward_norm=PartSpec("rmsnorm", f"{p}.post_attention_layernorm",
                                           {"size": self.hidden_size, "eps": self.rms_norm_eps})))
        return ModelSpec(
            hidden_size=self.hidden_size, vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            layers=layers, schedule=[RunSpec(i) for i in range(self.num_hidden_layers)],
            final_norm=PartSpec("rmsnorm", "model.norm", {"size": self.hidden_size, "eps": self.rms_norm_eps}),
            embedding_name="model.embed_tokens.weight",
            head_name=None if self.tie_word_embeddings else "lm_head.weight",
            # older files store the rotation's frequency table; files of tied models may repeat the token table
            ignorable_tensors=("*.rotary_emb.inv_freq",) + (("lm_head.weight",) if self.tie_word_embeddings else ()))
