"""Typed configuration of the dense llama decoder, read from config.json keys.

Reference: `HfConfig` (crates/allpaca-safetensors/src/sidecar.rs:136-229) and the
use the loader makes of it (crates/allpaca-core/src/model.rs:7904-7940).  Unlike
the reference, keys that fix a tensor's shape have no silent default."""
from __future__ import annotations

from dataclasses import dataclass, field, asdict
from typing import Any, Mapping, Optional, Tuple


DEFAULT_MAX_POSITIONS = 2048   # `max_position_embeddings` of a llama config.json that does not name it


class ConfigError(ValueError):
    pass


def _need(d: Mapping[str, Any], key: str, kind=int):
    if key not in d or d[key] is None:
        raise ConfigError(f"config.json: required key {key!r} is missing")
    v = d[key]
    if kind is int and (isinstance(v, bool) or not isinstance(v, int) or v <= 0):
        raise ConfigError(f"config.json: {key!r} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class Llama3RopeScaling:
    """`rope_scaling` with rope_type "llama3".  The reference's llama path has
    no frequency scaling (ModelConfig carries rope_theta only,
    crates/allpaca-core/src/model.rs:181-274); the keys and their meaning are
    those of the published Llama-3.1 config.json."""
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int
    rope_type: str = "llama3"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Llama3RopeScaling":
        kind = d.get("rope_type") or d.get("type")
        if kind != "llama3":
            raise ConfigError(f"config.json: rope_scaling.rope_type {kind!r} is not supported (known: 'llama3')")
        try:
            out = cls(float(d["factor"]), float(d["low_freq_factor"]), float(d["high_freq_factor"]),
                      int(d["original_max_position_embeddings"]))
        except KeyError as e:
            raise ConfigError(f"config.json: rope_scaling lacks key {e.args[0]!r}") from None
        if out.factor <= 0 or out.high_freq_factor <= out.low_freq_factor or out.low_freq_factor <= 0:
            raise ConfigError("config.json: rope_scaling needs factor > 0 and high_freq_factor > low_freq_factor > 0")
        if out.original_max_position_embeddings <= 0:
            raise ConfigError("config.json: rope_scaling.original_max_position_embeddings must be positive")
        return out


@dataclass(frozen=True)
class LlamaConfig:
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    rms_norm_eps: float
    rope_theta: float
    rope_scaling: Optional[Llama3RopeScaling]
    max_position_embeddings: int
    tie_word_embeddings: bool
    hidden_act: str = "silu"
    architectures: Tuple[str, ...] = ("LlamaForCausalLM",)
    model_type: str = "llama"
    torch_dtype: Optional[str] = None

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "LlamaConfig":
        hidden = _need(d, "hidden_size")
        heads = _need(d, "num_attention_heads")
        # num_key_value_heads defaults to the head count and head_dim to
        # hidden/heads (model.rs:7920-7921, 366-372).
        kv_heads = d.get("num_key_value_heads") or heads
        head_dim = d.get("head_dim") or 0
        if not head_dim:
            if hidden % heads:
                raise ConfigError(f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads "
                                  f"{heads} and no head_dim is given")
            head_dim = hidden // heads
        act = str(d.get("hidden_act", "silu")).lower()
        if act not in ("silu", "swish", "silu_and_mul"):  # sidecar.rs:239-247
            raise ConfigError(f"config.json: unsupported hidden_act {d.get('hidden_act')!r} (llama uses silu)")
        for key in ("num_local_experts", "n_routed_experts", "num_experts", "num_experts_per_tok"):
            if d.get(key):  # sidecar.rs:232-237, model.rs:7908-7913
                raise ConfigError(f"config.json: {key} = {d[key]!r}: routed experts are not part of the dense llama decoder")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"config.json: {key} = true is not supported (the llama decoder has no biases)")
        # Newer config.json files carry theta and the scaling in one `rope_parameters` table
        # (HfRopeParameters, sidecar.rs:17-29); the top-level keys win where both are there.
        nested = d.get("rope_parameters") or {}
        theta = d.get("rope_theta")
        if theta is None:
            theta = nested.get("rope_theta", 10000.0)   # sidecar.rs:217-219
        scaling = d.get("rope_scaling")
        if not scaling and (nested.get("rope_type") or nested.get("type")) not in (None, "default"):
            scaling = nested
        if scaling and (scaling.get("rope_type") or scaling.get("type")) == "default":
            scaling = None
        cfg = cls(
            vocab_size=_need(d, "vocab_size"),
            hidden_size=hidden,
            num_hidden_layers=_need(d, "num_hidden_layers"),
            num_attention_heads=heads,
            num_key_value_heads=int(kv_heads),
            head_dim=int(head_dim),
            intermediate_size=_need(d, "intermediate_size"),
            rms_norm_eps=float(d.get("rms_norm_eps", 1e-5)),   # sidecar.rs:214-216
            rope_theta=float(theta),
            rope_scaling=Llama3RopeScaling.from_dict(scaling) if scaling else None,
            # positions the tables are made for unless the engine is set up for fewer; the reference does not read
            # the key (no tensor's shape hangs on it), so a file without it is taken with the published default
            max_position_embeddings=(_need(d, "max_position_embeddings") if d.get("max_position_embeddings") is not None
                                     else DEFAULT_MAX_POSITIONS),
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            hidden_act="silu",
            architectures=tuple(d.get("architectures") or ("LlamaForCausalLM",)),
            model_type=str(d.get("model_type") or "llama"),
            torch_dtype=d.get("torch_dtype"),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        if self.num_attention_heads % self.num_key_value_heads:  # kernels.rs:306-310
            raise ConfigError(f"config.json: num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: head_dim {self.head_dim} must be even (rotation pairs i, i + d/2)")
        if not (self.rms_norm_eps >= 0.0):
            raise ConfigError("config.json: rms_norm_eps must be >= 0")
        if not (self.rope_theta > 0.0):
            raise ConfigError("config.json: rope_theta must be > 0")

    def to_dict(self) -> dict:
        d = asdict(self)
        d["architectures"] = list(self.architectures)
        if self.rope_scaling is None:
            d["rope_scaling"] = None
        if d.get("torch_dtype") is None:
            d.pop("torch_dtype", None)
        return d
