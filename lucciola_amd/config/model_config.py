"""Typed configuration of the Qwen3 dense decoder, read from the keys of its config.json.

The reference reads seven integers (src/qwen.cc:50-58: hidden_size, intermediate_size,
num_attention_heads, num_key_value_heads, head_dim, num_hidden_layers, vocab_size) and keeps
rope_theta (src/qwen.cc:636), the norms' eps (src/qwen.cc:588) and the end-of-sequence ids
(src/async_engine.cc:143) as literals.  Here every one of them is a field read from the file;
defaults follow the reference where it has one (num_key_value_heads = num_attention_heads,
head_dim = hidden_size / num_attention_heads: src/qwen.cc:53-56).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple


class ConfigError(ValueError):
    pass


def _require_int(data: Dict[str, Any], key: str, default: Optional[int] = None) -> int:
    if key not in data or data[key] is None:
        if default is None:
            raise ConfigError(f"config.json: required key '{key}' is missing")
        return default
    value = data[key]
    if isinstance(value, bool) or not isinstance(value, int):
        raise ConfigError(f"config.json: '{key}' must be an integer, got {value!r}")
    return value


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1000000.0
    tie_word_embeddings: bool = False
    max_position_embeddings: int = 40960
    hidden_act: str = "silu"
    initializer_range: float = 0.02
    # sliding_window applies to the layers whose entry in layer_types is "sliding_attention"
    sliding_window: Optional[int] = None
    layer_types: Tuple[str, ...] = ()
    eos_token_ids: Tuple[int, ...] = ()
    architectures: Tuple[str, ...] = ("Qwen3ForCausalLM",)

    # ------------------------------------------------------------------ reading
    @staticmethod
    def from_dict(data: Dict[str, Any]) -> "Qwen3Config":
        hidden = _require_int(data, "hidden_size")
        heads = _require_int(data, "num_attention_heads")
        layers = _require_int(data, "num_hidden_layers")
        kv_heads = _require_int(data, "num_key_value_heads", heads)
        if heads <= 0:
            raise ConfigError("config.json: num_attention_heads must be positive")
        head_dim = _require_int(data, "head_dim", hidden // heads)

        if data.get("rope_scaling") not in (None, {}):
            scaling = data["rope_scaling"]
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if kind not in (None, "default"):
                raise ConfigError(f"config.json: rope_scaling {scaling!r} is not supported "
                                  f"(only plain rotary embedding)")
        if data.get("attention_bias", False):
            raise ConfigError("config.json: attention_bias=true is not supported "
                              "(the Qwen3 dense decoder has no projection biases)")

        window = data.get("sliding_window")
        use_window = bool(data.get("use_sliding_window", False))
        layer_types = data.get("layer_types")
        if layer_types is None:
            # layers from max_window_layers on slide, when sliding is switched on at all
            first_sliding = _require_int(data, "max_window_layers", layers)
            layer_types = ["sliding_attention" if (use_window and window is not None
                                                   and i >= first_sliding)
                           else "full_attention" for i in range(layers)]
        layer_types = tuple(str(t) for t in layer_types)
        if not any(t == "sliding_attention" for t in layer_types):
            window = None

        eos = data.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (int(eos),)

        cfg = Qwen3Config(
            vocab_size=_require_int(data, "vocab_size"),
            hidden_size=hidden,
            intermediate_size=_require_int(data, "intermediate_size"),
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            rms_norm_eps=float(data.get("rms_norm_eps", 1e-6)),
            rope_theta=float(data.get("rope_theta", 1000000.0)),
            tie_word_embeddings=bool(data.get("tie_word_embeddings", False)),
            max_position_embeddings=_require_int(data, "max_position_embeddings", 40960),
            hidden_act=str(data.get("hidden_act", "silu")),
            initializer_range=float(data.get("initializer_range", 0.02)),
            sliding_window=None if window is None else int(window),
            layer_types=layer_types,
            eos_token_ids=eos_ids,
            architectures=tuple(data.get("architectures") or ("Qwen3ForCausalLM",)),
        )
        cfg.validate()
        return cfg

    @staticmethod
    def from_folder(folder: str) -> "Qwen3Config":
        return Qwen3Config.from_dict(read_config_json(folder))

    # ------------------------------------------------------------------ checking
    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim",
                    "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config.json: '{key}' must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"config.json: num_attention_heads ({self.num_attention_heads}) must be a "
                f"multiple of num_key_value_heads ({self.num_key_value_heads})")
        if self.head_dim % 2 != 0:
            raise ConfigError(f"config.json: head_dim ({self.head_dim}) must be even for the "
                              f"half-split rotary embedding")
        if not self.rms_norm_eps > 0:
            raise ConfigError("config.json: rms_norm_eps must be positive")
        if not self.rope_theta > 0:
            raise ConfigError("config.json: rope_theta must be positive")
        if self.hidden_act != "silu":
            raise ConfigError(f"config.json: hidden_act '{self.hidden_act}' is not supported "
                              f"(the gated feed-forward uses silu)")
        if len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError(f"config.json: layer_types has {len(self.layer_types)} entries "
                              f"for {self.num_hidden_layers} layers")
        for t in self.layer_types:
            if t not in ("full_attention", "sliding_attention"):
                raise ConfigError(f"config.json: unknown layer type '{t}'")
        if any(t == "sliding_attention" for t in self.layer_types):
            if self.sliding_window is None or self.sliding_window <= 0:
                raise ConfigError("config.json: sliding_attention layers need a positive "
                                  "sliding_window")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architectures": list(self.architectures),
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "max_position_embeddings": self.max_position_embeddings,
            "hidden_act": self.hidden_act,
            "initializer_range": self.initializer_range,
            "attention_bias": False,
        }
        if self.sliding_window is not None:
            out["sliding_window"] = self.sliding_window
            out["use_sliding_window"] = True
            out["layer_types"] = list(self.layer_types)
        if self.eos_token_ids:
            out["eos_token_id"] = (self.eos_token_ids[0] if len(self.eos_token_ids) == 1
                                   else list(self.eos_token_ids))
        return out


def read_config_json(folder: str) -> Dict[str, Any]:
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in model folder '{folder}'")
    with open(path, "r", encoding="utf-8") as fh:
        try:
            data = json.load(fh)
        except json.JSONDecodeError as exc:
            raise ConfigError(f"{path}: not valid JSON ({exc})") from exc
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return data
