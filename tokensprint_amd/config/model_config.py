"""Typed Qwen3 configuration read from the checkpoint's own config.json keys.

The reference hard-codes its sizes in Python factories
(engine/models/qwen/_archs.py:92-125) and never parses config.json
(engine/generation/config.py:27,49-52 are commented out).  Here every size and
constant comes from the file; the fields carry the same meaning as the reference's
ModelConfig / AttentionConfig / FFNConfig (engine/models/_registry.py:12-38,
engine/nn/attention.py:75-84, engine/nn/layers.py:33-39).
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any


class ConfigError(ValueError):
    """config.json is missing a key, or holds a value this engine does not run."""


_REQUIRED = (
    "hidden_size", "num_hidden_layers", "num_attention_heads", "intermediate_size",
    "vocab_size", "rms_norm_eps", "rope_theta", "max_position_embeddings",
)


def read_config_json(model_dir) -> dict[str, Any]:
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise FileNotFoundError(f"no config.json in model folder {model_dir}")
    return json.loads(path.read_text())


def architecture_of(raw: dict[str, Any]) -> str:
    archs = raw.get("architectures")
    if not archs or not isinstance(archs, list):
        raise ConfigError("config.json has no 'architectures' list; cannot choose a model")
    return archs[0]


@dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense.  Field <- config.json key (reference field in brackets)."""

    hidden_size: int                 # hidden_size [model_dim]
    num_layers: int                  # num_hidden_layers [num_layers]
    num_heads: int                   # num_attention_heads [num_heads]
    num_kv_heads: int                # num_key_value_heads, absent -> num_heads [num_kv_heads]
    head_dim: int                    # head_dim, absent -> hidden_size // num_heads [head_dim]
    intermediate_size: int           # intermediate_size [inner_dim]
    vocab_size: int                  # vocab_size [vocab_dim]
    rms_norm_eps: float              # rms_norm_eps [norm_eps and qk_norm_eps]
    rope_theta: float                # rope_theta [rope_theta]
    max_position: int                # max_position_embeddings [max_seq_len]
    tie_word_embeddings: bool        # tie_word_embeddings, absent -> False [tie_weights]
    layer_windows: tuple[int | None, ...]  # per layer: None = all keys, W = last W keys
    eos_token_id: int | None = None  # eos_token_id
    bos_token_id: int | None = None  # bos_token_id
    stored_dtype: str | None = None  # torch_dtype / dtype
    architecture: str = "Qwen3ForCausalLM"
    raw: dict = field(default_factory=dict, compare=False, repr=False)

    @property
    def group_size(self) -> int:
        return self.num_heads // self.num_kv_heads

    @property
    def q_width(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.num_kv_heads * self.head_dim

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "Qwen3Config":
        missing = [k for k in _REQUIRED if k not in raw]
        if missing:
            raise ConfigError(f"config.json lacks required key(s): {', '.join(missing)}")

        def positive_int(key, value):
            if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
                raise ConfigError(f"config.json: '{key}' must be a positive integer, got {value!r}")
            return value

        hidden = positive_int("hidden_size", raw["hidden_size"])
        layers = positive_int("num_hidden_layers", raw["num_hidden_layers"])
        nq = positive_int("num_attention_heads", raw["num_attention_heads"])
        nkv = raw.get("num_key_value_heads")
        nkv = nq if nkv is None else positive_int("num_key_value_heads", nkv)
        hd = raw.get("head_dim")
        if hd is None:
            if hidden % nq:
                raise ConfigError(
                    f"config.json gives no head_dim and hidden_size={hidden} is not "
                    f"divisible by num_attention_heads={nq}")
            hd = hidden // nq
        hd = positive_int("head_dim", hd)
        if nq % nkv:
            raise ConfigError(
                f"num_attention_heads={nq} is not a multiple of num_key_value_heads={nkv}")
        if hd % 2:
            raise ConfigError(f"head_dim={hd} must be even for rotate-half position encoding")

        if raw.get("attention_bias", False):
            raise ConfigError("attention_bias=true: Qwen3 dense has no q/k/v bias")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act={act!r}: only 'silu' (SwiGLU) is built")
        if raw.get("rope_scaling") not in (None, {}):
            raise ConfigError(f"rope_scaling={raw['rope_scaling']!r} is not supported")
        eps = float(raw["rms_norm_eps"])
        theta = float(raw["rope_theta"])
        if not eps > 0.0 or not theta > 0.0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")

        windows = cls._layer_windows(raw, layers)

        eos = raw.get("eos_token_id")
        if isinstance(eos, list):
            eos = eos[0] if eos else None
        return cls(
            hidden_size=hidden, num_layers=layers, num_heads=nq, num_kv_heads=nkv,
            head_dim=hd,
            intermediate_size=positive_int("intermediate_size", raw["intermediate_size"]),
            vocab_size=positive_int("vocab_size", raw["vocab_size"]),
            rms_norm_eps=eps, rope_theta=theta,
            max_position=positive_int("max_position_embeddings", raw["max_position_embeddings"]),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            layer_windows=windows, eos_token_id=eos, bos_token_id=raw.get("bos_token_id"),
            stored_dtype=raw.get("torch_dtype", raw.get("dtype")),
            architecture=architecture_of(raw) if raw.get("architectures") else "Qwen3ForCausalLM",
            raw=dict(raw),
        )

    @staticmethod
    def _layer_windows(raw, layers) -> tuple[int | None, ...]:
        window = raw.get("sliding_window")
        types = raw.get("layer_types")
        if types is not None:
            if len(types) != layers:
                raise ConfigError(
                    f"layer_types has {len(types)} entries for {layers} layers")
            out = []
            for i, kind in enumerate(types):
                if kind == "full_attention":
                    out.append(None)
                elif kind == "sliding_attention":
                    if not isinstance(window, int) or window <= 0:
                        raise ConfigError(
                            f"layer {i} is 'sliding_attention' but sliding_window={window!r}")
                    out.append(window)
                else:
                    raise ConfigError(f"layer_types[{i}]={kind!r} is not a Qwen3 layer type")
            return tuple(out)
        if raw.get("use_sliding_window") and window is not None:
            if not isinstance(window, int) or window <= 0:
                raise ConfigError(f"sliding_window={window!r} must be a positive integer")
            first = raw.get("max_window_layers", layers)
            return tuple(window if i >= first else None for i in range(layers))
        return (None,) * layers

    @classmethod
    def from_model_dir(cls, model_dir) -> "Qwen3Config":
        return cls.from_dict(read_config_json(model_dir))

    def to_dict(self) -> dict[str, Any]:
        """config.json content that reads back to this configuration."""
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_layers,
            "num_attention_heads": self.num_heads,
            "num_key_value_heads": self.num_kv_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "attention_bias": False,
            "rope_scaling": None,
        }
        if any(w is not None for w in self.layer_windows):
            sizes = {w for w in self.layer_windows if w is not None}
            if len(sizes) != 1:
                raise ConfigError("config.json can name only one sliding_window size")
            out["sliding_window"] = sizes.pop()
            out["use_sliding_window"] = True
            out["layer_types"] = [
                "full_attention" if w is None else "sliding_attention"
                for w in self.layer_windows]
        else:
            out["sliding_window"] = None
            out["use_sliding_window"] = False
        if self.eos_token_id is not None:
            out["eos_token_id"] = self.eos_token_id
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        if self.stored_dtype is not None:
            out["torch_dtype"] = self.stored_dtype
        return out
