"""Typed model configuration read from a checkpoint's ``config.json``.

The reference keeps the same information in two dataclasses
(``fastgen/model.py:12-40``) filled from the HF keys in
``fastgen/utils/loading.py:55-84``.  Here the parsing is a classmethod of
the typed record, every size comes from the file, and a missing or
unsupported key raises an error that names the key.
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Mapping, Optional


class ConfigError(ValueError):
    """A ``config.json`` that this engine cannot run, with the reason."""


def _require(config: Mapping[str, Any], key: str) -> Any:
    if key not in config or config[key] is None:
        raise ConfigError(f"config.json: required key {key!r} is missing")
    return config[key]


@dataclass(frozen=True)
class RopeArgs:
    """Rotary position encoding constants (``fastgen/model.py:12-20``).

    ``scaled`` switches the llama3 piecewise frequency scaling on; the four
    numbers after it are only meaningful then.
    """

    theta: float
    scaled: bool = False
    original_context: int = 0
    factor: float = 1.0
    low_freq_factor: float = 1.0
    high_freq_factor: float = 1.0

    @classmethod
    def from_hf_config(cls, config: Mapping[str, Any]) -> "RopeArgs":
        theta = float(_require(config, "rope_theta"))
        scaling = config.get("rope_scaling")
        if not scaling:
            return cls(theta=theta)
        kind = scaling.get("rope_type", scaling.get("type", "llama3"))
        if kind == "default":
            return cls(theta=theta)
        if kind != "llama3":
            raise ConfigError(
                f"config.json: rope_scaling.rope_type {kind!r} is not supported"
                " (supported: 'llama3', 'default')"
            )
        try:
            return cls(
                theta=theta,
                scaled=True,
                original_context=int(scaling["original_max_position_embeddings"]),
                factor=float(scaling["factor"]),
                low_freq_factor=float(scaling["low_freq_factor"]),
                high_freq_factor=float(scaling["high_freq_factor"]),
            )
        except KeyError as e:
            raise ConfigError(
                f"config.json: rope_scaling is missing required key {e.args[0]!r}"
            ) from None

    def to_hf_config(self) -> dict:
        out: dict = {"rope_theta": self.theta}
        if self.scaled:
            out["rope_scaling"] = {
                "rope_type": "llama3",
                "factor": self.factor,
                "low_freq_factor": self.low_freq_factor,
                "high_freq_factor": self.high_freq_factor,
                "original_max_position_embeddings": self.original_context,
            }
        else:
            out["rope_scaling"] = None
        return out


@dataclass(frozen=True)
class ModelArgs:
    """Hyper-parameters of a dense Llama decoder (``fastgen/model.py:23-40``).

    ``head_dim`` is ``dim // n_heads`` in the reference (``model.py:54``,
    ``forward.py:364``); a ``head_dim`` key in the file is accepted only
    when it says the same.  ``max_position`` caps a request's length; the
    reference never reads it and bounds length by its cache instead.
    """

    architecture: str
    dim: int
    ffn_dim: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    norm_eps: float
    vocab_size: int
    tie_embeddings: bool
    max_position: int
    rope: RopeArgs
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False)

    @classmethod
    def from_hf_config(cls, config: Mapping[str, Any]) -> "ModelArgs":
        # A multimodal wrapper nests the text model's keys
        # (fastgen/utils/loading.py:232,249).
        if "language_config" in config:
            inner = dict(config["language_config"])
            inner.setdefault("architectures", config.get("architectures"))
            config = inner
        archs = config.get("architectures") or [None]
        dim = int(_require(config, "hidden_size"))
        n_heads = int(_require(config, "num_attention_heads"))
        n_kv_heads = int(config.get("num_key_value_heads") or n_heads)
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ConfigError(
                f"config.json: num_attention_heads={n_heads} is not a multiple of"
                f" num_key_value_heads={n_kv_heads}"
            )
        if dim % n_heads:
            raise ConfigError(
                f"config.json: hidden_size={dim} is not a multiple of"
                f" num_attention_heads={n_heads}"
            )
        head_dim = dim // n_heads
        if config.get("head_dim") not in (None, head_dim):
            raise ConfigError(
                f"config.json: head_dim={config['head_dim']} differs from"
                f" hidden_size // num_attention_heads = {head_dim}; this"
                " architecture fixes it to the quotient"
            )
        for flag in ("attention_bias", "mlp_bias"):
            if config.get(flag):
                raise ConfigError(f"config.json: {flag}=true is not supported")
        act = config.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"config.json: hidden_act={act!r} is not supported")
        return cls(
            architecture=archs[0],
            dim=dim,
            ffn_dim=int(_require(config, "intermediate_size")),
            n_layers=int(_require(config, "num_hidden_layers")),
            n_heads=n_heads,
            n_kv_heads=n_kv_heads,
            head_dim=head_dim,
            norm_eps=float(_require(config, "rms_norm_eps")),
            vocab_size=int(_require(config, "vocab_size")),
            tie_embeddings=bool(config.get("tie_word_embeddings", False)),
            max_position=int(config.get("max_position_embeddings") or 0),
            rope=RopeArgs.from_hf_config(config),
            extra={k: config[k] for k in ("bos_token_id", "eos_token_id") if k in config},
        )

    def to_hf_config(self) -> dict:
        out = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.dim,
            "intermediate_size": self.ffn_dim,
            "num_hidden_layers": self.n_layers,
            "num_attention_heads": self.n_heads,
            "num_key_value_heads": self.n_kv_heads,
            "head_dim": self.head_dim,
            "hidden_act": "silu",
            "rms_norm_eps": self.norm_eps,
            "vocab_size": self.vocab_size,
            "tie_word_embeddings": self.tie_embeddings,
            "max_position_embeddings": self.max_position,
            "attention_bias": False,
            "mlp_bias": False,
        }
        out.update(self.rope.to_hf_config())
        out.update(self.extra)
        return out


def read_config_json(model_dir: str | Path) -> dict:
    """``config.json`` of a model folder as a dict (``loading.py:224-233``)."""
    path = Path(model_dir) / "config.json"
    if not path.is_file():
        raise ConfigError(f"{path} does not exist: not a model folder")
    with open(path) as f:
        return json.load(f)


def architecture_name(config: Mapping[str, Any]) -> Optional[str]:
    archs = config.get("architectures")
    if isinstance(archs, (list, tuple)) and len(archs) == 1:
        return archs[0]
    if isinstance(archs, str):
        return archs
    return None
