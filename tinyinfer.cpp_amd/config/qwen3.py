"""Typed configuration of the Qwen3 dense decoder.

The reference reads nine hyper-parameters from GGUF keys into `Qwen3Config`
(/root/reference/src/model.h:11-21, src/model.cpp:32-47) and refuses a model
whose required sizes are zero.  Here the same fields come from the
architecture's `config.json`; keys the reference has no counterpart for
(untied head, a sliding window on some layers) are read too, and options that
would change the math but are not served (attention bias, rope scaling, another
activation) are refused by name instead of being ignored.
"""
from __future__ import annotations

from dataclasses import dataclass, field, asdict
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, take

FULL = "full_attention"
SLIDING = "sliding_attention"


@dataclass(frozen=True)
class Qwen3Config:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float
    rope_theta: float
    # None: decided by whether the weights hold `lm_head.weight`
    tie_word_embeddings: Optional[bool]
    # one entry per layer: FULL or SLIDING
    layer_types: Tuple[str, ...]
    # tokens a SLIDING layer looks back over, itself included; None if no layer slides
    sliding_window: Optional[int]
    max_position_embeddings: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    architecture: str = "Qwen3ForCausalLM"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen3Config":
        n_layer = take(d, "num_hidden_layers", int)
        hidden = take(d, "hidden_size", int)
        heads = take(d, "num_attention_heads", int)
        kv_heads = take(d, "num_key_value_heads", int, heads)
        if heads <= 0:
            raise ConfigError("config.json: 'num_attention_heads' must be positive")
        if "head_dim" in d and d["head_dim"] is not None:
            head_dim = take(d, "head_dim", int)
        else:
            if hidden % heads:
                raise ConfigError(
                    "config.json: 'head_dim' is absent and 'hidden_size' "
                    f"({hidden}) is not a multiple of 'num_attention_heads' ({heads})")
            head_dim = hidden // heads

        act = take(d, "hidden_act", str, "silu")
        if act != "silu":
            raise ConfigError(f"config.json: 'hidden_act' = {act!r} is not served (only 'silu')")
        if take(d, "attention_bias", bool, False):
            raise ConfigError("config.json: 'attention_bias' = true is not served "
                              "(the projections carry no bias)")
        scaling = d.get("rope_scaling")
        if scaling is not None:
            kind = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if kind != "default":
                raise ConfigError(f"config.json: 'rope_scaling' = {scaling!r} is not served")

        window = take(d, "sliding_window", int, None)
        use_window = take(d, "use_sliding_window", bool, False)
        types = d.get("layer_types")
        if types is not None:
            if not isinstance(types, (list, tuple)) or len(types) != n_layer:
                raise ConfigError("config.json: 'layer_types' must list one entry per layer "
                                  f"({n_layer}), got {types!r}")
            for t in types:
                if t not in (FULL, SLIDING):
                    raise ConfigError(f"config.json: 'layer_types' entry {t!r} is not served")
            layer_types = tuple(types)
        elif use_window and window is not None:
            first = take(d, "max_window_layers", int, n_layer)
            layer_types = tuple(SLIDING if i >= first else FULL for i in range(n_layer))
        else:
            layer_types = tuple(FULL for _ in range(n_layer))
        if SLIDING in layer_types:
            if window is None:
                raise ConfigError("config.json: a layer slides but 'sliding_window' is absent")
        else:
            window = None

        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, (list, tuple)):
            eos_ids = tuple(int(e) for e in eos)
        else:
            eos_ids = (take(d, "eos_token_id", int),)

        archs = d.get("architectures")
        arch = archs[0] if isinstance(archs, (list, tuple)) and archs else "Qwen3ForCausalLM"

        tie = d.get("tie_word_embeddings")
        if tie is not None and not isinstance(tie, bool):
            raise ConfigError(f"config.json: 'tie_word_embeddings' must be true or false, got {tie!r}")

        cfg = cls(
            vocab_size=take(d, "vocab_size", int),
            hidden_size=hidden,
            intermediate_size=take(d, "intermediate_size", int),
            num_hidden_layers=n_layer,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            # defaults of the reference's loader: src/model.cpp:39-40
            rms_norm_eps=take(d, "rms_norm_eps", float, 1e-6),
            rope_theta=take(d, "rope_theta", float, 1000000.0),
            tie_word_embeddings=tie,
            layer_types=layer_types,
            sliding_window=window,
            max_position_embeddings=take(d, "max_position_embeddings", int, None),
            eos_token_ids=eos_ids,
            architecture=arch,
        )
        cfg.validate()
        return cfg

    # --------------------------------------------------------------- validation
    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"config.json: '{key}' must be positive, got {getattr(self, key)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"config.json: 'num_attention_heads' ({self.num_attention_heads}) must be a "
                f"multiple of 'num_key_value_heads' ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"config.json: 'head_dim' ({self.head_dim}) must be even "
                              "(rotation pairs k with k + head_dim/2)")
        if not (self.rms_norm_eps > 0.0):
            raise ConfigError("config.json: 'rms_norm_eps' must be positive")
        if not (self.rope_theta > 0.0):
            raise ConfigError("config.json: 'rope_theta' must be positive")
        if self.sliding_window is not None and self.sliding_window <= 0:
            raise ConfigError("config.json: 'sliding_window' must be positive")
        if len(self.layer_types) != self.num_hidden_layers:
            raise ConfigError("config.json: 'layer_types' must list one entry per layer")

    # ------------------------------------------------------------------ writing
    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        d = {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "hidden_act": "silu",
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "attention_bias": False,
            "tie_word_embeddings": self.tie_word_embeddings,
            "layer_types": list(self.layer_types),
            "sliding_window": self.sliding_window,
            "use_sliding_window": SLIDING in self.layer_types,
        }
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_ids:
            d["eos_token_id"] = (self.eos_token_ids[0] if len(self.eos_token_ids) == 1
                                 else list(self.eos_token_ids))
        return d

    def replace(self, **kw) -> "Qwen3Config":
        d = asdict(self)
        d.update(kw)
        c = Qwen3Config(**d)
        c.validate()
        return c
