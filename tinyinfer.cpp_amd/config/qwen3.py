"""Typed configuration of the Qwen3 dense decoder.

The reference reads nine hyper-parameters from GGUF keys into `Qwen3Config`
(/root/reference/src/model.h:11-21, src/model.cpp:32-47) and refuses a model
whose required sizes are zero.  Here the same fields come from the
architecture's `config.json`; reading and validation are the host library's
(`Qwen3Config::from_json`, config/config.cpp), this class holds the result.
"""
from __future__ import annotations

import json
from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple

from .. import native

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

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "Qwen3Config":
        """Read and validate; an error names the key."""
        return cls.from_normalized(json.loads(native.text("ti_qwen3_config", json.dumps(dict(d)).encode())))

    @classmethod
    def from_normalized(cls, n: Mapping[str, Any]) -> "Qwen3Config":
        """From the keys as the library writes them back (validated, defaults filled in)."""
        eos = n.get("eos_token_id")
        return cls(
            vocab_size=n["vocab_size"], hidden_size=n["hidden_size"], intermediate_size=n["intermediate_size"],
            num_hidden_layers=n["num_hidden_layers"], num_attention_heads=n["num_attention_heads"],
            num_key_value_heads=n["num_key_value_heads"], head_dim=n["head_dim"], rms_norm_eps=n["rms_norm_eps"],
            rope_theta=n["rope_theta"], tie_word_embeddings=n["tie_word_embeddings"],
            layer_types=tuple(n["layer_types"]), sliding_window=n["sliding_window"],
            max_position_embeddings=n.get("max_position_embeddings"),
            eos_token_ids=() if eos is None else tuple(eos) if isinstance(eos, list) else (eos,),
            architecture=n["architectures"][0])

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        d = {
            "architectures": [self.architecture], "model_type": "qwen3", "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size, "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers, "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads, "head_dim": self.head_dim, "hidden_act": "silu",
            "rms_norm_eps": self.rms_norm_eps, "rope_theta": self.rope_theta, "rope_scaling": None,
            "attention_bias": False, "tie_word_embeddings": self.tie_word_embeddings,
            "layer_types": list(self.layer_types), "sliding_window": self.sliding_window,
            "use_sliding_window": SLIDING in self.layer_types,
        }
        if self.max_position_embeddings is not None:
            d["max_position_embeddings"] = self.max_position_embeddings
        if self.eos_token_ids:
            d["eos_token_id"] = self.eos_token_ids[0] if len(self.eos_token_ids) == 1 else list(self.eos_token_ids)
        return d
