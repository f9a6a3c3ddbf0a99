"""The Qwen3 dense decoder as a `ModelSpec`.

Layer order and formulas: /root/reference/src/inference.cu:28-72.  Tensor names
follow the checkpoint convention of the architecture (`model.layers.{i}.…`);
the reference's GGUF names (`blk.{i}.attn_q.weight`, src/model.cpp:120-150) map
onto them one to one.
"""
from __future__ import annotations

from ..spec import LayerSpec, ModelSpec, PartSpec
from ..config.qwen3 import Qwen3Config, SLIDING
from ..registry import register_architecture


def build_qwen3_spec(cfg: Qwen3Config) -> ModelSpec:
    H = cfg.hidden_size
    layers = []
    for i in range(cfg.num_hidden_layers):
        window = cfg.sliding_window if cfg.layer_types[i] == SLIDING else None
        layers.append(LayerSpec(
            prefix=f"model.layers.{i}",
            block=PartSpec("pre_norm"),
            parts={
                "norm1": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, "input_layernorm"),
                "mixer": PartSpec("attention", {
                    "hidden": H, "heads": cfg.num_attention_heads,
                    "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                    "qk_norm": True, "eps": cfg.rms_norm_eps, "window": window,
                    "pos": PartSpec("rope_neox", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta}),
                }, "self_attn"),
                "norm2": PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, "post_attention_layernorm"),
                "ffn": PartSpec("swiglu", {"hidden": H, "intermediate": cfg.intermediate_size}, "mlp"),
            }))
    return ModelSpec(
        architecture=cfg.architecture,
        vocab_size=cfg.vocab_size,
        hidden_size=H,
        embedding=PartSpec("table", {"vocab": cfg.vocab_size, "dim": H}, "model.embed_tokens"),
        layers=layers,
        final_norm=PartSpec("rmsnorm", {"dim": H, "eps": cfg.rms_norm_eps}, "model.norm"),
        lm_head=PartSpec("linear", {"vocab": cfg.vocab_size, "dim": H,
                                    "tied": cfg.tie_word_embeddings,
                                    "tied_to": "model.embed_tokens.weight"}, "lm_head"),
        eos_token_ids=cfg.eos_token_ids,
        max_position_embeddings=cfg.max_position_embeddings,
    )


register_architecture(("Qwen3ForCausalLM", "qwen3"), Qwen3Config.from_dict, build_qwen3_spec)
