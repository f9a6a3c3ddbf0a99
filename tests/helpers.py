"""Tiny configurations and helpers shared by the tests.

The configurations differ in every size and option: layers, width, heads and
groups, head size, feed-forward width, vocabulary, rotation base, eps, tied or
untied head, window.  None of their sizes is a power of two where it can be
avoided (B, C)."""
import json
import os

import numpy as np

CONFIGS = {
    # 2 layers, width 64, 4 heads in 2 groups, head 16, tied head, theta 1e4, eps 1e-6
    "A": dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=64,
              num_attention_heads=4, num_key_value_heads=2, head_dim=16, intermediate_size=128,
              vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              attention_bias=False, hidden_act="silu", max_position_embeddings=4096),
    # 3 layers, width 96, 6 heads in 2 groups (ratio 3), head 32 (heads*head = 192 != width), untied
    "B": dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3, hidden_size=96,
              num_attention_heads=6, num_key_value_heads=2, head_dim=32, intermediate_size=224,
              vocab_size=1000, rope_theta=1000000.0, rms_norm_eps=1e-5, tie_word_embeddings=False,
              attention_bias=False, hidden_act="silu", max_position_embeddings=4096),
    # 4 layers, width 80, 5 heads each its own group, head 48, a window of 20 on layers 2 and 3
    "C": dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=4, hidden_size=80,
              num_attention_heads=5, num_key_value_heads=5, head_dim=48, intermediate_size=176,
              vocab_size=517, rope_theta=500000.0, rms_norm_eps=3e-6, tie_word_embeddings=False,
              attention_bias=False, hidden_act="silu", max_position_embeddings=4096,
              use_sliding_window=True, sliding_window=20, max_window_layers=2),
    # 3 layers, width 96, 3 heads on one kv head, head 64 (served by the matrix-core attention
    # kernels), a window of 37 on layers 1 and 2
    "D": dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=3, hidden_size=96,
              num_attention_heads=3, num_key_value_heads=1, head_dim=64, intermediate_size=160,
              vocab_size=333, rope_theta=200000.0, rms_norm_eps=2e-6, tie_word_embeddings=True,
              attention_bias=False, hidden_act="silu", max_position_embeddings=4096,
              layer_types=["full_attention", "sliding_attention", "sliding_attention"], sliding_window=37),
    # not tiny in its widths: the layer sizes of Qwen3-0.6B (width 1024, 16 heads in 8 groups, head 128,
    # feed-forward 3072), 2 layers, a small vocabulary.  The kernels chosen for these widths (the tiles
    # of the products, the projection that finishes its heads, two-group prefill attention, the norm
    # inside a product, decode attention that prepares its query) differ from the tiny models' ones.
    "E": dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=2, hidden_size=1024,
              num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072,
              vocab_size=1500, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              attention_bias=False, hidden_act="silu", max_position_embeddings=4096),
    # one layer with the widths of Qwen3-4B: 2,560 is no multiple of 1,024 (other tiles of the products:
    # 160 columns wide), 32 query heads on 8 kv heads, a feed-forward of 9,728
    "F": dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=1, hidden_size=2560,
              num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=9728,
              vocab_size=1200, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              attention_bias=False, hidden_act="silu", max_position_embeddings=4096),
}

# Shapes at the edges of what a configuration may say: the largest and the smallest head, one head per group and
# seventeen, a window on every layer, widths that are multiples of 8 only, an odd vocabulary.  Used in one way of
# cutting the work each (tests/test_engine_gpu.py).
_ODD = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", rope_theta=10000.0, rms_norm_eps=1e-6,
            tie_word_embeddings=True, attention_bias=False, hidden_act="silu", max_position_embeddings=4096)
ODD_CONFIGS = {
    "head 256": dict(_ODD, num_hidden_layers=2, hidden_size=72, num_attention_heads=2, num_key_value_heads=1, head_dim=256,
                     intermediate_size=100, vocab_size=301),
    "head 16": dict(_ODD, num_hidden_layers=5, hidden_size=56, num_attention_heads=7, num_key_value_heads=7, head_dim=16,
                    intermediate_size=24, vocab_size=97, rms_norm_eps=1e-4),
    "head 80, a window of 5 everywhere": dict(_ODD, num_hidden_layers=2, hidden_size=128, num_attention_heads=4,
                                              num_key_value_heads=2, head_dim=80, intermediate_size=192, vocab_size=513,
                                              use_sliding_window=True, sliding_window=5, max_window_layers=0),
    "head 112": dict(_ODD, num_hidden_layers=1, hidden_size=40, num_attention_heads=3, num_key_value_heads=3, head_dim=112,
                     intermediate_size=88, vocab_size=1001, tie_word_embeddings=False, rope_theta=1e6),
    "three heads a group, head 128": dict(_ODD, num_hidden_layers=2, hidden_size=192, num_attention_heads=12,
                                          num_key_value_heads=4, head_dim=128, intermediate_size=320, vocab_size=777),
    "seventeen heads on one group": dict(_ODD, num_hidden_layers=2, hidden_size=64, num_attention_heads=17,
                                         num_key_value_heads=1, head_dim=64, intermediate_size=128, vocab_size=200),
}


def read_folder(path):
    """(config dict, {name: float64 array}) of a model folder, read with the
    safetensors package (not with the framework's own reader)."""
    import torch
    from safetensors.torch import load_file
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    w = {k: v.to(torch.float64).numpy() for k, v in load_file(os.path.join(path, "model.safetensors")).items()}
    return cfg, w


def sharpen_folder(path, factor=4.0):
    """Scale every q_norm weight so that attention scores spread out and single
    keys dominate: a wrong key, mask edge or page then changes the logits visibly."""
    import torch
    from safetensors.torch import load_file, save_file
    fn = os.path.join(path, "model.safetensors")
    t = load_file(fn)
    for k in t:
        if k.endswith("q_norm.weight"):
            t[k] = (t[k].to(torch.float32) * factor).to(t[k].dtype)
    save_file(t, fn)


def random_tokens(n, vocab, seed):
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, size=n)]
