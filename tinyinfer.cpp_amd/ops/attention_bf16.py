"""How a step's rows are handed to the bfloat16 matrix-core attention kernels: the
choice is the host library's (`Ops::attention`, ops/ops.cpp).  These functions
name it for tests that run the attention on its own."""
from __future__ import annotations

from .. import native

SERVED_HEAD_DIMS = (32, 64, 128)
MAX_SPLITS = 64               # the merge kernel's limit
MIN_BLOCKS_PER_SPLIT = 16     # four 16-key blocks per wavefront at least


def compute_units() -> int:
    from .kernels import get_ops
    return int(get_ops()._call("compute_units", libs=["core"]))


def decode_splits(n_rows: int, kv_heads: int, heads: int, context: int, typical: int = 0, head_dim: int = 128) -> int:
    """Into how many runs the decode kernel splits the context (`Ops::decode_splits`)."""
    return int(native.lib().ti_decode_splits(n_rows, kv_heads, heads, context, typical or context, compute_units(), head_dim))


def portion_launch(ctx, heads: int, window: int):
    """(runs of keys, paired) for the prefill kernel with 64-row tiles (`Ops::portion_launch`)."""
    import ctypes
    paired = ctypes.c_int()
    runs = native.lib().ti_portion_launch(ctx.n_tiles_small, heads, getattr(ctx, "portion_context", 0), int(window or 0),
                                          compute_units(), ctypes.byref(paired))
    return int(runs), bool(paired.value)


def run(ops, ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window) -> bool:
    """The step's rows through the matrix-core kernels; False if they do not serve the sizes (the
    rows have then gone through the generic kernel)."""
    P = pool.shape[3]
    ops.attention(ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window)
    return head_dim in SERVED_HEAD_DIMS and P % 16 == 0


def run_decode_prepared(ops, ctx, view, qkv, q_w, k_w, eps, inv_freq, rope_table, pool, write_kv, out, heads, kv_heads,
                        head_dim, scale, window) -> bool:
    return ops.attention_from_projections(ctx, view, qkv, q_w, k_w, eps, inv_freq, rope_table, pool, write_kv, out, heads,
                                          kv_heads, head_dim, scale, window)
