"""How a step's rows are handed to the bfloat16 matrix-core attention kernels:
rows of single-token entries go to the flash-decoding kernel (split over the
context so that the launch fills the chip), rows of longer entries to the tiled
prefill kernel.  Head sizes or page sizes the kernels do not serve are left to
the generic kernel (`run` returns False)."""
from __future__ import annotations

import functools

import torch

SERVED_HEAD_DIMS = (32, 64, 128)
MAX_SPLITS = 64               # the merge kernel's limit
MIN_BLOCKS_PER_SPLIT = 16     # four 16-key blocks per wavefront at least (fewer, and the merge costs more than the split gains)
# What a launch of the decode kernel costs, as measured on an MI355X at Qwen3-0.6B's head size (a
# workgroup per row, kv head and split; a compute unit streams about as fast with one workgroup as
# with two, so workgroups beyond one per unit wait for a second round):
SPLIT_PROLOGUE_US = 5.0       # position, table row, query, page ids: before a workgroup's first key arrives
SPLIT_TOKEN_US = 0.019        # per token of context that one workgroup walks
SPLIT_MERGE_US = 4.0          # the merge kernel, which a launch without splits does without


def decode_splits(n_rows: int, kv_heads: int, heads: int, context: int, typical: int = 0) -> int:
    """Into how many runs the decode kernel splits the context.  `context`: the longest context the
    launch is sized for (it bounds the number); `typical`: the context the choice is made for (a
    captured graph is sized for the longest sequence, but replayed mostly on shorter ones).
    The number that makes rounds x (prologue + run) + merge the least, rounds being the
    workgroups over the compute units, rounded up: 12 rows of 8 kv heads take 2 runs (192
    workgroups, one round of half the context: 1.67 ms a step) rather than 3 (288: two rounds of
    a third, 1.90 ms)."""
    return _decode_splits(n_rows, kv_heads, heads, context, typical or context, compute_units())


@functools.lru_cache(maxsize=512)          # every layer of a step asks the same question
def _decode_splits(n_rows: int, kv_heads: int, heads: int, context: int, typical: int, units: int) -> int:
    parts = (heads // kv_heads + 15) // 16
    base = max(1, n_rows * kv_heads * parts)
    blocks = -(-max(1, context) // 16)
    limit = max(1, min(blocks // MIN_BLOCKS_PER_SPLIT, MAX_SPLITS))
    walk = SPLIT_TOKEN_US * max(1, typical)
    best, best_cost = 1, None
    for s in range(1, limit + 1):
        rounds = -(-base * s // units)
        cost = rounds * (SPLIT_PROLOGUE_US + walk / s) + (SPLIT_MERGE_US if s > 1 else 0.0)
        if best_cost is None or cost < best_cost - 1e-9:
            best, best_cost = s, cost
    return best


def typical_context(ctx) -> int:
    """The context a launch's splits are chosen for: the step's own, but for a launch sized for more
    than its step (a graph being captured) no less than half of that size."""
    return max(ctx.max_context, ctx.split_context // 2) if ctx.split_context > ctx.max_context else ctx.max_context


def _ptr(t):
    return None if t is None else t.data_ptr()       # argument types are declared: see kernels.declare_signatures


PREPARED_HEAD_DIMS = (64, 128)   # head sizes whose queries the decode kernel prepares itself
PAIRED_HEAD_DIMS = (64, 128)     # head sizes of the prefill kernel that pairs tiles
PAIRED_BELOW = 1025              # (tiles of 128 rows) x heads below which a launch takes that kernel:
                                 # measured faster up to 8,192 tokens of 16 heads, slower at 16,384


def run_decode_prepared(ops, ctx, view, qkv, q_w, k_w, eps, inv_freq, rope_table, pool, write_kv, out,
                        heads, kv_heads, head_dim, scale, window) -> bool:
    """A step of single-token rows, straight from the 32-bit projections: per-head norm,
    rotation and the write of each row's key and value happen inside the decode kernel.
    False if the kernel does not serve the sizes (nothing has been done then)."""
    P = pool.shape[3]
    if head_dim not in PREPARED_HEAD_DIMS or P % 16 != 0 or heads // kv_heads > 16 or not ctx.decode_only:
        return False
    lib = ops.lib("attention_bf16")
    table = view.table
    win = int(window or 0)
    n = ctx.M
    context = ctx.split_context if win == 0 else min(ctx.split_context, win + 16)
    S = decode_splits(n, kv_heads, heads, context, min(context, typical_context(ctx)))
    part_o = part_ml = None
    if S > 1:
        part_o = ctx.buf("attn.part_o", (n, heads, S, head_dim), torch.float32)
        part_ml = ctx.buf("attn.part_ml", (n, heads, S, 2), torch.float32)
    rc = lib.ti_attention_decode_prepared_bf16(
        _ptr(qkv), qkv.shape[1], _ptr(q_w), _ptr(k_w), eps, _ptr(inv_freq), _ptr(rope_table),
        0 if rope_table is None else rope_table.shape[0], _ptr(pool), 1 if write_kv else 0,
        _ptr(table), table.shape[1], _ptr(ctx.positions), _ptr(ctx.slots), _ptr(out), _ptr(part_o), _ptr(part_ml),
        n, heads, kv_heads, head_dim, P, scale, win, S, ops._stream())
    if rc == 3:
        return False
    ops._check(lib, rc, "attention(decode, prepared)")
    return True


PORTION_SPLIT_KEYS = 512         # a portion's keys are cut into runs of at least this many ...
PORTION_SPLIT_MAX = 8            # ... at most this many runs


def portion_launch(ctx, heads: int, window: int):
    """(runs of keys, paired) for the prefill kernel with 64-row tiles.  A launch whose tiles all find
    a compute unit at once gives each tile a workgroup of its own (it lasts as long as its heaviest
    tile then); a larger one pairs the heaviest tile with the lightest.  The keys are cut into
    runs when the launch would leave most units idle (a short portion) while every workgroup walks a
    long context (191 us a layer for 512 rows against 6,144 cached tokens in one run)."""
    longest = getattr(ctx, "portion_context", 0)
    context = longest if window == 0 else min(longest, window + 64)
    units = compute_units()
    paired = ctx.n_tiles_small * heads > units
    workgroups = ((ctx.n_tiles_small + 1) // 2 if paired else ctx.n_tiles_small) * heads
    if workgroups * 2 > units or context < 2 * PORTION_SPLIT_KEYS:
        return 1, paired
    return max(1, min(PORTION_SPLIT_MAX, units // workgroups, context // PORTION_SPLIT_KEYS)), paired


_units = {}


def compute_units() -> int:
    dev = torch.cuda.current_device()
    if dev not in _units:
        _units[dev] = torch.cuda.get_device_properties(dev).multi_processor_count
    return _units[dev]


def run(ops, ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window) -> bool:
    P = pool.shape[3]
    if head_dim not in SERVED_HEAD_DIMS or P % 16 != 0:
        return False
    lib = ops.lib("attention_bf16")
    stream = ops._stream()
    table = view.table
    win = int(window or 0)
    # the portions first: with their keys cut into runs, the merge writes every row of the step, and
    # the rows of single tokens get their own result afterwards
    if ctx.n_tiles and head_dim in PAIRED_HEAD_DIMS and ctx.n_tiles * heads < PAIRED_BELOW \
            and getattr(ctx, "tiles_small", None) is not None and ops.use_paired_prefill:
        # few tiles: under a causal mask they differ much in work, and a launch lasts as long as its
        # heaviest workgroup; the paired kernel gives every workgroup a heavy and a light tile
        S, paired = portion_launch(ctx, heads, win)
        if not ops.use_portion_splits:
            S = 1
        if ops.force_paired_tiles is not None:
            paired = ops.force_paired_tiles
        part_o = part_ml = None
        if S > 1:
            part_o = ctx.buf("attn.portion_o", (ctx.M, heads, S, head_dim), torch.float32)
            part_ml = ctx.buf("attn.portion_ml", (ctx.M, heads, S, 2), torch.float32)
        rc = lib.ti_attention_prefill_paired_bf16(
            _ptr(q), _ptr(pool), _ptr(table), table.shape[1], _ptr(ctx.tiles_small), _ptr(ctx.entry_meta), _ptr(out),
            ctx.n_tiles_small, heads, kv_heads, head_dim, P, scale, win, ctx.M, _ptr(part_o),
            _ptr(part_ml), S, int(paired), stream)
        if rc == 3:
            return False
        ops._check(lib, rc, "attention(prefill, paired)")
    elif ctx.n_tiles:
        rc = lib.ti_attention_prefill_bf16(
            _ptr(q), _ptr(pool), _ptr(table), table.shape[1], _ptr(ctx.tiles), _ptr(ctx.entry_meta), _ptr(out),
            ctx.n_tiles, heads, kv_heads, head_dim, P, scale, win, stream)
        if rc == 3:
            return False
        ops._check(lib, rc, "attention(prefill)")
    n_dec = ctx.M if ctx.decode_only else ctx.n_decode_rows
    if n_dec:
        rows = None if ctx.decode_only else ctx.decode_rows
        context = ctx.split_context if win == 0 else min(ctx.split_context, win + 16)
        S = decode_splits(n_dec, kv_heads, heads, context, min(context, typical_context(ctx)))
        part_o = part_ml = None
        if S > 1:
            part_o = ctx.buf("attn.part_o", (n_dec, heads, S, head_dim), torch.float32)
            part_ml = ctx.buf("attn.part_ml", (n_dec, heads, S, 2), torch.float32)
        rc = lib.ti_attention_decode_bf16(
            _ptr(q), _ptr(pool), _ptr(table), table.shape[1], _ptr(ctx.positions), _ptr(ctx.slots), _ptr(rows),
            _ptr(out), _ptr(part_o), _ptr(part_ml), n_dec, heads, kv_heads, head_dim, P, scale,
            win, S, stream)
        if rc == 3:
            return False
        ops._check(lib, rc, "attention(decode)")
    return True
