"""Operator selftest: every kernel against a plain float64 computation on the CPU, in the
manner of the reference's `QWEN_SELFTEST=1` (/root/reference/src/selftest.cpp:463-473; its
cases and tolerances: 33-72 product, 74-100 RMSNorm, 102-134 rotation, 136-390 per-head
norm + rotation + cache + attention, 392-459 products of the model's shapes with timings).

    TINY_SELFTEST=1 bin/tinyinfer          or          python -m tinyinfer_amd.selftest

The exit code is the number of failed cases.  The cases keep the reference's sizes where the
reference names them; operands are drawn from a seeded generator, rounded to bfloat16 where
the kernels take bfloat16, and the CPU side computes in float64 from those same values.
"""
from __future__ import annotations

import math
import sys
import time

import numpy as np
import torch


def _say(name: str, err: float, tol: float, extra: str = "") -> int:
    ok = err < tol and math.isfinite(err)
    print(f"[selftest] {name:46s} max err {err:.3e}  (< {tol:.1e})  {'ok' if ok else 'FAIL'}{extra}", flush=True)
    return 0 if ok else 1


def _dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def _f64(t) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy()


def _bf16(a: np.ndarray) -> np.ndarray:
    """Round to bfloat16 (nearest even) and come back as float64."""
    return torch.as_tensor(a, dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy()


class _View:
    def __init__(self, table):
        self.table = table


class _Ctx:
    """What the attention dispatch reads of a step: rows of single tokens, or one portion."""

    def __init__(self, positions, one_portion: bool):
        M = len(positions)
        self.M = M
        self.positions = _dev(np.asarray(positions, dtype=np.int32))
        self.slots = _dev(np.zeros(M, dtype=np.int32))
        self.decode_only = not one_portion
        self.decode_rows, self.n_decode_rows = None, 0
        self.n_tiles = -(-M // 128) if one_portion else 0
        self.tiles = _dev(np.array([[0, 128 * i] for i in range(self.n_tiles)], dtype=np.int32)) if one_portion else None
        self.n_tiles_small = -(-M // 64) if one_portion else 0     # from the most keys to the fewest
        self.tiles_small = _dev(np.array([[0, 64 * i] for i in reversed(range(self.n_tiles_small))],
                                         dtype=np.int32)) if one_portion else None
        self.entry_meta = _dev(np.array([[0, M, positions[0], 0]], dtype=np.int32))
        self.max_context = self.split_context = int(max(positions)) + 1

    def buf(self, name, shape, dtype):
        return torch.empty(tuple(shape), dtype=dtype, device="cuda")


# ------------------------------------------------------------------ the cases
def case_linear(ops, rng) -> int:
    fails = 0
    M, N, K = 5, 261, 1024                       # the reference's case: N odd, bounds of the tiles
    a, w = _bf16(rng.uniform(-1, 1, (M, K))), _bf16(rng.uniform(-1, 1, (N, K)))
    want = a @ w.T
    for dtype in (torch.bfloat16, torch.float32):
        out = torch.empty(M, N, device="cuda")
        ops.linear(_dev(a, dtype), _dev(w, dtype), out, "store")
        fails += _say(f"product {M}x{N}x{K} {str(dtype)[6:]}", float(np.abs(_f64(out) - want).max()), 2e-5 * K)
    # all epilogues at a size that is no multiple of anything, many rows (the tiled kernels)
    M, N, K = 203, 130, 192
    a, w = _bf16(rng.uniform(-1, 1, (M, K))), _bf16(rng.uniform(-1, 1, (N, K)))
    base = rng.normal(size=(M, N)).astype(np.float32)
    want = a @ w.T
    out = _dev(base.copy())
    ops.linear(_dev(a, torch.bfloat16), _dev(w, torch.bfloat16), out, "add")
    fails += _say("product + residual add", float(np.abs(_f64(out) - (want + base)).max()), 2e-5 * K + 1e-5)
    F = N // 2
    g, u = want[:, :F], want[:, F:]
    out = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
    ops.linear(_dev(a, torch.bfloat16), _dev(w, torch.bfloat16), out, "swiglu")
    swi = g / (1 + np.exp(-g)) * u
    fails += _say("product + SwiGLU (bfloat16 out)", float(np.abs(_f64(out) - swi).max()), 0.005 * np.abs(swi).max() + 1e-3)
    # few rows times a long K (the token rows go through LDS in pieces; with a long K under few weight
    # rows the sums of several workgroups are left to whatever reads the residual next)
    for M, N, K in ((7, 2100, 5120), (16, 2064, 17408)):
        a, w = _bf16(rng.uniform(-1, 1, (M, K))), _bf16(rng.uniform(-1, 1, (N, K)))
        base = rng.normal(size=(M, N)).astype(np.float32)
        out = _dev(base.copy())
        ops.linear(_dev(a, torch.bfloat16), _dev(w, torch.bfloat16), out, "add", may_defer=True)
        ops.flush()
        fails += _say(f"product {M}x{N}x{K} + residual add (K in pieces)", float(np.abs(_f64(out) - (a @ w.T + base)).max()),
                      2e-5 * K)
    return fails


def case_model_shapes(ops, rng) -> int:
    """The projections of a 0.6B layer at two rows, with timings (reference: printed only)."""
    fails = 0
    for N, K in ((4096, 1024), (2048, 1024), (1024, 1024), (1024, 3072), (2048, 3072)):
        a, w = _bf16(rng.uniform(-1, 1, (2, K))), _bf16(rng.uniform(-1, 1, (N, K)) * 0.05)
        ad, wd = _dev(a, torch.bfloat16), _dev(w, torch.bfloat16)
        out = torch.empty(2, N, device="cuda")
        ops.linear(ad, wd, out, "store")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(100):
            ops.linear(ad, wd, out, "store")
        torch.cuda.synchronize()
        us = (time.perf_counter() - t0) / 100 * 1e6
        fails += _say(f"product 2x{N}x{K} (a layer's shape)", float(np.abs(_f64(out) - a @ w.T).max()), 0.02,
                      f"  {us:6.1f} us  {N * K * 2 / us / 1e3:6.0f} GB/s")
    return fails


def case_rmsnorm(ops, rng) -> int:
    rows, n, eps = 3, 1024, 1e-6
    x, w = rng.uniform(-1, 1, (rows, n)).astype(np.float32), rng.uniform(-1, 1, n).astype(np.float32)
    xd = x.astype(np.float64)
    want = xd / np.sqrt((xd * xd).mean(-1, keepdims=True) + eps) * w
    out = torch.empty(rows, n, device="cuda")
    ops.rmsnorm(_dev(x), _dev(w), eps, out)
    fails = _say("RMSNorm 3x1024", float(np.abs(_f64(out) - want).max()), 1e-4)
    # rows wider than 4,096 take a workgroup each
    rows, n = 5, 5120
    x, w = rng.uniform(-1, 1, (rows, n)).astype(np.float32), rng.uniform(-1, 1, n).astype(np.float32)
    xd = x.astype(np.float64)
    want = xd / np.sqrt((xd * xd).mean(-1, keepdims=True) + eps) * w
    out = torch.empty(rows, n, device="cuda")
    ops.rmsnorm(_dev(x), _dev(w), eps, out)
    fails += _say("RMSNorm 5x5120", float(np.abs(_f64(out) - want).max()), 1e-4)
    return fails


def _rotate(x, positions, theta):
    """x [M, heads, hd] float64; pairs (k, k + hd/2), angle pos * theta^(-2k/hd)."""
    hd = x.shape[-1]
    half = hd // 2
    ang = np.asarray(positions, dtype=np.float64)[:, None] * theta ** (-2.0 * np.arange(half) / hd)[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return np.concatenate([lo * c - hi * s, lo * s + hi * c], axis=-1)


def case_rope(ops, rng) -> int:
    rows, heads, hd, theta = 2, 4, 128, 1e6
    x = rng.uniform(-1, 1, (rows, heads, hd)).astype(np.float32)
    pos = [0, 5]
    inv = (theta ** (-2.0 * np.arange(hd // 2) / hd)).astype(np.float32)
    xd = _dev(x)
    ops.rope_neox(xd, _dev(np.asarray(pos, dtype=np.int32)), _dev(inv))
    return _say("rotation 2x4x128, positions 0 and 5", float(np.abs(_f64(xd) - _rotate(x.astype(np.float64), pos, theta)).max()), 1e-4)


def case_attention(ops, rng, nh, nkv, hd, T, dtype, eps=1e-6, theta=1e6, P=16) -> int:
    """Per-head norm, rotation, cache write and causal attention of T tokens of one request: as one
    portion, and as T steps of one token; against float64 from the rounded cache values."""
    name = f"norm+rotation+cache+attention hd={hd} {nh}/{nkv} heads {str(dtype)[6:]}"
    width = (nh + 2 * nkv) * hd
    qkv = rng.uniform(-1, 1, (T, width)).astype(np.float32)
    q_w, k_w = rng.uniform(0.5, 1.5, hd).astype(np.float32), rng.uniform(0.5, 1.5, hd).astype(np.float32)
    inv = (theta ** (-2.0 * np.arange(hd // 2) / hd)).astype(np.float32)

    def heads(a, n):
        return a.reshape(T, n, hd).astype(np.float64)

    def norm(a, w):
        return a / np.sqrt((a * a).mean(-1, keepdims=True) + eps) * w
    pos = list(range(T))
    rnd = _bf16 if dtype == torch.bfloat16 else (lambda z: z)
    q = rnd(_rotate(norm(heads(qkv[:, :nh * hd], nh), q_w), pos, theta))
    k = rnd(_rotate(norm(heads(qkv[:, nh * hd:(nh + nkv) * hd], nkv), k_w), pos, theta))
    v = rnd(heads(qkv[:, (nh + nkv) * hd:], nkv))
    want = np.zeros((T, nh, hd))
    for h in range(nh):
        s = q[:, h] @ k[:, h // (nh // nkv)].T / math.sqrt(hd)
        s[np.triu_indices(T, 1)] = -np.inf
        p = np.exp(s - s.max(-1, keepdims=True))
        want[:, h] = (p / p.sum(-1, keepdims=True)) @ v[:, h // (nh // nkv)]
    want = want.reshape(T, nh * hd)
    n_pages = -(-T // P) + 1
    table = _dev(np.arange(n_pages, dtype=np.int32)[::-1].copy()[None, :])     # pages in descending order
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    fails = 0
    for mode in ("one portion", "token by token"):
        pool = torch.zeros(n_pages, 2, nkv, P, hd, device="cuda", dtype=dtype)
        got = torch.empty(T, nh * hd, device="cuda", dtype=dtype)
        steps = [pos] if mode == "one portion" else [[p] for p in pos]
        for rows in steps:
            ctx = _Ctx(rows, one_portion=(mode == "one portion"))
            qd = torch.empty(len(rows), nh * hd, device="cuda", dtype=dtype)
            ops.qk_norm_rope_kv_write(_dev(qkv[rows]), _dev(q_w), _dev(k_w), eps, _dev(inv), ctx.positions, ctx.slots,
                                      _View(table), pool, qd, nh, nkv, hd)
            out = torch.empty_like(qd)
            ops.attention(ctx, _View(table), qd, pool, out, nh, nkv, hd, 1.0 / math.sqrt(hd), None)
            got[rows[0]:rows[-1] + 1] = out
        fails += _say(f"{name}, {mode}", float(np.abs(_f64(got) - want).max()), tol)
    return fails


def case_embed_argmax_sample(ops, rng) -> int:
    fails = 0
    V, H = 1000, 96
    E = _bf16(rng.normal(size=(V, H)))
    toks = np.array([5, 0, 999, 5], dtype=np.int32)
    x = torch.empty(4, H, device="cuda")
    ops.embed(_dev(E, torch.bfloat16), _dev(toks), x)
    fails += _say("embedding rows", float(np.abs(_f64(x) - E[toks]).max()), 1e-12)
    logits = rng.normal(size=(3, 151936)).astype(np.float32)
    logits[1, 77] = logits[1, 4000] = 9.0                        # a tie: the lowest index wins
    out = torch.empty(3, dtype=torch.int32, device="cuda")
    ops.argmax(_dev(logits), out)
    fails += _say("argmax, ties to the lowest index", float(np.abs(out.cpu().numpy() - logits.argmax(-1)).max()), 0.5)
    # temperature sampling: the token is where the inverse CDF of softmax(logits / T) crosses u
    small = rng.normal(size=(2, 50)).astype(np.float32) * 3
    T, u = 0.7, np.array([0.25, 0.9], dtype=np.float32)
    z = small.astype(np.float64) / T
    p = np.exp(z - z.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    cdf = np.cumsum(p, -1)
    got = torch.empty(2, dtype=torch.int32, device="cuda")
    ops.sample(_dev(small), _dev(np.full(2, T, dtype=np.float32)), _dev(np.full(2, 50, dtype=np.int32)),
               _dev(np.ones(2, dtype=np.float32)), _dev(u), got)
    tok = got.cpu().numpy()
    # u must fall into the drawn token's interval of the cumulative distribution
    miss = max(max(cdf[i, tok[i]] - p[i, tok[i]] - u[i], u[i] - cdf[i, tok[i]], 0.0) for i in range(2))
    fails += _say("temperature sampling, inverse CDF", float(miss), 1e-4)
    return fails


def case_head_bandwidth(ops, rng) -> int:
    """One row through an output matrix of the real vocabulary (reference: timing only)."""
    N, K = 151936, 1024
    w = (torch.randn(N, K, device="cuda") * 0.02).to(torch.bfloat16)
    a = torch.randn(1, K, device="cuda").to(torch.bfloat16)
    out = torch.empty(1, N, device="cuda")
    ops.linear(a, w, out, "store")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        ops.linear(a, w, out, "store")
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) / 20 * 1e6
    want = _f64(a) @ _f64(w[:64]).T
    return _say("product 1x151936x1024 (the output matrix)", float(np.abs(_f64(out[:, :64]) - want).max()), 0.02,
                f"  {us:6.1f} us  {N * K * 2 / us / 1e3:6.0f} GB/s")


def run_selftest() -> int:
    if not torch.cuda.is_available():
        print("[selftest] no GPU: the kernels of this framework run on an AMD GPU (gfx950) only", flush=True)
        return 1
    from .engine.engine import required_libraries
    from .ops.kernels import get_ops
    ops = get_ops()
    ops.preload(required_libraries("bfloat16"))
    rng = np.random.default_rng(1)
    fails = 0
    fails += case_linear(ops, rng)
    fails += case_rmsnorm(ops, rng)
    fails += case_rope(ops, rng)
    fails += case_attention(ops, rng, nh=4, nkv=2, hd=64, T=5, dtype=torch.float32)
    fails += case_attention(ops, rng, nh=4, nkv=2, hd=64, T=150, dtype=torch.bfloat16)
    fails += case_attention(ops, rng, nh=16, nkv=8, hd=128, T=2, dtype=torch.float32)
    fails += case_attention(ops, rng, nh=16, nkv=8, hd=128, T=300, dtype=torch.bfloat16)
    fails += case_attention(ops, rng, nh=3, nkv=1, hd=48, T=40, dtype=torch.bfloat16)
    fails += case_embed_argmax_sample(ops, rng)
    fails += case_model_shapes(ops, rng)
    fails += case_head_bandwidth(ops, rng)
    print(f"[selftest] {'all cases passed' if fails == 0 else str(fails) + ' case(s) FAILED'}", flush=True)
    return fails


if __name__ == "__main__":
    sys.exit(run_selftest())
