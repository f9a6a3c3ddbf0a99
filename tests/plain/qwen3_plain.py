"""A plain, slow implementation of the Qwen3 dense decoder, written from the
reference's formulas.  Whole sequences, no cache, one function per part, numpy
float64.  It shares no code with the engine: the tests compare the two.

Every function cites the lines of /root/reference it was written from.
`rnd(site, array)` is applied where the reference rounds to bfloat16; the
default rounds nothing, which gives the mathematically exact model.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, Optional, Sequence

import numpy as np

Rounder = Callable[[str, np.ndarray], np.ndarray]


def no_rounding(site: str, a: np.ndarray) -> np.ndarray:
    return a


def round_bf16(a: np.ndarray) -> np.ndarray:
    """Round to the nearest bfloat16 (ties to even), returned as float64."""
    f = np.asarray(a, dtype=np.float32)
    u = f.view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = ((u + 0x7FFF + lsb) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32)
    out = np.where(np.isfinite(f), out, f)
    return out.astype(np.float64).reshape(np.shape(a))


def bf16_sites(sites: Sequence[str]) -> Rounder:
    """A rounder that rounds to bfloat16 at the named sites only."""
    chosen = set(sites)

    def rnd(site: str, a: np.ndarray) -> np.ndarray:
        return round_bf16(a) if site in chosen else a
    return rnd


def float32_angles(rnd: Rounder = no_rounding) -> Rounder:
    """`rnd`, and the rotation's frequencies and angles rounded to 32-bit floats as well (their sine and cosine
    stay exact): what an engine that keeps to "angles in 32-bit" computes (src/cuda/rope.cu:20)."""
    def both(site: str, a: np.ndarray) -> np.ndarray:
        if site in ("rope_inv_freq", "rope_angle"):
            return np.asarray(a, dtype=np.float32).astype(np.float64)
        return rnd(site, a)
    return both


# The places where the reference drops to bfloat16: the operand of every matrix
# product (src/inference.cu:40,53,59,63; src/cuda/lm_head.cu:8) and the cached
# keys and values (src/cuda/attention.cu:83-84).
REFERENCE_SITES = ("gemm_in", "kv_cache")


def embed(table: np.ndarray, tokens: Sequence[int]) -> np.ndarray:
    """x[m,:] = E[tok[m],:], no scaling.  src/inference.cu:14-24."""
    return np.asarray(table, dtype=np.float64)[np.asarray(tokens, dtype=np.int64)]


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """x * rsqrt(mean(x^2) + eps) * w over the last axis; eps inside the root,
    the weight multiplies directly.  src/cuda/rms_norm.cu:15-25."""
    x = np.asarray(x, dtype=np.float64)
    ms = np.mean(x * x, axis=-1, keepdims=True)
    return x / np.sqrt(ms + eps) * np.asarray(w, dtype=np.float64)


def linear(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    """C = A . W^T with W stored [out, in].  src/cuda/gemm.cuh:5-6."""
    return np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T


def rope_neox(x: np.ndarray, positions: Sequence[int], theta: float, rnd: Rounder = no_rounding) -> np.ndarray:
    """Half-split rotation over the whole head: for k < hd/2 the angle is
    pos * theta^(-2k/hd); (x[k], x[k+hd/2]) -> (x[k] c - x[k+hd/2] s,
    x[k] s + x[k+hd/2] c).  x: [T, heads, hd].
    src/cuda/attention.cu:38,64-74; src/cuda/rope.cu:20-28.  The reference has the frequency and
    the angle in 32-bit (rope.cu:20); `rnd` may round them at the sites "rope_inv_freq" and
    "rope_angle" (see `float32_angles`): thousands of tokens in, that is what limits the agreement
    of a 32-bit engine with this model."""
    x = np.asarray(x, dtype=np.float64)
    hd = x.shape[-1]
    half = hd // 2
    k = np.arange(half, dtype=np.float64)
    inv = rnd("rope_inv_freq", theta ** (-2.0 * k / hd))
    ang = rnd("rope_angle", np.asarray(positions, dtype=np.float64)[:, None] * inv[None, :])   # [T, half]
    c = np.cos(ang)[:, None, :]
    s = np.sin(ang)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return np.concatenate([lo * c - hi * s, lo * s + hi * c], axis=-1)


def qk_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """RMSNorm of every head by itself over head_dim, one weight for all heads.
    x: [T, heads, hd].  src/cuda/attention.cu:51-62."""
    return rms_norm(x, w, eps)


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray,
              window: Optional[int] = None) -> np.ndarray:
    """Causal grouped-query attention.  q: [T, nh, hd]; k, v: [T, nkv, hd].
    Head h reads kv head h // (nh/nkv); score = (q.k) / sqrt(hd); keys p <= t
    (src/cuda/attention.cu:127-130,143-197).  With `window` w a row also drops
    keys p <= t - w (the reference has no window; this is the usual sliding
    rule: the newest w keys, the row's own included)."""
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    T, nh, hd = q.shape
    nkv = k.shape[1]
    G = nh // nkv
    out = np.zeros((T, nh, v.shape[-1]), dtype=np.float64)
    scale = 1.0 / math.sqrt(hd)
    for h in range(nh):
        kh = h // G
        for t in range(T):
            lo = 0 if window is None else max(0, t - window + 1)
            s = (k[lo:t + 1, kh, :] @ q[t, h, :]) * scale
            s = s - s.max()
            p = np.exp(s)
            p = p / p.sum()
            out[t, h, :] = p @ v[lo:t + 1, kh, :]
    return out


def swiglu(g: np.ndarray, u: np.ndarray) -> np.ndarray:
    """y = g / (1 + exp(-g)) * u.  src/cuda/ffn.cu:13-15."""
    g = np.asarray(g, dtype=np.float64)
    return g / (1.0 + np.exp(-g)) * np.asarray(u, dtype=np.float64)


def attention_block(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, cfg: dict,
                    positions: Sequence[int], window: Optional[int], rnd: Rounder) -> np.ndarray:
    """Projections, per-head norm (before rotation; V is not normed), rotation of
    q and k, attention, output projection.  src/inference.cu:41-54."""
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    eps, theta = cfg["rms_norm_eps"], cfg["rope_theta"]
    T = h.shape[0]
    hb = rnd("gemm_in", h)
    q = linear(hb, w[prefix + ".q_proj.weight"]).reshape(T, nh, hd)
    k = linear(hb, w[prefix + ".k_proj.weight"]).reshape(T, nkv, hd)
    v = linear(hb, w[prefix + ".v_proj.weight"]).reshape(T, nkv, hd)
    q = rope_neox(qk_norm(q, w[prefix + ".q_norm.weight"], eps), positions, theta, rnd)
    k = rope_neox(qk_norm(k, w[prefix + ".k_norm.weight"], eps), positions, theta, rnd)
    q = rnd("q", q)
    k = rnd("kv_cache", k)
    v = rnd("kv_cache", v)
    a = attention(q, k, v, window).reshape(T, nh * hd)
    return linear(rnd("gemm_in", a), w[prefix + ".o_proj.weight"])


def ffn_block(h: np.ndarray, w: Dict[str, np.ndarray], prefix: str, rnd: Rounder) -> np.ndarray:
    """gate and up projections, SwiGLU, down projection.  src/inference.cu:60-64."""
    hb = rnd("gemm_in", h)
    y = swiglu(linear(hb, w[prefix + ".gate_proj.weight"]), linear(hb, w[prefix + ".up_proj.weight"]))
    return linear(rnd("gemm_in", y), w[prefix + ".down_proj.weight"])


def layer_windows(cfg: dict):
    """The window of each layer (None: all keys), from config.json's keys."""
    n = cfg["num_hidden_layers"]
    types = cfg.get("layer_types")
    win = cfg.get("sliding_window")
    if types is None:
        if cfg.get("use_sliding_window") and win is not None:
            first = cfg.get("max_window_layers", n)
            types = ["sliding_attention" if i >= first else "full_attention" for i in range(n)]
        else:
            types = ["full_attention"] * n
    return [win if t == "sliding_attention" else None for t in types]


def forward(w: Dict[str, np.ndarray], cfg: dict, tokens: Sequence[int],
            rnd: Rounder = no_rounding, first_position: int = 0) -> np.ndarray:
    """Logits [T, V] of a whole sequence.  Pre-norm residual blocks
    x += Attn(Norm1(x)); x += FFN(Norm2(x)) (src/inference.cu:35-66), final norm
    and the head, tied to the embedding unless the weights hold `lm_head.weight`
    (src/inference.cu:68-71).  `first_position` shifts every position: only
    distances count, so the logits must not change."""
    eps = cfg["rms_norm_eps"]
    T = len(tokens)
    positions = [first_position + t for t in range(T)]
    windows = layer_windows(cfg)
    x = embed(w["model.embed_tokens.weight"], tokens)
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}"
        h = rms_norm(x, w[p + ".input_layernorm.weight"], eps)
        x = x + attention_block(h, w, p + ".self_attn", cfg, positions, windows[i], rnd)
        h = rms_norm(x, w[p + ".post_attention_layernorm.weight"], eps)
        x = x + ffn_block(h, w, p + ".mlp", rnd)
    h = rms_norm(x, w["model.norm.weight"], eps)
    tied = cfg.get("tie_word_embeddings")
    if tied is None:
        tied = "lm_head.weight" not in w
    head = w["model.embed_tokens.weight"] if tied else w["lm_head.weight"]
    return linear(rnd("gemm_in", h), head)


# ------------------------------------------------------------------- sampling
def argmax_lowest(logits: np.ndarray) -> int:
    """Greedy choice; of equal logits the lowest index wins.
    src/cuda/sample.cu:5-11; src/main.cpp:31-38."""
    return int(np.argmax(np.asarray(logits)))


def sample_distribution(logits: np.ndarray, temperature: float, top_k: int = 0,
                        top_p: float = 1.0) -> np.ndarray:
    """The distribution the reference's host sampler draws from
    (src/main.cpp:40-73): keep the K largest logits (K = top_k, or 512 when
    top_k is 0), weights exp(l/T - max), then the shortest prefix in descending
    order whose mass reaches top_p, renormalised.  Returned over the whole
    vocabulary.  The reference subtracts the unscaled maximum (main.cpp:60),
    which only changes a common factor; max(l)/T is used here."""
    l = np.asarray(logits, dtype=np.float64)
    V = l.shape[0]
    K = max(1, min(V, top_k if top_k > 0 else 512))
    order = np.argsort(-l, kind="stable")
    keep = order[:K]
    # everything equal to the K-th value stays too (the reference's nth_element
    # picks among equals arbitrarily)
    keep = np.nonzero(l >= l[keep[-1]])[0]
    keep = keep[np.argsort(-l[keep], kind="stable")]
    wts = np.exp((l[keep] - l[keep[0]]) / temperature)
    if top_p < 1.0:
        acc = np.cumsum(wts / wts.sum())
        cut = int(np.searchsorted(acc, top_p, side="left")) + 1
        cut = min(cut, len(keep))
        # equal weights at the cut stay together
        last = wts[cut - 1]
        while cut < len(keep) and wts[cut] == last:
            cut += 1
        keep, wts = keep[:cut], wts[:cut]
    p = np.zeros(V, dtype=np.float64)
    p[keep] = wts / wts.sum()
    return p


def draw(p: np.ndarray, u: float) -> int:
    """Inverse CDF over the index order: the first index whose cumulative
    probability exceeds u."""
    c = np.cumsum(p)
    i = int(np.searchsorted(c, u * c[-1], side="right"))
    nz = np.nonzero(p)[0]
    return int(min(max(i, nz[0]), nz[-1]))
