"""Each kernel alone against a plain PyTorch reference of the same op (float64
on the CPU), at sizes other than the engine's.  Vectors that the reference's own
selftest holds are marked with its file:line."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def run_attention(ops, ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window):
    """The step's rows through `Ops.attention`; whether the matrix-core kernels serve these sizes (else the rows
    went through the generic kernel)."""
    from tinyinfer_amd.ops import kernels
    ops.attention(ctx, view, q, pool, out, heads, kv_heads, head_dim, scale, window)
    return head_dim in kernels.SERVED_HEAD_DIMS and pool.shape[3] % 16 == 0


@pytest.fixture(scope="module")
def ops():
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.ops.kernels import get_ops
    return get_ops()


def dev(t):
    return t.to("cuda")


def f64(t):
    return t.detach().to("cpu", torch.float64)


# ------------------------------------------------------------------ embedding
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embed(ops, dtype):
    g = torch.Generator().manual_seed(5)
    V, H, M = 301, 72, 9
    table = torch.randn(V, H, generator=g).to(DT[dtype])
    tok = torch.randint(0, V, (M,), generator=g, dtype=torch.int32)
    x = torch.full((M, H), 7.0, device="cuda")
    ops.embed(dev(table), dev(tok), x)
    assert torch.equal(x.cpu(), table.float()[tok.long()])


# -------------------------------------------------------------------- RMSNorm
def ref_rmsnorm(x, w, eps):
    x = f64(x)
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * f64(w)


def test_rmsnorm_reference_vector(ops):
    """n=1024, rows=3, U(-1,1), eps 1e-6, tolerance 1e-4: src/selftest.cpp:74-100."""
    g = torch.Generator().manual_seed(2)
    x = torch.rand(3, 1024, generator=g) * 2 - 1
    w = torch.rand(1024, generator=g) * 2 - 1
    out = torch.empty(3, 1024, device="cuda")
    ops.rmsnorm(dev(x), dev(w), 1e-6, out)
    assert (f64(out) - ref_rmsnorm(x, w, 1e-6)).abs().max() < 1e-4


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H", [4100, 5120, 8192, 8196, 17000])
def test_rmsnorm_wide_rows(ops, dtype, H):
    """Rows wider than 4,096 take a workgroup per row: whole, gathered, with one element that dominates."""
    g = torch.Generator().manual_seed(H)
    x = torch.randn(7, H, generator=g) * 2
    x[3, H - 1] = 300.0
    w = 1 + 0.1 * torch.randn(H, generator=g)
    rows = torch.tensor([6, 3, 3, 0], dtype=torch.int32)
    out = torch.empty(7, H, device="cuda", dtype=DT[dtype])
    ops.rmsnorm(dev(x), dev(w), 1e-6, out)
    ref = ref_rmsnorm(x, w, 1e-6)
    # bfloat16 keeps 8 bits: half a unit in the last place is 2^-9 of the value (the dominant element is ~60)
    allowed = 1e-5 * (1 + ref.abs()) if dtype == "float32" else 2.0 ** -8 * ref.abs() + 1e-3
    assert bool(((f64(out) - ref).abs() <= allowed).all())
    some = torch.empty(4, H, device="cuda", dtype=DT[dtype])
    ops.rmsnorm(dev(x), dev(w), 1e-6, some, dev(rows))
    assert torch.equal(some, out[rows.long()])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rmsnorm_gather_odd_width(ops, dtype):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(11, 100, generator=g) * 3
    w = 1 + 0.1 * torch.randn(100, generator=g)
    rows = torch.tensor([10, 0, 3, 3], dtype=torch.int32)
    out = torch.empty(4, 100, device="cuda", dtype=DT[dtype])
    ops.rmsnorm(dev(x), dev(w), 1e-5, out, dev(rows))
    ref = ref_rmsnorm(x[rows.long()], w, 1e-5)
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert (f64(out) - ref).abs().max() < tol


def test_rmsnorm_eps_inside_root(ops):
    """Tiny inputs tell rsqrt(mean + eps) from 1/(rms + eps)."""
    x = torch.full((1, 64), 1e-4)
    w = torch.ones(64)
    out = torch.empty(1, 64, device="cuda")
    ops.rmsnorm(dev(x), dev(w), 1e-6, out)
    want = 1e-4 / math.sqrt(1e-8 + 1e-6)
    assert abs(out[0, 0].item() - want) < 1e-6
    assert abs(out[0, 0].item() - 1e-4 / (1e-4 + 1e-6)) > 0.5


# ----------------------------------------------------------------------- rope
def ref_rope(x, pos, theta):
    x = f64(x)
    hd = x.shape[-1]
    half = hd // 2
    k = torch.arange(half, dtype=torch.float64)
    ang = torch.tensor(pos, dtype=torch.float64)[:, None] * theta ** (-2.0 * k / hd)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return torch.cat([lo * c - hi * s, lo * s + hi * c], -1)


def inv_freq(hd, theta):
    k = torch.arange(hd // 2, dtype=torch.float64)
    return (theta ** (-2.0 * k / hd)).to(torch.float32)


def test_rope_reference_vector(ops):
    """rows=2, heads=4, hd=128, theta=1e6, positions {0,5}, tolerance 1e-4: src/selftest.cpp:102-134."""
    g = torch.Generator().manual_seed(3)
    x = torch.rand(2, 4, 128, generator=g) * 2 - 1
    xd = dev(x.clone())
    ops.rope_neox(xd, dev(torch.tensor([0, 5], dtype=torch.int32)), dev(inv_freq(128, 1e6)))
    ref = ref_rope(x, [0, 5], 1e6)
    assert (f64(xd) - ref).abs().max() < 1e-4
    assert torch.equal(xd[0].cpu(), x[0])           # position 0 is the identity


def test_rope_pairs_are_half_split(ops):
    """Only pair (k, k + hd/2) mixes: a one-hot at dim 1 spreads to dims 1 and 1 + hd/2."""
    x = torch.zeros(1, 1, 16)
    x[0, 0, 1] = 1.0
    xd = dev(x.clone())
    ops.rope_neox(xd, dev(torch.tensor([3], dtype=torch.int32)), dev(inv_freq(16, 100.0)))
    nz = set(torch.nonzero(xd[0, 0].cpu().abs() > 1e-7).flatten().tolist())
    assert nz == {1, 9}


# ------------------------------------------------- qk norm + rope + cache write
class View:
    def __init__(self, table):
        self.table = table


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("table_len", [None, 7, 64])
@pytest.mark.parametrize("hd,nh,nkv,P", [(48, 3, 3, 4), (128, 4, 2, 16), (16, 6, 2, 8), (256, 1, 1, 16)])
def test_qk_norm_rope_kv_write(ops, dtype, hd, nh, nkv, P, table_len):
    """With a sin/cos table that covers all, some (positions 0..6) or none of the positions."""
    g = torch.Generator().manual_seed(11)
    M, pages, W = 7, 9, 5
    eps, theta = 1e-5, 3e4
    width = (nh + 2 * nkv) * hd
    qkv = torch.randn(M, width, generator=g)
    qw = 1 + 0.1 * torch.randn(hd, generator=g)
    kw = 1 + 0.1 * torch.randn(hd, generator=g)
    # two requests: rows 0..3 are request 0 at positions 5..8, rows 4..6 request 1 at 0..2
    pos = torch.tensor([5, 6, 7, 8, 0, 1, 2], dtype=torch.int32)
    slot = torch.tensor([0, 0, 0, 0, 1, 1, 1], dtype=torch.int32)
    table = torch.full((2, W), -1, dtype=torch.int32)
    table[0, :3] = torch.tensor([7, 2, 5])[: 3]
    table[1, :1] = 4
    need0 = 8 // P + 1
    assert need0 <= 3
    pool = torch.zeros(pages, 2, nkv, P, hd, dtype=DT[dtype], device="cuda")
    q_out = torch.empty(M, nh * hd, dtype=DT[dtype], device="cuda")
    freqs = dev(inv_freq(hd, theta))
    rope_table = None if table_len is None else ops.rope_table(freqs, table_len)
    ops.qk_norm_rope_kv_write(dev(qkv), dev(qw), dev(kw), eps, freqs, dev(pos), dev(slot),
                              View(dev(table)), pool, q_out, nh, nkv, hd, rope_table)
    q = qkv[:, :nh * hd].reshape(M, nh, hd)
    k = qkv[:, nh * hd:(nh + nkv) * hd].reshape(M, nkv, hd)
    v = qkv[:, (nh + nkv) * hd:].reshape(M, nkv, hd)
    q_ref = ref_rope(ref_rmsnorm(q, qw, eps), pos.tolist(), theta).reshape(M, -1)
    k_ref = ref_rope(ref_rmsnorm(k, kw, eps), pos.tolist(), theta)
    tol = 2e-5 if dtype == "float32" else 3e-2
    assert (f64(q_out) - q_ref).abs().max() < tol
    pool_c = f64(pool)
    touched = torch.zeros(pages, P, dtype=torch.bool)
    for m in range(M):
        page = table[slot[m], pos[m] // P].item()
        r = pos[m].item() % P
        touched[page, r] = True
        assert (pool_c[page, 0, :, r, :] - k_ref[m]).abs().max() < tol
        vt = pool_c[page, 1].reshape(nkv, hd, P)              # values lie transposed in a page: [head][d][row]
        assert (vt[:, :, r] - f64(v[m])).abs().max() < (1e-7 if dtype == "float32" else 2e-2)
    # nothing else was written
    keys = pool_c[:, 0]                                        # [pages, nkv, P, hd]
    vals = pool_c[:, 1].reshape(pages, nkv, hd, P).transpose(2, 3)
    mask = ~touched[:, None, :, None].expand(pages, nkv, P, hd)
    assert keys[mask].abs().max() == 0 and vals[mask].abs().max() == 0


# -------------------------------------------------------------- matrix products
def test_qk_norm_in_place(ops):
    """The per-head norm alone, in place on 32-bit projections: the same numbers as the fused
    kernel produces without rotation, value heads untouched, a missing weight leaves heads alone."""
    g = torch.Generator().manual_seed(12)
    M, nh, nkv, hd = 7, 3, 2, 48
    qkv = torch.randn(M, (nh + 2 * nkv) * hd, generator=g) * 2
    q_w, k_w = 1 + 0.1 * torch.randn(hd, generator=g), 1 + 0.1 * torch.randn(hd, generator=g)
    x = dev(qkv.clone())
    ops.qk_norm_inplace(x, dev(q_w), dev(k_w), 1e-3, nh, nkv, hd)
    want = f64(qkv).clone()
    for u in range(nh + nkv):
        h = want[:, u * hd:(u + 1) * hd]
        w = f64(q_w) if u < nh else f64(k_w)
        want[:, u * hd:(u + 1) * hd] = h / torch.sqrt((h * h).mean(-1, keepdim=True) + 1e-3) * w
    assert (f64(x) - want).abs().max() < 1e-5
    assert torch.equal(x[:, (nh + nkv) * hd:].cpu(), qkv[:, (nh + nkv) * hd:])
    y = dev(qkv.clone())
    ops.qk_norm_inplace(y, None, dev(k_w), 1e-3, nh, nkv, hd)
    assert torch.equal(y[:, :nh * hd].cpu(), qkv[:, :nh * hd])
    assert torch.equal(y[:, nh * hd:], x[:, nh * hd:])


def ref_linear(a, w):
    return f64(a) @ f64(w).T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,K", [(5, 261, 1024), (70, 130, 50), (1, 17, 33), (130, 64, 96)])
def test_linear_generic_all_epilogues(ops, dtype, M, N, K):
    """(5, 261, 1024) with U(-1,1) rounded to bfloat16 is the reference's own
    case: src/selftest.cpp:33-72."""
    g = torch.Generator().manual_seed(1)
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(DT[dtype])
    w = (torch.rand(N, K, generator=g) * 2 - 1).to(DT[dtype])
    fast = ops.use_fast_gemm
    ops.use_fast_gemm = False
    try:
        ref = ref_linear(a, w)
        tol = 1e-4 * math.sqrt(K) if dtype == "float32" else 1e-4 * math.sqrt(K)
        out = torch.empty(M, N, device="cuda")
        ops.linear(dev(a), dev(w), out, "store")
        assert (f64(out) - ref).abs().max() < tol
        base = torch.randn(M, N, generator=g)
        out = dev(base.clone())
        ops.linear(dev(a), dev(w), out, "add")
        assert (f64(out) - (ref + f64(base))).abs().max() < tol
        out = torch.empty(M, N, device="cuda", dtype=DT[dtype])
        ops.linear(dev(a), dev(w), out, "store_act")
        assert (f64(out) - ref).abs().max() < (tol if dtype == "float32" else 0.01 * ref.abs().max())
        if N % 2 == 0:
            F = N // 2
            out = torch.empty(M, F, device="cuda", dtype=DT[dtype])
            ops.linear(dev(a), dev(w), out, "swiglu")
            gte, up = ref[:, :F], ref[:, F:]
            want = gte / (1 + torch.exp(-gte)) * up
            assert (f64(out) - want).abs().max() < (10 * tol if dtype == "float32" else 0.01 * want.abs().max() + 1e-3)
    finally:
        ops.use_fast_gemm = fast


def test_linear_identity_and_strided_rows(ops):
    """W = I copies; rows of A may be strided (a slice of a wider buffer)."""
    g = torch.Generator().manual_seed(2)
    wide = torch.randn(6, 40, generator=g)
    a = dev(wide)[:, 8:24]
    out = torch.empty(6, 16, device="cuda")
    ops.linear(a, dev(torch.eye(16)), out, "store")
    assert torch.equal(out.cpu(), wide[:, 8:24])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_linear_rows_do_not_depend_on_the_batch(ops, dtype):
    """Row m of the result is the same bits whether it is computed alone or among others."""
    g = torch.Generator().manual_seed(4)
    a = torch.randn(37, 200, generator=g).to(DT[dtype])
    w = torch.randn(150, 200, generator=g).to(DT[dtype])
    fast = ops.use_fast_gemm
    ops.use_fast_gemm = False
    try:
        full = torch.empty(37, 150, device="cuda")
        ops.linear(dev(a), dev(w), full, "store")
        one = torch.empty(1, 150, device="cuda")
        for m in (0, 17, 36):
            ops.linear(dev(a[m:m + 1].contiguous()), dev(w), one, "store")
            assert torch.equal(one[0], full[m])
    finally:
        ops.use_fast_gemm = fast


# ------------------------------------------------------------------ attention
def ref_attention(q, k, v, scale, window=None):
    """q [T, nh, hd], k/v [T, nkv, hd], causal, float64."""
    q, k, v = f64(q), f64(k), f64(v)
    T, nh, hd = q.shape
    G = nh // k.shape[1]
    out = torch.zeros(T, nh, hd, dtype=torch.float64)
    for h in range(nh):
        s = (q[:, h] @ k[:, h // G].T) * scale
        i = torch.arange(T)
        mask = i[None, :] > i[:, None]
        if window is not None:
            mask |= i[None, :] <= i[:, None] - window
        s = s.masked_fill(mask, float("-inf"))
        out[:, h] = torch.softmax(s, -1) @ v[:, h // G]
    return out


def paged_case(dtype, T, nh, nkv, hd, P, seed, sharp=1.0):
    """One request of T tokens whose pages are scattered over a larger pool."""
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(T, nh, hd, generator=g) * sharp).to(DT[dtype])
    k = torch.randn(T, nkv, hd, generator=g).to(DT[dtype])
    v = torch.randn(T, nkv, hd, generator=g).to(DT[dtype])
    n_pages = -(-T // P)
    pages = n_pages + 5
    perm = torch.randperm(pages, generator=g)[:n_pages]
    pool = torch.randn(pages, 2, nkv, P, hd, generator=g).to(DT[dtype]) * 50    # stale rubbish everywhere
    vt = pool[:, 1].reshape(pages, nkv, hd, P)                 # values lie transposed in a page
    for t in range(T):
        pool[perm[t // P], 0, :, t % P] = k[t]
        vt[perm[t // P], :, :, t % P] = v[t]
    table = torch.full((2, n_pages + 2), -1, dtype=torch.int32)
    table[1, :n_pages] = perm.to(torch.int32)
    return q, k, v, pool, table


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T,nh,nkv,hd,P,window", [
    (37, 4, 2, 64, 16, None), (70, 6, 2, 32, 4, None), (50, 5, 5, 48, 8, 13), (33, 2, 1, 256, 16, None),
    (300, 4, 4, 16, 16, 64)])
def test_attention_rows_against_softmax(ops, dtype, T, nh, nkv, hd, P, window):
    q, k, v, pool, table = paged_case(dtype, T, nh, nkv, hd, P, seed=T + hd, sharp=2.0)
    scale = 1.0 / math.sqrt(hd)
    out = torch.empty(T, nh * hd, dtype=DT[dtype], device="cuda")
    pos = torch.arange(T, dtype=torch.int32)
    slot = torch.ones(T, dtype=torch.int32)
    ops.attention_rows(dev(q.reshape(T, -1)), dev(pool), dev(table), dev(pos), dev(slot), out, nh, nkv, hd,
                       scale, window)
    ref = ref_attention(q, k, v, scale, window).reshape(T, -1)
    tol = 2e-5 if dtype == "float32" else 2e-2
    assert (f64(out) - ref).abs().max() < tol


def test_attention_single_key_returns_its_value(ops):
    """One position: the output is V_0 exactly; and q = 0 gives the mean of the values."""
    q, k, v, pool, table = paged_case("float32", 5, 2, 1, 32, 4, seed=9)
    out = torch.empty(5, 64, device="cuda")
    pos = torch.arange(5, dtype=torch.int32)
    slot = torch.ones(5, dtype=torch.int32)
    ops.attention_rows(dev(q.reshape(5, -1)), dev(pool), dev(table), dev(pos), dev(slot), out, 2, 1, 32, 0.3, None)
    assert torch.equal(out[0, :32].cpu(), v[0, 0])
    ops.attention_rows(dev(torch.zeros(5, 64)), dev(pool), dev(table), dev(pos), dev(slot), out, 2, 1, 32, 0.3, None)
    assert (f64(out[4, :32]) - f64(v[:5, 0]).mean(0)).abs().max() < 1e-6


def test_attention_far_key_among_hundreds(ops):
    """One key far back carries almost all the weight: a kernel that skips or
    misplaces it (a page edge, a split boundary) gives a different row."""
    T, hd, P = 700, 64, 16
    g = torch.Generator().manual_seed(21)
    k = torch.randn(T, 1, hd, generator=g) * 0.1
    v = torch.randn(T, 1, hd, generator=g)
    q = torch.randn(T, 1, hd, generator=g) * 0.1
    far = 17                      # second row of the second page
    k[far, 0] = 0
    k[far, 0, 3] = 30.0
    q[-1, 0, 3] = 30.0
    n_pages = -(-T // P)
    pool = torch.zeros(n_pages, 2, 1, P, hd)
    vt = pool[:, 1].reshape(n_pages, 1, hd, P)
    for t in range(T):
        pool[t // P, 0, 0, t % P] = k[t, 0]
        vt[t // P, 0, :, t % P] = v[t, 0]
    table = torch.arange(n_pages, dtype=torch.int32)[None, :].contiguous()
    out = torch.empty(T, hd, device="cuda")
    ops.attention_rows(dev(q.reshape(T, -1)), dev(pool), dev(table), dev(torch.arange(T, dtype=torch.int32)),
                       dev(torch.zeros(T, dtype=torch.int32)), out, 1, 1, hd, 1.0 / 8, None)
    assert (f64(out[-1]) - f64(v[far, 0])).abs().max() < 1e-4


# ------------------------------------------------------------------- sampling
def test_argmax_lowest_index_wins(ops):
    """Ties go to the lowest index: src/cuda/sample.cu:5-11."""
    V = 5000
    logits = torch.zeros(3, V)
    logits[0, 4000] = logits[0, 123] = logits[0, 124] = 2.5
    logits[1] = -1.0
    logits[2, V - 1] = 9.0
    out = torch.empty(3, dtype=torch.int32, device="cuda")
    ops.argmax(dev(logits), out)
    assert out.tolist() == [123, 0, V - 1]
    g = torch.Generator().manual_seed(0)
    r = torch.randn(6, 151936, generator=g)
    out = torch.empty(6, dtype=torch.int32, device="cuda")
    ops.argmax(dev(r), out)
    assert out.tolist() == r.argmax(-1).tolist()


def run_sample(ops, logits, temp, top_k, top_p, u):
    n = logits.shape[0]
    out = torch.empty(n, dtype=torch.int32, device="cuda")
    ops.sample(dev(logits), dev(torch.full((n,), temp)), dev(torch.full((n,), top_k, dtype=torch.int32)),
               dev(torch.full((n,), top_p)), dev(torch.tensor(u, dtype=torch.float32)), out)
    return out.tolist()


def test_sample_limits_reduce_to_argmax(ops):
    g = torch.Generator().manual_seed(1)
    logits = torch.randn(8, 777, generator=g) * 3
    u = [0.05, 0.2, 0.35, 0.5, 0.65, 0.8, 0.95, 0.999]
    want = logits.argmax(-1).tolist()
    assert run_sample(ops, logits, 0.0, 0, 1.0, u) == want           # temperature 0: greedy
    assert run_sample(ops, logits, 1e-3, 0, 1.0, u) == want          # T -> 0+
    assert run_sample(ops, logits, 1.0, 1, 1.0, u) == want           # top-k = 1
    assert run_sample(ops, logits, 1.0, 0, 1e-6, u) == want          # top-p -> 0


def test_sample_keeps_every_logit_equal_to_the_kth(ops):
    """Equal logits at the cut: top-k keeps every logit that is no smaller than the k-th largest, so the kept
    set may hold more than k (the reference's nth_element picks among equals arbitrarily and keeps exactly k:
    /root/reference/src/main.cpp:47-53; which of the equals it keeps is not defined, so parity is unpinned
    there).  With logits [1, 3, 2, 2, 2, 0] and k = 2 the kept set is {1, 2, 3, 4}: weights e^1 : 1 : 1 : 1 at
    T = 1, and a uniform number near the end of [0, 1) draws index 4, which a cut to exactly two would never do."""
    row = torch.tensor([[1.0, 3.0, 2.0, 2.0, 2.0, 0.0]])
    e = math.e
    edges = [e / (e + 3), (e + 1) / (e + 3), (e + 2) / (e + 3)]
    u = [0.01, edges[0] - 0.01, edges[0] + 0.01, edges[1] + 0.01, edges[2] + 0.01, 0.999]
    got = run_sample(ops, row.repeat(len(u), 1), 1.0, 2, 1.0, u)
    assert got == [1, 1, 2, 3, 4, 4]
    # and the plain sampler says the same
    from plain.qwen3_plain import sample_distribution, draw
    p = sample_distribution(row[0].double().numpy(), 1.0, 2, 1.0)
    assert [draw(p, x) for x in u] == got
    # -0 and +0 are equal logits too: a cut to the largest keeps both, by radix and by the walk
    zeros = torch.tensor([[-1.0, -0.0, -2.0, 0.0, -3.0] + [-5.0] * 20])
    for radix in (True, False):
        ops.use_radix_sample = radix
        try:
            assert run_sample(ops, zeros.repeat(4, 1), 1.0, 1, 1.0, [0.1, 0.4, 0.6, 0.9]) == [1, 1, 3, 3]
            assert run_sample(ops, zeros.repeat(2, 1), 0.0, 0, 1.0, [0.1, 0.9]) == [1, 1]      # greedy: the lowest index
        finally:
            ops.use_radix_sample = True


def test_sample_matches_inverse_cdf(ops):
    """The draw is the inverse CDF of softmax(l/T) over the index order at u."""
    from plain.qwen3_plain import sample_distribution
    g = torch.Generator().manual_seed(2)
    V, T = 300, 0.8
    row = torch.randn(V, generator=g) * 2
    us = np.linspace(0.001, 0.999, 64).astype(np.float32)
    logits = row[None, :].repeat(64, 1)
    for top_k, top_p in ((V, 1.0), (10, 1.0), (V, 0.7), (25, 0.9)):
        got = run_sample(ops, logits, T, top_k, top_p, us.tolist())
        p = sample_distribution(row.numpy(), T, top_k, top_p)
        c = np.cumsum(p)
        kept = np.nonzero(p)[0]
        for u, tok in zip(us, got):
            assert p[tok] > 0, (top_k, top_p, u, tok)
            lo = c[tok] - p[tok]
            # u must fall into tok's interval, up to 32-bit rounding of the running sum
            assert lo - 1e-4 <= u <= c[tok] + 1e-4, (top_k, top_p, u, tok, lo, c[tok])
        assert set(got) <= set(kept.tolist())


def test_sample_frequencies(ops):
    """Many draws with uniform u reproduce softmax(l/T) (chi-square, tiny vocabulary)."""
    rng = np.random.default_rng(3)
    V, n, T = 12, 4096, 1.3
    row = torch.tensor(rng.normal(size=V) * 1.5, dtype=torch.float32)
    u = rng.random(n).astype(np.float32)
    got = np.array(run_sample(ops, row[None, :].repeat(n, 1), T, 0, 1.0, u.tolist()))
    p = torch.softmax(row.double() / T, -1).numpy()
    counts = np.bincount(got, minlength=V)
    chi2 = ((counts - n * p) ** 2 / (n * p)).sum()
    assert chi2 < 40.0          # 11 degrees of freedom: P(chi2 > 40) < 4e-5


def check_draws(row, T, top_k, top_p, us, got):
    """Every draw lies in its token's interval of the plain sampler's CDF (32-bit rounding of the running sums aside)."""
    from plain.qwen3_plain import sample_distribution
    p = sample_distribution(row.double().numpy(), T, top_k, top_p)
    c = np.cumsum(p)
    for u, tok in zip(us, got):
        assert 0 <= tok < row.numel() and p[tok] > 0, (T, top_k, top_p, u, tok)
        assert c[tok] - p[tok] - 1e-4 <= u <= c[tok] + 1e-4, (T, top_k, top_p, u, tok, c[tok] - p[tok], c[tok])


def test_sample_of_a_long_row_by_many_workgroups(ops):
    """A row of the real vocabulary's length, whose top-k cut is found by radix with many workgroups a row:
    the draws lie where the plain sampler's CDF puts them, and are those of the one workgroup that walks the
    row bit by bit, for cuts in the positive and in the negative logits, equal logits at the cut, NaN
    in the row and greedy rows beside drawn ones; a second call finds the workspace as the first left it."""
    g = torch.Generator().manual_seed(11)
    V = 151936
    us = np.linspace(0.003, 0.997, 24).astype(np.float32)
    row = torch.randn(V, generator=g) * 3
    row[1000:1040] = row[7]                                  # equal logits, far apart from the first of them
    row[5] = float("nan")
    row[150000] = float("nan")
    low = -row.abs() - 0.5                                   # every logit negative
    low[5] = low[150000] = 0.0
    low[5] = float("nan")
    for r in (row, low):
        logits = dev(r[None, :].repeat(len(us), 1))
        for T, top_k, top_p in ((0.8, 512, 1.0), (1.0, 50, 1.0), (0.7, 512, 0.9), (1.3, 20, 0.95), (1.0, 1, 1.0),
                                (2.0, 3000, 0.999), (1.0, 2, 0.5)):
            got = run_sample(ops, logits, T, top_k, top_p, us.tolist())
            check_draws(r.nan_to_num(nan=-1e30), T, top_k, top_p, us, got)
            ops.use_radix_sample = False
            try:
                walked = run_sample(ops, logits, T, top_k, top_p, us.tolist())
            finally:
                ops.use_radix_sample = True
            differ = sum(a != b for a, b in zip(got, walked))
            assert differ <= 1, (T, top_k, top_p, got, walked)      # a sum taken in another order may move one edge
    # the cut lands in 40 equal logits: all of them stay
    tie = torch.randn(V, generator=g)
    tie[20000:20040] = 4.0
    tie[3] = 9.0
    big = tie > 4.0
    k = int(big.sum()) + 5
    got = run_sample(ops, dev(tie[None, :].repeat(len(us), 1)), 1.0, k, 1.0, us.tolist())
    check_draws(tie, 1.0, k, 1.0, us, got)
    assert any(20000 <= t < 20040 for t in got)
    # rows of different kinds in one call
    n = 6
    logits = torch.randn(n, V, generator=g) * 2
    logits[2] = float("nan")                                 # nothing to draw from: index 0
    logits[3, :] = 1.5                                       # all equal: every index stays, far more than are collected
    temp = torch.tensor([0.0, 1.0, 1.0, 1.0, 0.0, 0.9])
    top_k = torch.tensor([7, 40, 40, 40, 0, 3500], dtype=torch.int32)
    top_p = torch.tensor([1.0, 0.8, 1.0, 1.0, 1.0, 0.97])
    u = torch.tensor([0.5, 0.31, 0.9, 0.25, 0.1, 0.77])
    out = torch.empty(n, dtype=torch.int32, device="cuda")
    for _ in range(2):
        ops.sample(dev(logits), dev(temp), dev(top_k), dev(top_p), dev(u), out)
        got = out.tolist()
        assert got[0] == int(logits[0].argmax()) and got[4] == int(logits[4].argmax())
        assert got[2] == 0
        assert got[3] == int(0.25 * V)
        check_draws(logits[1], 1.0, 40, 0.8, [0.31], [got[1]])
        check_draws(logits[5], 0.9, 3500, 0.97, [0.77], [got[5]])
    # a cut beyond what the radix kernels hold goes the long way, with the same meaning
    got = run_sample(ops, dev(row[None, :].repeat(4, 1)), 1.0, 5000, 1.0, us[:4].tolist())
    check_draws(row.nan_to_num(nan=-1e30), 1.0, 5000, 1.0, us[:4], got)


def test_sample_with_more_equal_logits_at_the_cut_than_are_collected(ops):
    """6,000 equal logits at the cut are more pairs than a row collects: the row is walked instead, and the
    next call, which is served, finds the workspace clean."""
    g = torch.Generator().manual_seed(12)
    V = 40000
    row = torch.randn(V, generator=g)
    row[10000:16000] = 2.0
    us = np.linspace(0.01, 0.99, 16).astype(np.float32)
    k = int((row > 2.0).sum()) + 10
    got = run_sample(ops, dev(row[None, :].repeat(16, 1)), 1.0, k, 1.0, us.tolist())
    check_draws(row, 1.0, k, 1.0, us, got)
    got = run_sample(ops, dev(row[None, :].repeat(16, 1)), 1.0, 30, 1.0, us.tolist())
    check_draws(row, 1.0, 30, 1.0, us, got)


# ------------------------------------------------- bfloat16 matrix-core products
@pytest.mark.parametrize("M,N,K", [
    (1, 48, 64), (5, 261, 1024), (8, 1000, 96), (16, 17, 200), (17, 130, 72), (33, 64, 3072), (64, 151, 256),
    (65, 130, 96), (128, 128, 32), (200, 261, 1024), (300, 520, 104), (77, 1000, 1032),
    (300, 520, 128), (257, 384, 192), (513, 200, 64), (1000, 1100, 320), (2048, 96, 1024)])
def test_linear_bf16_matrix_cores(ops, M, N, K):
    """The skinny (M <= 64) and tiled (M > 64) MFMA kernels against float64, every
    epilogue, at sizes that are no multiples of their tiles.  (5, 261, 1024) is the
    reference's own case, src/selftest.cpp:33-72."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(M * 7 + N)
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16)
    w = (torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16)
    ref = ref_linear(a, w)
    tol = 2e-5 * K                         # 32-bit accumulation of K products of size <= 1
    out = torch.empty(M, N, device="cuda")
    ops.linear(dev(a), dev(w), out, "store")
    assert (f64(out) - ref).abs().max() < tol
    base = torch.randn(M, N, generator=g)
    out = dev(base.clone())
    ops.linear(dev(a), dev(w), out, "add")
    assert (f64(out) - (ref + f64(base))).abs().max() < tol
    out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    ops.linear(dev(a), dev(w), out, "store_act")
    assert (f64(out) - ref).abs().max() < 0.005 * ref.abs().max() + tol
    if N % 2 == 0:
        F = N // 2
        out = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
        ops.linear(dev(a), dev(w), out, "swiglu")
        gte, up = ref[:, :F], ref[:, F:]
        want = gte / (1 + torch.exp(-gte)) * up
        assert (f64(out) - want).abs().max() < 0.005 * want.abs().max() + 10 * tol


@pytest.mark.parametrize("seed", [1, 2])
def test_linear_bf16_random_sizes(ops, seed):
    """Sixty products drawn from a seed, whichever kernel the sizes lead to: token rows from 1 to 2,100
    (around every border between kernels: 8, 12, 16, 64, 128, 256), weights from 2 to 12,288 rows, K from
    8 to 9,728, every epilogue, and a row behind the output that must stay as it was."""
    import random
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    rnd = random.Random(seed)
    for case in range(60):
        M = rnd.choice([1, 2, 3, 5, 8, 9, 12, 13, 16, 17, 31, 32, 33, 48, 63, 64, 65, 100, 127, 128, 129, 255, 256,
                        257, 300, 511, 777, 1024, 2048, 2100])
        N = rnd.choice([2, 6, 16, 34, 64, 130, 160, 256, 320, 522, 1000, 1024, 1280, 2048, 3072, 4096, 4100, 6144,
                        8192, 9728, 12288])
        K = 8 * rnd.choice([1, 2, 3, 4, 8, 9, 13, 16, 24, 32, 33, 64, 96, 128, 129, 256, 320, 384, 512, 640, 1024, 1216])
        if M * N > 2100 * 4100 * 2 or N * K > 12288 * 5120:
            continue
        what = f"case {case}: {M} rows, weight {N} x {K}"
        g = torch.Generator().manual_seed(seed * 1000 + case)
        a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
        w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
        ref = (a.double() @ w.double().T).cpu()
        tol = 2e-5 * K
        out = torch.full((M + 1, N), 7.0, device="cuda")
        ops.linear(a, w, out[:M], "store")
        assert (f64(out[:M]) - ref).abs().max() < tol, what
        assert bool((out[M] == 7.0).all()), what
        base = torch.randn(M, N, generator=g)
        acc = dev(base.clone())
        ops.linear(a, w, acc, "add")
        assert (f64(acc) - (ref + f64(base))).abs().max() < tol, what
        out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
        ops.linear(a, w, out, "store_act")
        assert (f64(out) - ref).abs().max() < 0.005 * ref.abs().max() + tol, what
        F = N // 2
        out = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
        ops.linear(a, w, out, "swiglu")
        gte, up = ref[:, :F], ref[:, F:]
        want = gte / (1 + torch.exp(-gte)) * up
        assert (f64(out) - want).abs().max() < 0.005 * want.abs().max() + 10 * tol, what


@pytest.mark.parametrize("M,N,K", [(1, 1, 8), (1, 1024, 2048), (8, 1024, 3072), (3, 7, 4096), (2, 4095, 520),
                                   (4, 33, 1032), (8, 5, 24), (5, 1000, 2056), (7, 130, 3080)])
def test_linear_bf16_weight_row_per_wavefront(ops, M, N, K):
    """Up to 8 tokens and a weight of fewer than 4,096 rows: the kernel with a weight row per
    wavefront, at the edges of what it serves (one row, one piece of K, the longest K, every
    template variant of M and K), with strided token rows, against float64 and against the
    kernels that take these sizes when it is switched off (same values up to rounding)."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(M * 11 + N + K)
    wide = (torch.rand(M, K + 24, generator=g) * 2 - 1).to(torch.bfloat16)
    a = dev(wide)[:, 8:8 + K]                                    # rows 16 bytes into a wider matrix
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    ref = ref_linear(wide[:, 8:8 + K], w.cpu())
    tol = 2e-5 * K
    lib = ops.lib("gemm_bf16")
    base = torch.randn(M, N, generator=g)
    results = {}
    try:
        for on in (1, 0):
            lib.ti_tuning_set(b"row_per_wave", on)
            out = torch.full((M + 1, N), 7.0, device="cuda")     # a row beyond: must stay untouched
            ops.linear(a, w, out[:M], "store")
            assert (f64(out[:M]) - ref).abs().max() < tol
            assert bool((out[M] == 7.0).all())
            acc = dev(base.clone())
            ops.linear(a, w, acc, "add")
            assert (f64(acc) - (ref + f64(base))).abs().max() < tol
            results[on] = (out[:M].clone(), acc)
        # the token rows straight into registers (up to K = 3,072 at 8 tokens) or through LDS: the same bits
        lib.ti_tuning_set(b"row_per_wave", 1)
        lib.ti_tuning_set(b"rows_direct", 0)
        through_lds = torch.empty(M, N, device="cuda")
        ops.linear(a, w, through_lds, "store")
        assert torch.equal(through_lds, results[1][0])
        acc = dev(base.clone())
        ops.linear(a, w, acc, "add")
        assert torch.equal(acc, results[1][1])
    finally:
        lib.ti_tuning_set(b"row_per_wave", 1)
        lib.ti_tuning_set(b"rows_direct", 1)
    assert (results[1][0] - results[0][0]).abs().max() < tol
    # a row's bits do not depend on the rows beside it
    if M > 1:
        one = torch.empty(1, N, device="cuda")
        ops.linear(a[M - 1:M], w, one, "store")
        assert torch.equal(one[0], results[1][0][M - 1])


@pytest.mark.parametrize("M,N,K,ks", [(1, 16, 64, 1), (17, 1024, 2048, 4), (64, 1024, 3072, 8), (33, 50, 256, 3),
                                      (48, 7, 128, 2), (5, 40, 192, 1), (64, 130, 1024, 5)])
def test_linear_bf16_mfma_fed_from_memory(ops, M, N, K, ks):
    """The kernel for 17 to 64 rows alone (16x16x32 MFMAs whose operands come straight from
    memory), through its test entry point: every epilogue, 1 to 4 blocks of 16 rows, columns that
    do not fill a tile, K split over workgroups with the partial sums added afterwards, strided
    rows; against float64.  A row's bits do not depend on the rows beside it."""
    import ctypes
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    lib = ops.lib("gemm_bf16")
    g = torch.Generator().manual_seed(M * 7 + N + K + ks)
    wide = (torch.rand(M, K + 24, generator=g) * 2 - 1).to(torch.bfloat16)
    a = dev(wide)[:, 8:8 + K]
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    ref = ref_linear(wide[:, 8:8 + K], w.cpu())
    tol = 2e-5 * K
    partial = torch.empty(ks * M * N, device="cuda")

    def run(rows, out, epi, splits=1):
        ptr = lambda t: ctypes.c_void_p(t.data_ptr())
        rc = lib.ti_gemm_bf16_mblocks_any(ptr(rows), ptr(w), ptr(out), rows.shape[0], out.shape[1], K,
                                          ctypes.c_long(rows.stride(0)), epi, ptr(partial), splits, None)
        assert rc == 0, lib.ti_last_error()
    out = torch.full((M + 1, N), 7.0, device="cuda")
    run(a, out[:M], 0)
    assert (f64(out[:M]) - ref).abs().max() < tol
    assert bool((out[M] == 7.0).all())
    one = torch.empty(1, N, device="cuda")
    run(a[M - 1:M], one, 0)
    assert torch.equal(one[0], out[M - 1])
    base = torch.randn(M, N, generator=g)
    for splits in sorted({1, ks}):
        acc = dev(base.clone())
        run(a, acc, 1, splits)
        assert (f64(acc) - (ref + f64(base))).abs().max() < tol
    act = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    run(a, act, 2)
    assert (f64(act) - ref).abs().max() < 0.005 * ref.abs().max() + tol
    if N % 2 == 0:
        F = N // 2
        sw = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
        run(a, sw, 3)
        gte, up = ref[:, :F], ref[:, F:]
        want = gte / (1 + torch.exp(-gte)) * up
        assert (f64(sw) - want).abs().max() < 0.005 * want.abs().max() + 10 * tol


@pytest.mark.parametrize("M,N,K,ks", [(1, 16, 64, 1), (8, 1024, 5120, 3), (16, 50, 2048, 2), (5, 40, 1088, 1), (13, 7, 4160, 5),
                                      (3, 130, 3072, 2), (16, 260, 8192, 4), (2, 48, 25600, 6)])
def test_linear_bf16_token_rows_in_pieces(ops, M, N, K, ks):
    """The kernel for up to 16 rows that takes the token rows through LDS in pieces of 1,024 columns while the
    next piece's weights are on their way, alone through its test entry point: every epilogue, a K of one
    piece, of several and of several and a part, columns that do not fill a tile, K split over workgroups
    (also into more workgroups than some have pieces for), strided rows; against float64.  A row's bits do
    not depend on the rows beside it, and with K in one workgroup they are the bits of the kernels that take
    all of K into LDS at once."""
    import ctypes
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    lib = ops.lib("gemm_bf16")
    g = torch.Generator().manual_seed(M * 7 + N + K + ks)
    wide = (torch.rand(M, K + 24, generator=g) * 2 - 1).to(torch.bfloat16)
    a = dev(wide)[:, 8:8 + K]
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    ref = ref_linear(wide[:, 8:8 + K], w.cpu())
    tol = 2e-5 * K
    split_counts = sorted({1, ks, min(ks + 3, -(-K // 1024))})
    partial = torch.empty(max(split_counts) * M * N, device="cuda")
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())

    def run(rows, out, epi, splits=1):
        assert splits * rows.shape[0] * out.shape[1] <= partial.numel()
        rc = lib.ti_gemm_bf16_pieces_any(ptr(rows), ptr(w), ptr(out), rows.shape[0], out.shape[1], K,
                                         ctypes.c_long(rows.stride(0)), epi, ptr(partial), splits, None)
        assert rc == 0, lib.ti_last_error()
    out = torch.full((M + 1, N), 7.0, device="cuda")
    run(a, out[:M], 0)
    assert (f64(out[:M]) - ref).abs().max() < tol
    assert bool((out[M] == 7.0).all())
    one = torch.empty(1, N, device="cuda")
    run(a[M - 1:M], one, 0)
    assert torch.equal(one[0], out[M - 1])
    # the kernels that hold all of K at once: the same order of summation
    lib.ti_tuning_set(b"pieces", 0)
    lib.ti_tuning_set(b"row_per_wave", 0)
    lib.ti_tuning_set(b"skinny_waves", 4)
    try:
        old = torch.empty(M, N, device="cuda")
        rc = lib.ti_gemm_bf16(ptr(a), ptr(w), ptr(old), M, N, K, ctypes.c_long(a.stride(0)), 0, None)
        assert rc == 0, lib.ti_last_error()
        assert torch.equal(old, out[:M])
    finally:
        lib.ti_tuning_set(b"pieces", 1)
        lib.ti_tuning_set(b"row_per_wave", 1)
        lib.ti_tuning_set(b"skinny_waves", 0)
    base = torch.randn(M, N, generator=g)
    for splits in split_counts:
        acc = dev(base.clone())
        run(a, acc, 1, splits)
        assert (f64(acc) - (ref + f64(base))).abs().max() < tol, splits
    act = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    run(a, act, 2)
    assert (f64(act) - ref).abs().max() < 0.005 * ref.abs().max() + tol
    if N % 2 == 0:
        F = N // 2
        sw = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
        run(a, sw, 3)
        gte, up = ref[:, :F], ref[:, F:]
        want = gte / (1 + torch.exp(-gte)) * up
        assert (f64(sw) - want).abs().max() < 0.005 * want.abs().max() + 10 * tol


@pytest.mark.parametrize("M", [1, 8, 16])
def test_linear_bf16_long_k_split_for_few_rows(ops, M):
    """Up to 16 rows added into a residual through a weight with a long K and few rows (the shape of a
    large model's down projection): K goes to several workgroups; their sums are left to the next norm,
    or added at once, with the same bits; a row's bits do not depend on the rows beside it."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    N, K = 2064, 17408
    g = torch.Generator().manual_seed(M)
    a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    base = torch.randn(M, N, generator=g)
    ref = ref_linear(a.cpu(), w.cpu()) + f64(base)
    x = dev(base.clone())
    ops.linear(a, w, x, "add", may_defer=True)
    assert ops._pending is not None and ops._pending > 1
    ops.flush()
    assert (f64(x) - ref).abs().max() < 2e-5 * K
    at_once = dev(base.clone())
    ops.linear(a, w, at_once, "add")
    assert ops._pending is None
    assert torch.equal(at_once, x)
    one = dev(base[M - 1:M].clone())
    ops.linear(a[M - 1:M], w, one, "add")
    assert torch.equal(one[0], x[M - 1])
    # and the norm that reads such a residual adds the sums on its way
    nw = dev(torch.rand(N, generator=g) + 0.5)
    y = dev(base.clone())
    ops.linear(a, w, y, "add", may_defer=True)
    h = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
    ops.rmsnorm(y, nw, 1e-6, h)
    assert ops._pending is None and torch.equal(y, x)
    h2 = torch.empty_like(h)
    ops.rmsnorm(x, nw, 1e-6, h2)
    assert torch.equal(h, h2)


@pytest.mark.parametrize("M", [17, 33, 64])
@pytest.mark.parametrize("epilogue", ["store", "add", "store_act", "swiglu"])
def test_linear_bf16_large_weight_at_17_to_64_rows(ops, M, epilogue):
    """17 to 64 rows times a weight of 16 Mi elements: from rows x elements = 280 Mi on the tiled
    kernels take the product (their tile partly empty), below that the kernels whose workgroups
    own 16 weight rows.  Both sides of the rule and the rule switched off agree with float64 and
    with one another up to rounding; the adding epilogue with its sums left to a later kernel too."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    N, K = 8192, 2048
    g = torch.Generator().manual_seed(M)
    a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    ref = ref_linear(a.cpu(), w.cpu())
    tol = 2e-5 * K
    base = torch.randn(M, N, generator=g)
    if epilogue == "swiglu":
        gte, up = ref[:, :N // 2], ref[:, N // 2:]
        want = gte / (1 + torch.exp(-gte)) * up
        bound = 0.005 * want.abs().max() + 10 * tol
    elif epilogue == "add":
        want, bound = ref + f64(base), tol
    else:
        want, bound = ref, tol if epilogue == "store" else 0.005 * ref.abs().max() + tol
    lib = ops.lib("gemm_bf16")
    outs = []
    try:
        for rule in (280 << 20, 1 << 60, 0):              # as shipped, never, always
            lib.ti_tuning_set(b"tiled_from", rule)
            if epilogue == "swiglu":
                out = torch.empty(M, N // 2, device="cuda", dtype=torch.bfloat16)
            elif epilogue == "store_act":
                out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
            else:
                out = dev(base.clone())
            ops.linear(a, w, out, epilogue, may_defer=True)
            ops.flush()
            assert (f64(out) - want).abs().max() < bound
            outs.append(f64(out))
    finally:
        lib.ti_tuning_set(b"tiled_from", 280 << 20)
    assert (outs[1] - outs[2]).abs().max() < 2 * bound
    # 17 rows x 16 Mi lie under the rule, 33 and 64 over it
    same_as = outs[1] if M == 17 else outs[2]
    assert torch.equal(outs[0], same_as)


def test_linear_bf16_large_weight_at_13_to_16_rows(ops):
    """13 to 16 rows times a weight of 48 Mi elements with a short K (one piece of the kernel that
    takes the token rows in pieces, which serves a longer K at these row counts): over the rule for
    these row counts (rows x elements of 600 Mi or more), so the tiled kernels take the product and
    a norm in front becomes a kernel of its own; 12 rows stay with the kernels that take the norm
    in.  Against float64, and the rule switched off."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    from tinyinfer_amd.ops.kernels import NormedRows
    N, K = 49152, 1024
    g = torch.Generator().manual_seed(3)
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    nw = dev(torch.rand(K, generator=g) + 0.5)
    lib = ops.lib("gemm_bf16")
    for M in (12, 13, 16):
        x = dev(torch.randn(M, K, generator=g))
        h_ref = ref_rmsnorm(x, nw, 1e-6).to(torch.bfloat16)
        ref = ref_linear(h_ref, w.cpu())
        outs = []
        try:
            for rule in (280 << 20, 1 << 60):
                lib.ti_tuning_set(b"tiled_from", rule)
                h = torch.empty(M, K, device="cuda", dtype=torch.bfloat16)
                out = torch.empty(M, N, device="cuda")
                ops.linear(NormedRows(x, nw, 1e-6, h), w, out, "store")
                assert (f64(out) - ref).abs().max() < 0.01 * ref.abs().max() + 2e-5 * K
                outs.append(out)
        finally:
            lib.ti_tuning_set(b"tiled_from", 280 << 20)
        assert torch.equal(outs[0], outs[1]) == (M == 12), M


@pytest.mark.parametrize("M,N,K", [(17, 16400, 64), (64, 20000, 1024), (40, 16387, 2048), (33, 17000, 192),
                                   (48, 16384, 1088)])
def test_linear_bf16_wide_weight_at_17_to_64_rows(ops, M, N, K):
    """17 to 64 rows times a weight of 16,384 rows or more (the head of a decode step of many
    requests): workgroups that keep their share of the token rows in registers and walk over the
    weight's tiles.  One to four k-blocks per wavefront, four and eight wavefronts, a last tile
    beyond the matrix, strided token rows; against float64 and against the kernels that take the
    product when this one is switched off; a row's bits do not depend on the rows beside it."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(M + N + K)
    wide = (torch.rand(M, K + 24, generator=g) * 2 - 1).to(torch.bfloat16)
    a = dev(wide)[:, 8:8 + K]
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    ref = ref_linear(wide[:, 8:8 + K], w.cpu())
    tol = 2e-5 * K
    lib = ops.lib("gemm_bf16")
    outs = {}
    try:
        for on in (1, 0):
            lib.ti_tuning_set(b"wide_rows", on)
            out = torch.full((M + 1, N), 7.0, device="cuda")
            ops.linear(a, w, out[:M], "store")
            assert (f64(out[:M]) - ref).abs().max() < tol
            assert bool((out[M] == 7.0).all())
            outs[on] = out[:M].clone()
    finally:
        lib.ti_tuning_set(b"wide_rows", 1)
    assert (outs[1] - outs[0]).abs().max() < tol
    fewer = torch.empty(17, N, device="cuda")
    ops.linear(a[M - 17:], w, fewer, "store")
    assert torch.equal(fewer, outs[1][M - 17:])


@pytest.mark.parametrize("M,N,K", [(17, 1024, 2048), (64, 1024, 3072), (40, 512, 1024), (33, 96, 1024),
                                   (20, 2048, 1024), (24, 256, 2048), (136, 1024, 2048), (300, 1000, 3072),
                                   (65, 520, 1024), (512, 1024, 2048), (2048, 1024, 2048), (1100, 1030, 3072)])
def test_partial_sums_left_to_the_next_norm(ops, M, N, K):
    """A product into the residual whose launch would have few tiles (17..64 rows and few columns:
    MFMAs fed from memory; up to ~512 rows: 64 x 64 tiles; a whole prompt times a weight of ~1,024
    rows: 128 x 128 tiles, each shared by two to four workgroups) splits K over workgroups.
    With `may_defer` its partial sums wait for whatever reads the residual next: the norm adds
    them on its way, any other launch (or `flush`) adds them with a kernel of their own.  All
    three give the bits of the product that adds them at once, and match float64."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(M + N + K)
    a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    base = torch.randn(M, N, generator=g)
    nw = dev(torch.rand(N, generator=g) + 0.5)
    ref = ref_linear(a.cpu(), w.cpu()) + f64(base)
    eps = 1e-5

    def product_then_norm(how):
        x = dev(base.clone())
        h = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
        ops.use_deferred_add = how != "at once"
        try:
            ops.linear(a, w, x, "add", may_defer=True)
        finally:
            ops.use_deferred_add = True
        if how == "flush":
            ops.flush()
        if how == "another launch":
            other = torch.empty(M, N, device="cuda")
            ops.linear(a, w, other, "store")              # reads nothing of x, but goes first
            assert ops._pending is None
        if how == "norm":
            assert ops._pending is not None               # these sizes do split K
        ops.rmsnorm(x, nw, eps, h)
        assert ops._pending is None
        return x, h
    want_x, want_h = product_then_norm("at once")
    assert (f64(want_x) - ref).abs().max() < 2e-5 * K
    assert (f64(want_h) - ref_rmsnorm(f64(want_x), f64(nw), eps)).abs().max() < 0.02
    for how in ("norm", "flush", "another launch"):
        x, h = product_then_norm(how)
        assert torch.equal(x, want_x), how
        assert torch.equal(h, want_h), how
    # switched off, the other kernels take these sizes: the same values up to rounding
    try:
        ops.use_split_k_add = False
        x = dev(base.clone())
        ops.linear(a, w, x, "add", may_defer=True)
        assert ops._pending is None
        assert (x - want_x).abs().max() < 2e-5 * K
    finally:
        ops.use_split_k_add = True


@pytest.mark.parametrize("rows,H,KS", [(5, 2304, 3), (3, 1028, 5), (9, 64, 1), (2, 1024, 4), (70, 1536, 2),
                                       (8, 5120, 4), (3, 4100, 2), (2, 8192, 3), (5, 9220, 2), (1, 20480, 1)])
def test_rmsnorm_that_adds_partial_sums(ops, rows, H, KS):
    """The norm that first adds KS partial sums to its rows, alone, at widths and counts that the
    products of the engine do not produce: the rows afterwards are x + p0 + ... in that order
    (bit for bit), and the output is the norm of them, in the bits of the plain norm kernel."""
    import ctypes
    g = torch.Generator().manual_seed(rows + H + KS)
    x0 = torch.randn(rows, H, generator=g)
    parts = torch.randn(KS, rows, H, generator=g)
    w = dev(torch.rand(H, generator=g) + 0.5)
    want_x = x0.clone()
    for s in range(KS):
        want_x += parts[s]
    lib = ops.lib("core")
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    for dtype, code in ((torch.float32, 0), (torch.bfloat16, 1)):
        x = dev(x0.clone())
        out = torch.empty(rows, H, device="cuda", dtype=dtype)
        rc = lib.ti_rmsnorm_add_partials(code, ptr(x), ptr(dev(parts)), KS, ptr(w), ptr(out), rows, H,
                                         ctypes.c_float(1e-6), None)
        assert rc == 0, lib.ti_last_error()
        torch.cuda.synchronize()
        assert torch.equal(x.cpu(), want_x)
        plain = torch.empty_like(out)
        ops.rmsnorm(x, w, 1e-6, plain)
        assert torch.equal(out, plain)
        assert (f64(out) - ref_rmsnorm(want_x, w, 1e-6)).abs().max() < (1e-5 if dtype == torch.float32 else 0.03)


@pytest.mark.parametrize("tile", [1, 3, 5, 6, 8, 9, 10])
@pytest.mark.parametrize("M,N,K", [(300, 520, 128), (257, 384, 192), (130, 200, 64), (700, 96, 320)])
def test_linear_bf16_every_tile(ops, tile, M, N, K):
    """Each tile of the pipelined kernel (256 x 128 with eight wavefronts, 128 x 64, 64 x 128 for the SwiGLU
    epilogue, 64 x 64, 128 x 160 and 256 x 160 with four wavefronts, which the SwiGLU epilogue does not
    take, and 256 x 256 with k-tiles of 32 in a ring of four stages), whatever the dispatch would have chosen
    for the shape, with every epilogue, against float64."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    lib = ops.lib("gemm_bf16")
    g = torch.Generator().manual_seed(M + N + tile)
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16)
    w = (torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16)
    ref = ref_linear(a, w)
    tol = 2e-5 * K
    ops.tune("gemm_bf16", "force_tile", tile)        # this object's own override: set around each of its calls
    try:
        out = torch.empty(M, N, device="cuda")
        ops.linear(dev(a), dev(w), out, "store")
        assert (f64(out) - ref).abs().max() < tol
        base = torch.randn(M, N, generator=g)
        out = dev(base.clone())
        ops.linear(dev(a), dev(w), out, "add")
        assert (f64(out) - (ref + f64(base))).abs().max() < tol
        out = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
        ops.linear(dev(a), dev(w), out, "store_act")
        assert (f64(out) - ref).abs().max() < 0.005 * ref.abs().max() + tol
        F = N // 2
        out = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
        ops.linear(dev(a), dev(w), out, "swiglu")
        gte, up = ref[:, :F], ref[:, F:]
        want = gte / (1 + torch.exp(-gte)) * up
        assert (f64(out) - want).abs().max() < 0.005 * want.abs().max() + 10 * tol
        with pytest.raises(Exception, match="no shape rule"):
            ops.tune("gemm_bf16", "no_such_rule", 1)
            ops.linear(dev(a), dev(w), torch.empty(M, N, device="cuda"), "store")
    finally:
        ops.tune()


@pytest.mark.parametrize("M,N,K", [(2000, 5130, 192), (2048, 5120, 64), (1100, 9000, 128)])
def test_columns_split_between_two_tile_shapes(ops, M, N, K):
    """256 x 128 tiles that fill the compute units once or more and leave a round mostly empty: the columns
    that make whole rounds take those tiles, the rest 128 x 64 tiles in a second launch.  Same bits as the
    smaller tile everywhere, and the values of float64, for every epilogue."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    lib = ops.lib("gemm_bf16")
    units = torch.cuda.get_device_properties(0).multi_processor_count
    big = -(-M // 256) * -(-N // 128)
    assert big >= units and 0 < big % units < units * 3 // 4 and big < 4 * units, "the shape does not take the rule"
    g = torch.Generator().manual_seed(M + N)
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16)
    w = (torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16)
    base = torch.randn(M, N, generator=g)
    ref = ref_linear(a, w)
    got = {}
    for split in (1, 0):
        lib.ti_tuning_set(b"two_ranges", split)
        try:
            out = torch.empty(M, N, device="cuda")
            ops.linear(dev(a), dev(w), out, "store")
            added = dev(base.clone())
            ops.linear(dev(a), dev(w), added, "add")
            act = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
            ops.linear(dev(a), dev(w), act, "store_act")
            paired = torch.empty(M, N // 2, device="cuda", dtype=torch.bfloat16)
            ops.linear(dev(a), dev(w), paired, "swiglu")
            got[split] = (out, added, act, paired)
        finally:
            lib.ti_tuning_set(b"two_ranges", 1)
    for x, y in zip(got[1], got[0]):
        assert torch.equal(x, y)
    tol = 2e-5 * K
    assert (f64(got[1][0]) - ref).abs().max() < tol
    assert (f64(got[1][1]) - (ref + f64(base))).abs().max() < tol
    assert (f64(got[1][2]) - ref).abs().max() < 0.005 * ref.abs().max() + tol
    gte, up = ref[:, :N // 2], ref[:, N // 2:]
    want = gte / (1 + torch.exp(-gte)) * up
    assert (f64(got[1][3]) - want).abs().max() < 0.005 * want.abs().max() + 10 * tol


@pytest.mark.parametrize("M,N,K", [(2000, 5120, 64), (1990, 2560, 128), (4000, 2560, 64)])
def test_widths_that_160_divides_take_tiles_of_160_columns(ops, M, N, K):
    """Where tiles of 256 x 160 or 128 x 160 make whole rounds of the compute units the dispatch takes them
    (widths of 2,560 and 5,120).  Same bits as without them, and the values of float64."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    lib = ops.lib("gemm_bf16")
    units = torch.cuda.get_device_properties(0).multi_processor_count
    assert (-(-M // 256) * (N // 160)) % units == 0 or (-(-M // 128) * (N // 160)) % units == 0, "the shape does not take the rule"
    g = torch.Generator().manual_seed(M + N)
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16)
    w = (torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16)
    base = torch.randn(M, N, generator=g)
    ref = ref_linear(a, w)
    got = {}
    for on in (1, 0):
        lib.ti_tuning_set(b"tiles_160", on)
        try:
            out = torch.empty(M, N, device="cuda")
            ops.linear(dev(a), dev(w), out, "store")
            added = dev(base.clone())
            ops.linear(dev(a), dev(w), added, "add")
            act = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
            ops.linear(dev(a), dev(w), act, "store_act")
            got[on] = (out, added, act)
        finally:
            lib.ti_tuning_set(b"tiles_160", 1)
    for x, y in zip(got[1], got[0]):
        assert torch.equal(x, y)
    tol = 2e-5 * K
    assert (f64(got[1][0]) - ref).abs().max() < tol
    assert (f64(got[1][1]) - (ref + f64(base))).abs().max() < tol
    assert (f64(got[1][2]) - ref).abs().max() < 0.005 * ref.abs().max() + tol


@pytest.mark.parametrize("tile,M,N,K", [(1, 700, 2048, 128), (1, 2300, 1024, 64), (3, 700, 1024, 192), (9, 1100, 1280, 64),
                                        (0, 1500, 2048, 128)])
@pytest.mark.parametrize("rows", [1, 3, 8])
def test_tiles_taken_in_the_dies_order(ops, tile, M, N, K, rows):
    """The order in which workgroups take a tiled product's tiles when the weight is larger than the cache
    in front of the memory (each die an eighth of the column tiles, in blocks of `rows` row tiles), forced
    here on small products: every tile is still computed once, with the bits of the grid's order; the last
    block of row tiles is short where `rows` does not divide their number; tile 0 is a launch in two ranges."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    lib = ops.lib("gemm_bf16")
    g = torch.Generator().manual_seed(M + N + rows)
    a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    base = torch.randn(M, N, generator=g)
    ref = ref_linear(a.cpu(), w.cpu())
    got = {}
    try:
        lib.ti_tuning_set(b"force_tile", tile)
        for order in (rows, -1):
            lib.ti_tuning_set(b"xcd_rows", order)
            out = torch.full((M + 1, N), 7.0, device="cuda")
            ops.linear(a, w, out[:M], "store")
            added = dev(base.clone())
            ops.linear(a, w, added, "add")
            act = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
            ops.linear(a, w, act, "store_act")
            res = [out, added, act]
            if tile != 9:
                glu = torch.empty(M, N // 2, device="cuda", dtype=torch.bfloat16)
                ops.linear(a, w, glu, "swiglu")
                res.append(glu)
            got[order] = res
    finally:
        lib.ti_tuning_set(b"force_tile", 0)
        lib.ti_tuning_set(b"xcd_rows", 0)
    for x, y in zip(got[rows], got[-1]):
        assert torch.equal(x, y)
    assert (f64(got[rows][0][:M]) - ref).abs().max() < 2e-5 * K
    assert bool((got[rows][0][M] == 7.0).all())


@pytest.mark.parametrize("M,F,K", [(2048, 4096, 4096), (2048, 9216, 4096), (1990, 4056, 4160)])
def test_stacked_gate_up_over_many_rows_takes_tiles_of_256_x_256(ops, M, F, K):
    """A [gate; up] weight over many rows with a long K: 256 x 256 tiles where they make whole rounds of the
    compute units (8 x 32 tiles), and where rounds are left over (8 x 72 tiles: two rounds and a quarter) the
    whole rounds' columns take them and the rest 256 x 128 tiles; rows and columns that fill no tile.
    The bits of the product with the rule switched off, and the values of float64."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    lib = ops.lib("gemm_bf16")
    units = torch.cuda.get_device_properties(0).multi_processor_count
    assert -(-M // 256) * -(-2 * F // 256) >= units, "the shape does not take the rule"
    g = torch.Generator().manual_seed(M + F)
    a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
    w = dev((torch.rand(2 * F, K, generator=g) * 2 - 1).to(torch.bfloat16) * 0.05)
    outs = []
    try:
        for on in (1, 0):
            lib.ti_tuning_set(b"tiles_256", on)
            out = torch.full((M + 1, F), 7.0, device="cuda", dtype=torch.bfloat16)
            ops.linear(a, w, out[:M], "swiglu")
            assert bool((out[M] == 7.0).all())
            outs.append(out[:M])
    finally:
        lib.ti_tuning_set(b"tiles_256", 1)
    assert torch.equal(outs[0], outs[1])
    ref = (a.double() @ w.double().T).cpu()
    want = ref[:, :F] / (1 + torch.exp(-ref[:, :F])) * ref[:, F:]
    assert (f64(outs[0]) - want).abs().max() < 0.005 * want.abs().max() + 2e-4 * K


@pytest.mark.parametrize("M", [17, 40, 64])
def test_swiglu_of_up_to_64_rows_under_a_wide_weight(ops, M):
    """17 to 64 rows times a stacked [gate; up] weight of 32,768 rows take 64 x 128 tiles (twice the weight
    under way per workgroup); the bits are those of the 128 x 64 tiles, and the values match float64."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    F, K = 16384, 1024
    g = torch.Generator().manual_seed(M)
    a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
    w = dev((torch.rand(2 * F, K, generator=g) * 2 - 1).to(torch.bfloat16) * 0.1)
    ref = ref_linear(a.cpu(), w.cpu())
    want = ref[:, :F] / (1 + torch.exp(-ref[:, :F])) * ref[:, F:]
    lib = ops.lib("gemm_bf16")
    outs = []
    try:
        for tile in (0, 3):
            lib.ti_tuning_set(b"force_tile", tile)
            out = torch.empty(M, F, device="cuda", dtype=torch.bfloat16)
            ops.linear(a, w, out, "swiglu")
            assert (f64(out) - want).abs().max() < 0.005 * want.abs().max() + 2e-4 * K
            outs.append(out)
    finally:
        lib.ti_tuning_set(b"force_tile", 0)
    assert torch.equal(outs[0], outs[1])


@pytest.mark.parametrize("M", [17, 40, 64])
def test_stored_product_of_17_to_64_rows_under_a_large_weight_splits_k(ops, M):
    """17 to 64 rows times a weight of 6,144 x 4,096 (the q/k/v projection of a large model), stored in
    32-bit: K goes to several workgroups a tile and a kernel of its own adds their sums.  Against float64,
    against the product with the split switched off (the same values up to the order of the sum), and a
    row's bits do not depend on the rows beside it."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    N, K = 6144, 4096
    g = torch.Generator().manual_seed(M)
    a = dev((torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16))
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    ref = ref_linear(a.cpu(), w.cpu())
    out = torch.full((M + 1, N), 7.0, device="cuda")
    ops.linear(a, w, out[:M], "store")
    assert (f64(out[:M]) - ref).abs().max() < 2e-5 * K
    assert bool((out[M] == 7.0).all())
    try:
        ops.use_split_k_add = False
        plain_out = torch.empty(M, N, device="cuda")
        ops.linear(a, w, plain_out, "store")
    finally:
        ops.use_split_k_add = True
    assert (plain_out - out[:M]).abs().max() < 2e-5 * K
    assert not torch.equal(plain_out, out[:M])              # the split did happen: another order of the sum
    fewer = torch.empty(17, N, device="cuda")
    ops.linear(a[M - 17:], w, fewer, "store")
    assert torch.equal(fewer, out[M - 17:M])


def test_linear_bf16_rows_do_not_depend_on_the_batch(ops):
    """Within one family of kernels a row's bits do not depend on the other rows: the tiled
    kernels (more than 64 rows), the kernels whose workgroups own 16 weight rows (9 to 64 rows
    here), and the kernel with a weight row per wavefront (up to 8 rows, a weight of few rows)."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(4)
    a = torch.randn(200, 264, generator=g).to(torch.bfloat16)
    w = torch.randn(150, 264, generator=g).to(torch.bfloat16)
    full = torch.empty(200, 150, device="cuda")
    ops.linear(dev(a), dev(w), full, "store")                   # tiled
    part = torch.empty(70, 150, device="cuda")
    ops.linear(dev(a[100:170].contiguous()), dev(w), part, "store")     # tiled, other rows
    assert torch.equal(part, full[100:170])
    small = torch.empty(40, 150, device="cuda")
    ops.linear(dev(a[:40].contiguous()), dev(w), small, "store")        # 16 weight rows a workgroup, 3 token tiles
    for lo, hi in ((0, 9), (17, 33), (24, 40)):
        some = torch.empty(hi - lo, 150, device="cuda")
        ops.linear(dev(a[lo:hi].contiguous()), dev(w), some, "store")   # the same family, fewer rows
        assert torch.equal(some, small[lo:hi])
    few = torch.empty(8, 150, device="cuda")
    ops.linear(dev(a[:8].contiguous()), dev(w), few, "store")           # a weight row per wavefront
    for lo, hi in ((0, 1), (3, 4), (2, 4), (4, 8), (7, 8)):
        some = torch.empty(hi - lo, 150, device="cuda")
        ops.linear(dev(a[lo:hi].contiguous()), dev(w), some, "store")
        assert torch.equal(some, few[lo:hi])
    assert (f64(few) - f64(small[:8])).abs().max() < 2e-5 * 264         # the families agree up to rounding


@pytest.mark.parametrize("M,N,K", [(1, 48, 1024), (7, 1000, 1096), (40, 130, 2048), (64, 2048, 1032)])
def test_linear_bf16_few_columns_many_wavefronts(ops, M, N, K):
    """Few output columns and a long K: up to 8 rows take the kernel with a weight row per
    wavefront, more rows the kernel with eight wavefronts that split K.  Same result as float64,
    and a row has the bits it has in a larger batch of the same family."""
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(M + N)
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16)
    w = (torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16)
    ref = ref_linear(a, w)
    base = torch.randn(M, N, generator=g)
    out = dev(base.clone())
    ops.linear(dev(a), dev(w), out, "add")
    assert (f64(out) - (ref + f64(base))).abs().max() < 2e-5 * K
    full = torch.empty(M, N, device="cuda")
    ops.linear(dev(a), dev(w), full, "store")
    k = 1 if M <= 8 else 9                       # fewer rows of the same family of kernels
    some = torch.empty(k, N, device="cuda")
    ops.linear(dev(a[M - k:].contiguous()), dev(w), some, "store")
    assert torch.equal(some, full[M - k:])


@pytest.mark.parametrize("M,N,K", [(1, 4100, 64), (5, 4096, 1024), (16, 40, 192), (9, 130, 1280), (12, 64, 2304),
                                   (2, 4112, 4096), (8, 6144, 1024)])
def test_linear_with_the_norm_inside(ops, M, N, K):
    """rmsnorm and product in one kernel (few tokens) give the bits of the norm kernel
    followed by the product kernel, for every epilogue; and both agree with float64.  (Up to 8
    tokens and a weight of fewer than 4,096 rows are left to the kernel with a weight row per
    wavefront, except for SwiGLU: see the next test.)"""
    from tinyinfer_amd.ops.kernels import NormedRows
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(M * 3 + N)
    x = dev(torch.randn(M, K, generator=g) * 3.0)
    nw = dev(1 + 0.1 * torch.randn(K, generator=g))
    w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
    eps = 1e-3
    h = torch.empty(M, K, device="cuda", dtype=torch.bfloat16)
    ops.rmsnorm(x, nw, eps, h)
    xd = f64(x)
    ref = f64((xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps) * f64(nw)).to(torch.bfloat16)) @ f64(w).T
    assert ops.can_fuse_norm(M, torch.bfloat16)
    for epi, dt in (("store", torch.float32), ("add", torch.float32), ("store_act", torch.bfloat16),
                    ("swiglu", torch.bfloat16)):
        if epi == "swiglu" and N % 2:
            continue
        cols = N // 2 if epi == "swiglu" else N
        base = torch.randn(M, cols, generator=g).to(dt)
        two, one = dev(base.clone()), dev(base.clone())
        ops.linear(h, w, two, epi)
        lazy = NormedRows(x, nw, eps, torch.empty_like(h))
        assert ops._linear_normed(lazy, w, one, epi), "the fused kernel refused a size it should serve"
        assert torch.equal(one, two), epi
        if epi == "store":
            # the norm kernel rounds its rows exactly where the float64 reference does, up to
            # a last bit of the 32-bit scale: allow one bfloat16 step on a few operands
            assert (f64(one) - ref).abs().max() < 2e-5 * K + 0.01 * ref.abs().max()


def test_linear_with_the_norm_inside_refuses_what_it_does_not_serve(ops):
    """More rows than the kernel holds, a K that is no multiple of 64, or few tokens with a weight
    of few rows (which another kernel takes): `linear` computes the norm first and the result
    is that of the norm kernel followed by the product."""
    from tinyinfer_amd.ops.kernels import NormedRows
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(9)
    for M, N, K in ((17, 32, 128), (4, 32, 72), (4, 32, 128), (8, 1024, 2048)):
        x = dev(torch.randn(M, K, generator=g))
        nw = dev(1 + 0.1 * torch.randn(K, generator=g))
        w = dev((torch.rand(N, K, generator=g) * 2 - 1).to(torch.bfloat16))
        h = torch.empty(M, K, device="cuda", dtype=torch.bfloat16)
        ops.rmsnorm(x, nw, 1e-6, h)
        two = torch.empty(M, N, device="cuda")
        ops.linear(h, w, two, "store")
        one = torch.empty(M, N, device="cuda")
        ops.linear(NormedRows(x, nw, 1e-6, torch.empty_like(h)), w, one, "store")
        assert torch.equal(one, two)


# ---------------------------------------------- bfloat16 matrix-core attention
class FakeCtx:
    """The fields of a step context that the attention dispatch reads."""

    def __init__(self, entries, decode_rows_only=False):
        # entries: [(n_tokens, start_pos)], rows laid out in order
        self.entries = entries
        pos, slot, tiles, dec, meta, small = [], [], [], [], [], []
        row0 = 0
        for e, (n, start) in enumerate(entries):
            meta.append([row0, n, start, 0])
            pos += list(range(start, start + n))
            slot += [e] * n
            if n > 1:
                tiles += [[e, row0 + q0] for q0 in range(0, n, 128)]
                small += [(start + min(q0 + 64, n) - 1, e, row0 + q0) for q0 in range(0, n, 64)]
            else:
                dec.append(row0)
            row0 += n
        small.sort(key=lambda t: -t[0])             # from the tile that sees the most keys to the fewest
        self.tiles_small = dev(torch.tensor([t[1:] for t in small], dtype=torch.int32)) if small else None
        self.n_tiles_small = len(small)
        self.M = row0
        self.decode_only = not tiles
        self.positions = dev(torch.tensor(pos, dtype=torch.int32))
        self.slots = dev(torch.tensor(slot, dtype=torch.int32))
        self.entry_meta = dev(torch.tensor(meta, dtype=torch.int32))
        self.tiles = dev(torch.tensor(tiles, dtype=torch.int32)) if tiles else None
        self.n_tiles = len(tiles)
        self.decode_rows = None if self.decode_only else (dev(torch.tensor(dec, dtype=torch.int32)) if dec else None)
        self.n_decode_rows = 0 if self.decode_only else len(dec)
        self.max_context = self.split_context = max(s + n for n, s in entries)
        self.portion_context = max([s + n for n, s in entries if n > 1], default=0)
        self._bufs = {}

    def buf(self, name, shape, dtype):
        t = torch.empty(tuple(shape), dtype=dtype, device="cuda")
        self._bufs[name] = t
        return t


def fast_attention_case(ops, entries_tokens, nh, nkv, hd, P, window, seed, sharp=2.0):
    """Several requests with full contexts in a scattered pool; the step holds the
    last `n` tokens of each.  Returns (got, want) for the step's rows."""
    from tinyinfer_amd.ops import kernels as attention_bf16
    g = torch.Generator().manual_seed(seed)
    lens = [s + n for n, s in entries_tokens]
    n_pages_each = [-(-L // P) for L in lens]
    pages = sum(n_pages_each) + 7
    perm = torch.randperm(pages, generator=g)
    pool = (torch.randn(pages, 2, nkv, P, hd, generator=g) * 30).to(torch.bfloat16)
    pool[0, 0, 0, 0, 0] = float("nan")                     # rubbish may be anything
    vt = pool[:, 1].reshape(pages, nkv, hd, P)
    W = max(n_pages_each) + 1
    table = torch.full((len(lens), W), -1, dtype=torch.int32)
    qs, refs = [], []
    used = 0
    for e, ((n, start), L) in enumerate(zip(entries_tokens, lens)):
        q = (torch.randn(L, nh, hd, generator=g) * sharp).to(torch.bfloat16)
        k = torch.randn(L, nkv, hd, generator=g).to(torch.bfloat16)
        v = torch.randn(L, nkv, hd, generator=g).to(torch.bfloat16)
        mine = perm[used:used + n_pages_each[e]]
        used += n_pages_each[e]
        table[e, :len(mine)] = mine.to(torch.int32)
        # the unwritten tail of the last page holds NaN: nothing of it may leak
        pool[mine[-1], 0] = float("nan")
        vt[mine[-1]] = float("nan")
        for t in range(L):
            pool[mine[t // P], 0, :, t % P] = k[t]
            vt[mine[t // P], :, :, t % P] = v[t]
        ref = ref_attention(q, k, v, 1.0 / math.sqrt(hd), window)
        qs.append(q[start:])
        refs.append(ref[start:])
    qd = dev(torch.cat(qs).reshape(-1, nh * hd))
    out = torch.zeros_like(qd)
    ctx = FakeCtx(entries_tokens)
    ok = run_attention(ops, ctx, View(dev(table)), qd, dev(pool), out, nh, nkv, hd, 1.0 / math.sqrt(hd), window)
    assert ok
    return f64(out), torch.cat(refs).reshape(-1, nh * hd)


@pytest.mark.parametrize("nh,nkv,hd,P,window", [
    (4, 2, 64, 16, None), (6, 2, 32, 16, None), (16, 8, 128, 16, None), (3, 1, 128, 32, None),
    (4, 4, 64, 16, 40), (20, 1, 32, 16, None), (8, 2, 128, 16, 300)])
def test_attention_bf16_decode_rows(ops, nh, nkv, hd, P, window):
    """Single-token entries at many context lengths, page edges included, split over the context."""
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    entries = [(1, s) for s in (0, 1, 15, 16, 17, 31, 32, 100, 511, 512, 777, 1500)]
    got, want = fast_attention_case(ops, entries, nh, nkv, hd, P, window, seed=nh * 100 + hd)
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() < 2e-2


@pytest.mark.parametrize("nh,nkv,hd,P,window", [
    (4, 2, 64, 16, None), (6, 2, 32, 16, None), (4, 2, 128, 16, None), (2, 1, 128, 32, None),
    (4, 4, 64, 16, 40), (2, 2, 32, 16, 7)])
@pytest.mark.parametrize("variant", ["one group", "two groups", "paired", "a tile each"])
def test_attention_bf16_portions_and_mixed(ops, nh, nkv, hd, P, window, variant):
    """Portions of every size, starting anywhere (a page's edge, the middle of a
    page, the start of a request), beside decode rows; with one and with two groups of
    wavefronts per workgroup, and with the kernel of 64-row tiles, giving a workgroup two
    tiles or one (the launch would choose by its size)."""
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    entries = [(2, 0), (7, 30), (1, 99), (16, 16), (17, 15), (64, 0), (65, 63), (130, 41), (1, 0), (3, 300), (200, 5),
               (333, 700)]
    lib = ops.lib("attention_bf16")
    lib.ti_tuning_set(b"prefill_groups", {"one group": 1, "two groups": 2}.get(variant, 0))
    ops.use_paired_prefill = variant in ("paired", "a tile each")
    ops.force_paired_tiles = variant == "paired"
    try:
        got, want = fast_attention_case(ops, entries, nh, nkv, hd, P, window, seed=nh * 10 + hd)
    finally:
        lib.ti_tuning_set(b"prefill_groups", 0)
        ops.use_paired_prefill = True
        ops.force_paired_tiles = None
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() < 2e-2


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_attention_bf16_random_shapes_and_batches(ops, seed):
    """Sixteen batches drawn from a seed: head size, heads and groups, page size, window, one to six entries
    of portions and single tokens starting anywhere, and the launch forced or left to choose.  Finds what the
    hand-picked cases leave out (an entry whose share of the keys is empty, a window that ends inside a
    run, a tile of one row beside one of 700)."""
    import random
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    rnd = random.Random(seed)
    lib = ops.lib("attention_bf16")
    for case in range(16):
        hd = rnd.choice([64, 128])
        nkv = rnd.choice([1, 2, 4, 8])
        nh = nkv * rnd.choice([1, 2, 4])
        P = rnd.choice([16, 32, 48, 64])
        window = rnd.choice([None, None, None, 40, 300, 1000])
        entries = [(rnd.choice([1, 2, 3, 16, 17, 31, 32, 33, 63, 64, 65, 100, 128, 129, 200, 333, 700]),
                    rnd.choice([0, 0, 1, 15, 16, 17, 31, 32, 63, 64, 100, 500, 1000, 1023, 1024, 1500, 3000]))
                   for _ in range(rnd.randint(1, 6))]
        variant = rnd.choice(["as the launch chooses", "paired", "a tile each", "one group", "two groups"])
        lib.ti_tuning_set(b"prefill_groups", {"one group": 1, "two groups": 2}.get(variant, 0))
        ops.use_paired_prefill = variant in ("as the launch chooses", "paired", "a tile each")
        ops.force_paired_tiles = {"paired": True, "a tile each": False}.get(variant)
        try:
            got, want = fast_attention_case(ops, entries, nh, nkv, hd, P, window, seed=seed * 100 + case)
        finally:
            lib.ti_tuning_set(b"prefill_groups", 0)
            ops.use_paired_prefill = True
            ops.force_paired_tiles = None
        what = f"case {case}: head size {hd}, heads {nh}/{nkv}, page {P}, window {window}, {variant}, entries {entries}"
        assert torch.isfinite(got).all(), what
        assert (got - want).abs().max() < 2e-2, what


def test_attention_bf16_far_into_long_contexts(ops):
    """Rows of single tokens behind 20,000 and 32,767 cached tokens (a block table wider than the 1,024 entries
    the decode kernel can hold in LDS, contexts cut into many runs) and portions of prompts deep inside a
    context (300 tokens behind 20,000, 70 behind 9,000: tiles that walk hundreds of pages, the keys in runs),
    against the softmax in float64 of just these rows.  In every request the key at position 7 is made to
    stand out for the last query of head 0, so that a page dropped far back would show."""
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    from tinyinfer_amd.ops import kernels as attention_bf16
    nh, nkv, hd, P = 4, 2, 128, 16
    entries = [(1, 20000), (300, 20000), (1, 32767), (70, 9000), (1, 5)]
    g = torch.Generator().manual_seed(21)
    lens = [s + n for n, s in entries]
    n_pages_each = [-(-L // P) for L in lens]
    pages = sum(n_pages_each) + 5
    perm = torch.randperm(pages, generator=g)
    pool = (torch.randn(pages, 2, nkv, P, hd, generator=g) * 30).to(torch.bfloat16)
    vt = pool[:, 1].reshape(pages, nkv, hd, P)
    table = torch.full((len(lens), max(n_pages_each) + 1), -1, dtype=torch.int32)
    qs, refs = [], []
    used = 0
    scale = 1.0 / math.sqrt(hd)
    for e, ((n, start), L) in enumerate(zip(entries, lens)):
        q = (torch.randn(n, nh, hd, generator=g) * 2.0).to(torch.bfloat16)
        k = torch.randn(L, nkv, hd, generator=g).to(torch.bfloat16)
        v = torch.randn(L, nkv, hd, generator=g).to(torch.bfloat16)
        if L > 7:
            k[7, 0] = (q[-1, 0].float() * 0.5).to(torch.bfloat16)          # score ~ 0.5 |q|^2 / sqrt(hd): far above the rest
        mine = perm[used:used + n_pages_each[e]]
        used += n_pages_each[e]
        table[e, :len(mine)] = mine.to(torch.int32)
        full = (L // P) * P
        pool[mine[:L // P], 0] = k[:full].reshape(L // P, P, nkv, hd).permute(0, 2, 1, 3)
        vt[mine[:L // P]] = v[:full].reshape(L // P, P, nkv, hd).permute(0, 2, 3, 1)
        for t in range(full, L):
            pool[mine[t // P], 0, :, t % P] = k[t]
            vt[mine[t // P], :, :, t % P] = v[t]
        ref = torch.zeros(n, nh, hd, dtype=torch.float64)
        for h in range(nh):
            sc = (f64(q[:, h]) @ f64(k[:, h // (nh // nkv)]).T) * scale           # [n, L]
            key = torch.arange(L)[None, :]
            sc = sc.masked_fill(key > (start + torch.arange(n))[:, None], float("-inf"))
            ref[:, h] = torch.softmax(sc, -1) @ f64(v[:, h // (nh // nkv)])
        if L > 7:
            w7 = torch.softmax((f64(q[-1, 0]) @ f64(k[:, 0]).T) * scale, -1)[7]
            assert w7 > 0.5                                                       # the far key carries the row
        qs.append(q)
        refs.append(ref)
    qd = dev(torch.cat(qs).reshape(-1, nh * hd))
    out = torch.zeros_like(qd)
    ctx = FakeCtx(entries)
    assert run_attention(ops, ctx, View(dev(table)), qd, dev(pool), out, nh, nkv, hd, scale, None)
    got, want = f64(out), torch.cat(refs).reshape(-1, nh * hd)
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() < 2e-2


def test_attention_bf16_paired_tiles_of_one_long_prompt(ops):
    """A prompt of 1,100 tokens in one step (an odd number of 64-row tiles, the last one short):
    the kernel that pairs the tile of the most keys with the one of the fewest, against the
    kernel that takes one tile of 128 rows per workgroup and against the softmax in float64."""
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    outs = []
    try:
        for paired in (True, False):
            ops.use_paired_prefill = ops.force_paired_tiles = paired
            got, want = fast_attention_case(ops, [(1100, 0), (1, 40)], 4, 2, 128, 16, None, seed=5)
            assert (got - want).abs().max() < 2e-2
            outs.append(got)
    finally:
        ops.use_paired_prefill = True
        ops.force_paired_tiles = None
    assert (outs[0] - outs[1]).abs().max() < 2e-2


@pytest.mark.parametrize("paired", [True, False])
@pytest.mark.parametrize("nh,nkv,hd,P,window", [(2, 1, 128, 16, None), (4, 2, 64, 32, None), (2, 2, 128, 16, 1500)])
def test_attention_bf16_short_portions_against_a_long_context(ops, nh, nkv, hd, P, window, paired):
    """Few tiles, thousands of keys: the keys of every tile are cut into runs with a workgroup
    each, and a kernel merges their results.  A portion deep in a long request, one at the
    start of a request (its later runs are empty), one in between, and a single token (its
    row is written by the decode kernel after the merge has passed over it); against float64
    and against the same launch with one run."""
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    from tinyinfer_amd.ops import kernels as attention_bf16
    entries = [(70, 3000), (40, 0), (1, 2500), (130, 1000)]
    ctx = FakeCtx(entries)
    assert attention_bf16.portion_launch(ctx, nh, int(window or 0))[0] >= 3
    outs = []
    ops.force_paired_tiles = paired
    try:
        for split in (True, False):
            ops.use_portion_splits = split
            got, want = fast_attention_case(ops, entries, nh, nkv, hd, P, window, seed=hd + nh)
            assert torch.isfinite(got).all()
            assert (got - want).abs().max() < 2e-2
            outs.append(got)
    finally:
        ops.use_portion_splits = True
        ops.force_paired_tiles = None
    assert (outs[0] - outs[1]).abs().max() < 2e-2
    assert not torch.equal(outs[0], outs[1]), "the switch did not change the launch"


@pytest.mark.parametrize("nh,nkv,hd,P,window,norm,rope", [
    (16, 8, 128, 16, None, True, "table"), (4, 2, 64, 16, None, True, "table"), (3, 1, 128, 32, 50, True, "computed"),
    (4, 4, 64, 16, 40, False, "table"), (16, 1, 64, 16, None, True, None), (8, 2, 128, 16, None, False, None)])
def test_attention_bf16_decode_from_projections(ops, nh, nkv, hd, P, window, norm, rope):
    """The decode kernel that norms and rotates its own queries and writes the row's key and
    value, against the two kernels it stands for, at context lengths around page edges and
    split over the context: the same bits in the cache; the same output up to the last
    bfloat16 bit (the row's own key enters the softmax last instead of in its block)."""
    decode_from_projections_case(ops, nh, nkv, hd, P, window, norm, rope, (0, 1, 15, 16, 17, 31, 32, 100, 511, 512, 777, 1500))


def test_attention_bf16_decode_from_projections_behind_long_contexts(ops):
    """The same behind 4,097, 20,000 and 32,767 cached tokens: block-table rows wider than the 1,024 entries the
    kernel can hold in LDS (the page ids are then looked up in memory), contexts cut into dozens of runs."""
    decode_from_projections_case(ops, 16, 8, 128, 16, None, True, "table", (9, 4097, 20000, 32767))


def decode_from_projections_case(ops, nh, nkv, hd, P, window, norm, rope, starts):
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    g = torch.Generator().manual_seed(nh * 31 + hd)
    entries = [(1, s) for s in starts]
    n_pages_each = [-(-(s + 1) // P) for s in starts]
    pages = sum(n_pages_each) + 5
    perm = torch.randperm(pages, generator=g)
    pool = (torch.randn(pages, 2, nkv, P, hd, generator=g)).to(torch.bfloat16)
    W = max(n_pages_each) + 1
    table = torch.full((len(starts), W), -1, dtype=torch.int32)
    used = 0
    for e, n in enumerate(n_pages_each):
        table[e, :n] = perm[used:used + n].to(torch.int32)
        used += n
    M = len(starts)
    qkv = dev(torch.randn(M, (nh + 2 * nkv) * hd, generator=g) * 2.0)
    q_w = dev(1 + 0.1 * torch.randn(hd, generator=g)) if norm else None
    k_w = dev(1 + 0.1 * torch.randn(hd, generator=g)) if norm else None
    inv_freq = tab = None
    if rope:
        inv_freq = dev((10000.0 ** (-torch.arange(hd // 2, dtype=torch.float64) * 2 / hd)).float())
        if rope == "table":
            tab = ops.rope_table(inv_freq, 600)          # positions beyond the table are computed
    scale = 1.0 / math.sqrt(hd)
    ctx = FakeCtx(entries)
    view = View(dev(table))
    # the two kernels
    pool_a = dev(pool.clone())
    q = torch.empty(M, nh * hd, device="cuda", dtype=torch.bfloat16)
    ops.qk_norm_rope_kv_write(qkv, q_w, k_w, 1e-5, inv_freq, ctx.positions, ctx.slots, view, pool_a, q, nh, nkv, hd, tab)
    out_a = torch.zeros_like(q)
    ops.attention(ctx, view, q, pool_a, out_a, nh, nkv, hd, scale, window)
    # the one kernel
    pool_b = dev(pool.clone())
    out_b = torch.zeros_like(q)
    assert ops.attention_from_projections(ctx, view, qkv, q_w, k_w, 1e-5, inv_freq, tab, pool_b, True, out_b,
                                          nh, nkv, hd, scale, window)
    assert torch.equal(pool_a.view(torch.int16), pool_b.view(torch.int16))
    assert torch.isfinite(out_b.float()).all()
    # told that row m of the step is row m of the block tables, both kernels fetch the row's page ids beside
    # the position instead of behind it: the same bits
    assert torch.equal(ctx.slots.cpu(), torch.arange(M, dtype=torch.int32))
    ctx.slots_are_rows = True
    try:
        out_a2 = torch.zeros_like(q)
        ops.attention(ctx, view, q, pool_a, out_a2, nh, nkv, hd, scale, window)
        assert torch.equal(out_a2.view(torch.int16), out_a.view(torch.int16))
        pool_b2 = dev(pool.clone())
        out_b2 = torch.zeros_like(q)
        assert ops.attention_from_projections(ctx, view, qkv, q_w, k_w, 1e-5, inv_freq, tab, pool_b2, True, out_b2,
                                              nh, nkv, hd, scale, window)
        assert torch.equal(out_b2.view(torch.int16), out_b.view(torch.int16))
        assert torch.equal(pool_b2.view(torch.int16), pool_b.view(torch.int16))
    finally:
        ctx.slots_are_rows = False

    def same_up_to_one_step(x, y):
        x, y = x.float(), y.float()
        return bool(((x - y).abs() <= 2.0 ** -7 * torch.maximum(x.abs(), y.abs()) + 1e-3 * x.abs().max()).all())
    assert same_up_to_one_step(out_a, out_b)
    # and without the write (a layer that reads another layer's keys and values): the cache stays as it is
    pool_c = pool_a.clone()
    out_c = torch.zeros_like(q)
    assert ops.attention_from_projections(ctx, view, qkv[:, :nh * hd].contiguous(), q_w, None, 1e-5, inv_freq, tab,
                                          pool_c, False, out_c, nh, nkv, hd, scale, window)
    assert torch.equal(pool_c.view(torch.int16), pool_a.view(torch.int16))
    assert torch.equal(out_c.view(torch.int16), out_a.view(torch.int16))     # nothing of its own: the same walk


@pytest.mark.parametrize("M,nh,nkv,hd,K,P,norm,rope", [
    (300, 3, 1, 64, 192, 16, True, "table"), (257, 4, 2, 128, 128, 16, True, "table"),
    (100, 2, 2, 128, 64, 32, False, "computed"), (513, 5, 1, 64, 256, 16, True, None), (70, 2, 0, 128, 64, 16, True, "table"),
    (40, 2, 1, 128, 64, 16, True, "table"), (17, 3, 1, 64, 128, 16, True, "computed")])
@pytest.mark.parametrize("tile_rows", [128, 256])
def test_qkv_product_with_prepared_heads(ops, tile_rows, M, nh, nkv, hd, K, P, norm, rope):
    """The q/k/v product whose epilogue norms, rotates and caches, with tiles of 128 and of 256
    rows (the dispatch takes the first while it makes no more workgroups than the chip has
    units), against the product followed by the kernel that prepares whole steps: the same bits
    in q and in the cache (rows that are no multiple of the tile, a last tile with a head beyond
    the matrix, no k/v heads)."""
    qkv_prepared_case(ops, tile_rows, M, nh, nkv, hd, K, P, norm, rope)


@pytest.mark.parametrize("M,nh,nkv,hd", [(2048, 32, 4, 128), (1900, 70, 5, 64)])
def test_qkv_product_with_prepared_heads_in_two_ranges(ops, M, nh, nkv, hd):
    """256-row tiles that would leave a round of workgroups mostly empty: the heads that make whole
    rounds take them, the other heads 128-row tiles in a second launch.  The same bits."""
    units = torch.cuda.get_device_properties(0).multi_processor_count
    big = -(-M // 256) * ((nh + 2 * nkv) * hd // 128)
    assert big >= units and 0 < big % units < units * 3 // 4, "the shape does not take the rule"
    qkv_prepared_case(ops, 0, M, nh, nkv, hd, 64, 16, True, "table")


@pytest.mark.parametrize("tile_rows,rows", [(128, 4), (256, 2)])
def test_qkv_product_with_prepared_heads_in_the_dies_order(ops, tile_rows, rows):
    """The same product with its tiles taken in the dies' order (eight column tiles of whole heads, six or
    three row tiles in blocks of four or two): the same bits in q and in the cache."""
    lib = ops.lib("gemm_bf16")
    lib.ti_tuning_set(b"xcd_rows", rows)
    try:
        qkv_prepared_case(ops, tile_rows, 700, 6, 1, 128, 128, 16, True, "table")
    finally:
        lib.ti_tuning_set(b"xcd_rows", 0)


def qkv_prepared_case(ops, tile_rows, M, nh, nkv, hd, K, P, norm, rope):
    assert ops.use_fast_gemm, "the bfloat16 MFMA kernels are switched off or not built"
    g = torch.Generator().manual_seed(M + nh)
    N = (nh + 2 * nkv) * hd
    a = dev((torch.randn(M, K, generator=g)).to(torch.bfloat16))
    w = dev((torch.randn(N, K, generator=g) * 0.2).to(torch.bfloat16))
    q_w = dev(1 + 0.1 * torch.randn(hd, generator=g)) if norm else None
    k_w = dev(1 + 0.1 * torch.randn(hd, generator=g)) if norm and nkv else None
    inv_freq = tab = None
    if rope:
        inv_freq = dev((10000.0 ** (-torch.arange(hd // 2, dtype=torch.float64) * 2 / hd)).float())
        if rope == "table":
            tab = ops.rope_table(inv_freq, 200)          # positions beyond the table are computed
    # two requests: rows [0, n0) continue one at position 37 (its rows straddle pages), the rest
    # start another at 0; for some sizes that one starts on a multiple of 16 rows, so that runs of
    # 16 tile rows are whole runs of a page (the values' fast path), for others not
    n0 = (M // 3) // 16 * 16 if M in (300, 513) else M // 3
    pos = torch.cat([torch.arange(37, 37 + n0), torch.arange(0, M - n0)]).to(torch.int32)
    slot = torch.cat([torch.zeros(n0), torch.ones(M - n0)]).to(torch.int32)
    pages_each = -(-(M + 40) // P)
    perm = torch.randperm(2 * pages_each + 3, generator=g).to(torch.int32)
    table = torch.stack([perm[:pages_each], perm[pages_each:2 * pages_each]]).contiguous()
    pool0 = torch.randn(2 * pages_each + 3, 2, max(nkv, 1), P, hd, generator=g).to(torch.bfloat16)
    view = View(dev(table))
    pos, slot = dev(pos), dev(slot)
    pool_a, pool_b = dev(pool0.clone()), dev(pool0.clone())
    qkv = torch.empty(M, N, device="cuda")
    ops.linear(a, w, qkv, "store")
    q_a = torch.zeros(M, nh * hd, device="cuda", dtype=torch.bfloat16)
    ops.qk_norm_rope_kv_write(qkv, q_w, k_w, 1e-5, inv_freq, pos, slot, view, pool_a, q_a, nh, nkv, hd, tab)
    q_b = torch.zeros_like(q_a)
    lib = ops.lib("gemm_bf16")
    lib.ti_tuning_set(b"qkv_prep_rows", tile_rows)
    try:
        assert ops.qkv_prepared(a, w, q_w, k_w, 1e-5, inv_freq, tab, pos, slot, view, pool_b, q_b, nh, nkv, hd)
    finally:
        lib.ti_tuning_set(b"qkv_prep_rows", 0)
    if M > 64:
        assert torch.equal(q_a.view(torch.int16), q_b.view(torch.int16))
        assert torch.equal(pool_a.view(torch.int16), pool_b.view(torch.int16))
    else:
        # up to 64 rows the product alone comes from kernels that sum in another order: the same
        # values up to the rounding of the result (rubbish in untouched cache rows may be NaN: bits there)
        assert (f64(q_a) - f64(q_b)).abs().max() <= 2 ** -7 * f64(q_a).abs().max()
        touched = pool_a.view(torch.int16) != dev(pool0).view(torch.int16)
        assert torch.equal(touched, pool_b.view(torch.int16) != dev(pool0).view(torch.int16)) or nkv == 0
        da, db = f64(pool_a)[touched.cpu()], f64(pool_b)[touched.cpu()]
        assert nkv == 0 or (da - db).abs().max() <= 2 ** -7 * da.abs().max()
    if nkv:
        assert not torch.equal(pool_a.view(torch.int16), dev(pool0).view(torch.int16))


def test_attention_bf16_far_key(ops):
    """One key far back carries the weight, for a decode row and for a row inside a portion."""
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    from tinyinfer_amd.ops import kernels as attention_bf16
    T, hd, P = 1000, 64, 16
    g = torch.Generator().manual_seed(21)
    k = (torch.randn(T, 1, hd, generator=g) * 0.1).to(torch.bfloat16)
    v = torch.randn(T, 1, hd, generator=g).to(torch.bfloat16)
    far = 17
    k[far, 0] = 0
    k[far, 0, 3] = 30.0
    n_pages = -(-T // P)
    pool = torch.zeros(n_pages, 2, 1, P, hd, dtype=torch.bfloat16)
    vt = pool[:, 1].reshape(n_pages, 1, hd, P)
    for t in range(T):
        pool[t // P, 0, 0, t % P] = k[t, 0]
        vt[t // P, 0, :, t % P] = v[t, 0]
    table = torch.arange(n_pages, dtype=torch.int32)[None, :].repeat(2, 1).contiguous()
    for entries in ([(1, T - 1)], [(100, T - 100)]):
        n = entries[0][0]
        q = torch.zeros(n, hd, dtype=torch.bfloat16)
        q[-1, 3] = 30.0
        out = torch.zeros(n, hd, dtype=torch.bfloat16, device="cuda")
        ctx = FakeCtx(entries)
        assert run_attention(ops, ctx, View(dev(table)), dev(q), dev(pool), out, 1, 1, hd, 1.0 / 8, None)
        assert (f64(out[-1]) - f64(v[far, 0])).abs().max() < 2e-2
