"""The logits where the bench runs: the whole depth and vocabulary of Qwen3-0.6B (28 layers, 151,936
tokens), random weights.  The reference's own whole-model check compares logits of a real checkpoint
with another implementation (/root/reference/docs/report.md:21-33); here the plain model under tests/
stands in, on ~96 tokens: the prompt whole, then its last 32 tokens one by one; one decode step of 64
requests whose pages lie scattered gives each request the logits it gets alone; the head's product over
all 151,936 columns against float64; and decode rows at contexts of 2,048 to 4,095 tokens."""
import math
import os
import shutil

import numpy as np
import pytest
import torch

from helpers import random_tokens, read_folder
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

CONFIG = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=28, hidden_size=1024,
              num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072,
              vocab_size=151936, rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
              attention_bias=False, hidden_act="silu", max_position_embeddings=40960)
V = CONFIG["vocab_size"]
ROUNDED = plain.bf16_sites(("gemm_in", "kv_cache", "q"))


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from tinyinfer_amd.weights import write_model_folder
    d = str(tmp_path_factory.mktemp("qwen3_0p6b_sizes"))
    write_model_folder(d, CONFIG, seed=77, dtype="bfloat16")
    yield d
    shutil.rmtree(d, ignore_errors=True)


@pytest.fixture(scope="module")
def plain_rows(folder):
    """Logits of the plain model for one request of 96 tokens: exact, and with bfloat16 rounding where the
    engine rounds."""
    cfg, w = read_folder(folder)
    tokens = random_tokens(96, V, 5)
    exact = plain.forward(w, cfg, tokens)
    rounded = plain.forward(w, cfg, tokens, ROUNDED)
    return tokens, exact, rounded


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_full_depth_whole_and_tail_one_by_one(folder, plain_rows, dtype):
    import tinyinfer_amd as ti
    tokens, exact, rounded = plain_rows
    want = exact if dtype == "float32" else rounded
    scale = max(1.0, float(np.abs(exact).max()))
    # float32: the bound of the tiny models, relative to the size of these logits (sums of 1,024 to 3,072 terms);
    # bfloat16: twice the rounding's own effect on this model and these tokens
    tol = 2e-5 * scale if dtype == "float32" else 2.0 * float(np.abs(rounded - exact).max())
    engine = ti.Engine.from_folder(folder, dtype, page_size=16, max_tokens=256, max_requests=2, max_seq=128)
    whole = engine.step([ti.StepEntry("w", tokens, list(range(96)))]).cpu().numpy().astype(np.float64)
    engine.release("w")
    tail = [engine.step([ti.StepEntry("t", tokens[:64], list(range(64)))]).cpu().numpy().astype(np.float64)]
    for i in range(64, 96):
        tail.append(engine.step([ti.StepEntry("t", tokens[i:i + 1], [0])]).cpu().numpy().astype(np.float64))
    tail = np.concatenate(tail)
    for name, got in (("whole", whole), ("tail", tail)):
        err = float(np.abs(got - want).max())
        print(f"\n[0.6B sizes {dtype} {name}] max |engine - plain| = {err:.3e} (allowed {tol:.3e}, logits up to {scale:.1f})")
        assert err < tol, (name, err, tol)
        assert (got.argmax(1) == want.argmax(1)).mean() > (0.99 if dtype == "float32" else 0.9)
    if dtype == "float32":
        assert np.array_equal(whole, tail)          # in 32-bit a cut changes no bit


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_step_of_64_requests_on_scattered_pages(folder, dtype):
    """64 requests of 3 to 180 tokens, four of them with contexts of 2,048 to 4,095, filled in turn while others
    come and go (so their pages lie scattered), then one step that decodes a token of each: every row is the row
    the request gets when it runs alone (bit for bit in 32-bit; in bfloat16 a step of 64 rows takes other product
    kernels than a step of one, so up to their order of summation)."""
    import tinyinfer_amd as ti
    rng = np.random.default_rng(3)
    lengths = [int(n) for n in rng.integers(3, 180, size=64)]
    for i, n in zip((5, 21, 40, 63), (2048, 2600, 3333, 4095)):
        lengths[i] = n
    prompts = [random_tokens(n, V, 100 + i) for i, n in enumerate(lengths)]
    nxt = [int(t) for t in rng.integers(0, V, size=64)]
    engine = ti.Engine.from_folder(folder, dtype, page_size=16, max_tokens=sum(lengths) + 64 * 32 + 4096, max_requests=66,
                                   max_seq=4097)
    for i, p in enumerate(prompts):
        if i % 3 == 1:                                  # someone else's pages in between, given back later
            engine.step([ti.StepEntry(("squat", i), random_tokens(50 + i, V, i), ())])
        engine.step([ti.StepEntry(i, p, ())])
        if i % 3 == 2:
            engine.release(("squat", i - 1))
    for r in list(engine.cache.live_requests()):
        if isinstance(r, tuple):
            engine.release(r)
    engine.cache.check()
    tables = [engine.cache.table(0, i) for i in range(64)]
    assert any(t != sorted(t) or t[-1] - t[0] + 1 != len(t) for t in tables), "the pages are not scattered"
    together = engine.step([ti.StepEntry(i, [nxt[i]], [0]) for i in range(64)]).cpu().numpy().astype(np.float64)
    for i in range(64):
        engine.release(i)
    alone = np.empty_like(together)
    for i, p in enumerate(prompts):
        engine.step([ti.StepEntry("solo", p, ())])
        alone[i] = engine.step([ti.StepEntry("solo", [nxt[i]], [0])]).cpu().numpy()[0]
        engine.release("solo")
    if dtype == "float32":
        assert np.array_equal(together, alone)
    else:
        err = np.abs(together - alone).max(axis=1)
        scale = float(np.abs(alone).max())
        print(f"\n[0.6B sizes bfloat16] 64 rows together against alone: max diff {err.max():.3e} (logits up to {scale:.2f})")
        # two orders of summation of the same bfloat16 products: far below one bfloat16 step of the logits' scale
        assert err.max() < 0.02 * scale
        assert (together.argmax(1) == alone.argmax(1)).mean() > 0.9


@pytest.mark.parametrize("M", [1, 17, 64])
def test_head_product_over_the_whole_vocabulary(M):
    """logits = h E^T over all 151,936 columns at 1, 17 and 64 rows (three different kernels) against float64."""
    from tinyinfer_amd.ops.kernels import get_ops
    ops = get_ops()
    g = torch.Generator().manual_seed(M)
    K = 1024
    a = (torch.rand(M, K, generator=g) * 2 - 1).to(torch.bfloat16)
    w = (torch.randn(V, K, generator=g) * 0.05).to(torch.bfloat16)
    w[V - 1] = 0.25
    w[0] = -0.25                                   # the first and the last column stand out
    out = torch.full((M, V), float("nan"), device="cuda")
    ops.linear(a.cuda(), w.cuda(), out, "store")
    ref = a.double() @ w.double().T
    got = out.cpu().double()
    assert torch.isfinite(got).all()
    assert (got - ref).abs().max() < 2e-5 * K
    float32 = torch.full((M, V), float("nan"), device="cuda")
    ops.linear(a.float().cuda(), w.float().cuda(), float32, "store")
    assert (float32.cpu().double() - ref).abs().max() < 2e-5 * math.sqrt(K)


def test_decode_attention_at_contexts_of_2048_to_4095():
    """Single-token rows whose contexts end at and beyond 2,048 tokens (a page's edge, the last position a
    4,096-token sequence has), one far key made to stand out in each: against float64."""
    from tinyinfer_amd.ops.kernels import get_ops
    from test_kernels_gpu import fast_attention_case
    ops = get_ops()
    assert ops.use_fast_attention, "the bfloat16 attention kernels are switched off or not built"
    entries = [(1, s) for s in (2047, 2048, 2049, 3000, 3583, 4094)]
    got, want = fast_attention_case(ops, entries, 16, 8, 128, 16, None, seed=4095)
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() < 2e-2
