"""The scheduler's workloads in bfloat16: three requests with prompts of 5, 17 and 33 tokens, portions of
7 beside decoding requests, pages of 4, temperature 0.8 (the reference's loop with batching:
/root/reference/src/main.cpp:210-297).  Every step's logits lie inside the bfloat16 bound of the plain
model, and the token drawn is the plain model's wherever its margin exceeds that bound.  Preemption with
graphs changes no token.  How far the engine's rounding (matrix operands, cached keys/values, and q and
the softmax weights in addition) is from rounding only where the reference rounds is reported and
bounded.  And a part that reads the residual stream with torch finds it complete at 17 to 64 rows, where
the built-in parts leave partial sums of a product to the next norm."""
import numpy as np
import pytest
import torch

from helpers import CONFIGS, random_tokens, read_folder
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

ENGINE_SITES = plain.bf16_sites(("gemm_in", "kv_cache", "q"))
REFERENCE_SITES = plain.bf16_sites(plain.REFERENCE_SITES)


def drive(engine, scheduler, sampler, use_graph, on_step):
    """The generation loop, step by step from Python so that every step's logits can be looked at."""
    import tinyinfer_amd as ti
    while scheduler.has_work():
        plan = scheduler.plan()
        entries = [ti.StepEntry(e.request.key, e.request.tokens[e.start:e.start + e.n_tokens],
                                (e.n_tokens - 1,) if e.sample else ()) for e in plan.entries]
        logits = engine.step_graph(entries) if use_graph else engine.step(entries)
        asked = [e.request for e in plan.entries if e.sample]
        sampled = {}
        if asked:
            toks = sampler.sample(logits, [r.params for r in asked], [r.number for r in asked],
                                  [len(r.generated) for r in asked])
            on_step(asked, logits.cpu().numpy().astype(np.float64), toks)
            sampled = {r.number: t for r, t in zip(asked, toks)}
        for done in scheduler.commit(plan, sampled):
            engine.release(done.key)


@pytest.mark.parametrize("top_k", [0, 4])
def test_config_b_workload_in_bfloat16(model_folders, top_k):
    """top_k 0 is the reference's default (the 512 largest logits): with random weights that distribution is
    nearly flat, so hardly any draw is decided beyond the rounding; with the 4 largest most are."""
    import tinyinfer_amd as ti
    from tinyinfer_amd.sampling import Sampler, uniform, DEFAULT_TOP_K
    d = model_folders("B", "bfloat16", True)
    cfg, w = read_folder(d)
    prompts = [random_tokens(n, 1000, 10 + n) for n in (5, 17, 33)]
    engine = ti.Engine.from_folder(d, "bfloat16", page_size=4, max_tokens=192, max_requests=3, max_seq=64)
    scheduler = ti.Scheduler(engine.cache, max_batched_tokens=12, chunk_size=7)
    params = ti.SamplingParams(0.8, top_k, 1.0, 123)
    K = top_k or DEFAULT_TOP_K
    requests = [scheduler.add(p, 6, params) for p in prompts]
    checked = {"rows": 0, "decided": 0, "worst": 0.0, "bound": 0.0, "reference": 0.0}

    def on_step(asked, logits, toks):
        for row, (r, tok) in enumerate(zip(asked, toks)):
            seq = r.tokens
            exact = plain.forward(w, cfg, seq)[-1]
            want = plain.forward(w, cfg, seq, ENGINE_SITES)[-1]
            ref = plain.forward(w, cfg, seq, REFERENCE_SITES)[-1]
            bound = 1.0 * max(float(np.abs(want - exact).max()), 1e-3)
            err = float(np.abs(logits[row] - want).max())
            assert err < bound, (r.number, len(seq), err, bound)
            checked["worst"] = max(checked["worst"], err)
            checked["bound"] = max(checked["bound"], bound)
            checked["reference"] = max(checked["reference"], float(np.abs(logits[row] - ref).max()))
            # the draw: the plain model's token, unless the distance of this row's logits from the plain ones could
            # change which logits are kept, or move an edge of the drawn token's share of [0, 1) across the
            # uniform number
            u = uniform(params.seed, r.number, len(r.generated))
            p = plain.sample_distribution(want, params.temperature, K, params.top_p)
            c = np.cumsum(p)
            margin = float(np.abs(c - u * c[-1]).min())
            slack = np.expm1(2.0 * err / params.temperature) + 1e-6  # |d log p| <= 2 err / T, so |d cdf| <= this
            order = np.sort(want)[::-1]
            kept_for_sure = K >= len(want) or order[K - 1] - order[K] > 2.0 * err
            checked["rows"] += 1
            if margin > slack and kept_for_sure:
                checked["decided"] += 1
                assert tok == plain.draw(p, u), (r.number, len(seq), tok, plain.draw(p, u), margin, slack)

    drive(engine, scheduler, Sampler(engine.ops), False, on_step)
    print(f"\n[B bfloat16 scheduled, top_k {top_k}] {checked['rows']} sampled rows, {checked['decided']} decided by "
          f"their margin; max |engine - plain(engine's rounding)| = {checked['worst']:.3e} (bound {checked['bound']:.3e}); "
          f"max |engine - plain(the reference's rounding: operands and cache only)| = {checked['reference']:.3e}")
    assert checked["rows"] == 18 and (top_k == 0 or checked["decided"] >= 10)
    # rounding q and the softmax weights as well moves the logits no further than the rounding the reference does
    assert checked["reference"] < 2.0 * checked["bound"]
    for r in requests:
        assert r.finish_reason == "length" and len(r.generated) == 6
    assert not engine.cache.live_requests()
    engine.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_preemption_with_graphs_changes_no_token(model_folders, dtype):
    """Too few pages, decode steps replayed from graphs: the youngest request gives way and is fed again
    later; the tokens are the ones a roomy pool gives without graphs."""
    import tinyinfer_amd as ti
    d = model_folders("B", "bfloat16", True)
    prompts = [random_tokens(n, 1000, 70 + n) for n in (12, 12, 9)]
    roomy = ti.Engine.from_folder(d, dtype, page_size=4, max_tokens=256, max_requests=3, max_seq=48)
    want = ti.generate_ids(roomy, prompts, max_new_tokens=20, temperature=0.0)
    tight = ti.Engine.from_folder(d, dtype, page_size=4, max_tokens=64, max_requests=3, max_seq=48)
    stats = ti.GenerationStats()
    got = ti.generate_ids(tight, prompts, max_new_tokens=20, temperature=0.0, stats=stats, use_graph=True)
    assert stats.preemptions > 0 and tight.graph_keys()
    if dtype == "float32":
        assert got == want
    else:
        # a request fed again in one portion sums its products in another order than token by token: a greedy
        # choice between two nearly equal logits may differ; until then the tokens are the same
        same = sum(a == b for g, h in zip(got, want) for a, b in zip(g, h))
        assert got[0] == want[0] and same >= 50, (got, want)
    assert not tight.cache.live_requests()
    tight.cache.check()


def test_failed_generation_leaves_the_cache_clean(model_folders):
    """A step that fails in the middle of a generation (here: a sampler that raises) gives every request the
    scheduler still holds back to the cache, and the next generation on the same engine is the one a fresh
    engine gives."""
    import tinyinfer_amd as ti
    d = model_folders("B", "bfloat16", True)
    prompts = [random_tokens(n, 1000, 30 + n) for n in (9, 14)]
    fresh = ti.Engine.from_folder(d, "float32", page_size=4, max_tokens=128, max_requests=2, max_seq=48)
    want = ti.generate_ids(fresh, prompts, max_new_tokens=8)
    engine = ti.Engine.from_folder(d, "float32", page_size=4, max_tokens=128, max_requests=2, max_seq=48)
    calls = {"n": 0}

    def boom(request, token):
        calls["n"] += 1
        if calls["n"] == 5:
            raise RuntimeError("stop here")

    scheduler = ti.Scheduler(engine.cache)
    for p in prompts:
        scheduler.add(p, 8)
    from tinyinfer_amd.api import run_requests
    with pytest.raises(Exception):
        run_requests(engine, scheduler, on_token=boom)
    assert not engine.cache.live_requests() and engine.cache.num_free_pages() == 32
    engine.cache.check()
    assert ti.generate_ids(engine, prompts, max_new_tokens=8) == want
    # an entry that does not start where the cache ends is refused, and nothing is taken for it
    engine.step([ti.StepEntry("x", prompts[0], ())])
    with pytest.raises(ti.engine.EngineError):
        engine.step([ti.StepEntry("x", [1, 2, 3, 10 ** 6], ())])             # a token outside the vocabulary
    assert engine.cache.length("x") == len(prompts[0])
    engine.cache.check()


def test_a_part_that_reads_the_residual_with_torch_finds_it_complete(tmp_path):
    """At 17 to 64 rows the built-in attention and feed-forward leave partial sums of their last product to
    the norm that reads the residual next.  A block defined here reads the residual with a torch expression
    instead: the engine completes the sums before it runs, so its logits are those of the same steps with the
    sums added at once."""
    import tinyinfer_amd as ti
    from tinyinfer_amd.parts import Part
    from tinyinfer_amd.spec import LayerSpec, ModelSpec, PartSpec
    from tinyinfer_amd.weights import write_model_folder

    class TorchReadingBlock(Part):
        """x += 0.5 * tanh(x), computed by torch on the residual stream itself."""
        family = "block"
        slots = {}

        def forward(self, ctx, x):
            x += 0.5 * torch.tanh(x)

    def spec_of(c):
        H = c["hidden"]
        attn = PartSpec("attention", {"hidden": H, "heads": 16, "kv_heads": 8, "head_dim": 128, "qk_norm": True, "eps": 1e-6,
                                      "pos": PartSpec("rope_neox", {"head_dim": 128, "theta": 1e6})}, "attn")
        full = lambda i: LayerSpec(f"l.{i}", PartSpec("pre_norm"), {
            "norm1": PartSpec("rmsnorm", {"dim": H, "eps": 1e-6}, "n1"), "mixer": attn,
            "norm2": PartSpec("rmsnorm", {"dim": H, "eps": 1e-6}, "n2"),
            "ffn": PartSpec("swiglu", {"hidden": H, "intermediate": 3072}, "ffn")})
        layers = [full(0), LayerSpec("l.1", PartSpec("torch_reader"), {}), full(2)]
        return ModelSpec("TorchReader", c["vocab"], H, PartSpec("table", {"vocab": c["vocab"], "dim": H}, "emb"), layers,
                         PartSpec("rmsnorm", {"dim": H, "eps": 1e-6}, "norm"),
                         PartSpec("linear", {"vocab": c["vocab"], "dim": H, "tied": True, "tied_to": "emb.weight"}, "head"))

    ti.register_part("block", "torch_reader", TorchReadingBlock)
    ti.register_architecture("TorchReader", dict, spec_of)
    cfg = dict(architectures=["TorchReader"], vocab=500, hidden=1024)
    d = str(tmp_path / "reader")
    write_model_folder(d, cfg, seed=2, dtype="bfloat16")
    toks = random_tokens(130, 500, 8)
    cuts = ((0, 40), (40, 57), (57, 121), (121, 130))          # 40, 17, 64 and 9 rows
    results = []
    for deferred in (True, False):
        engine = ti.Engine.from_folder(d, "bfloat16", page_size=16, max_tokens=256, max_requests=1, max_seq=256)
        engine.ops.use_deferred_add = deferred
        results.append(torch.cat([engine.step([ti.StepEntry("r", toks[a:b], list(range(b - a)))]).clone() for a, b in cuts]))
    assert torch.isfinite(results[0]).all()
    assert torch.equal(results[0], results[1])
