"""The engine against the plain implementation, in 32-bit and in bfloat16, under
every way of cutting the work: each request alone and whole; most of it in one
step and the last 32 tokens one by one; in portions of changing size, down to
two tokens; and mixed, up to four live requests, portions of some beside decoded
tokens of others, with so few pages that they are used again."""
import numpy as np
import pytest
import torch

import traces
from helpers import CONFIGS, ODD_CONFIGS, random_tokens, read_folder, sharpen_folder
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

# Largest allowed |engine - plain| over all logits.  Random-weight logits of the
# tiny models are of order 0.1 to 1.
#   float32: against the plain model in float64 with no rounding: 2e-5.
#   bfloat16: against the plain model with bfloat16 rounding where the engine
#   rounds (matrix operands, cached keys/values, q), from the same bfloat16
#   weights.  A value that lies near a rounding boundary may round the other way
#   in the engine (its 32-bit sums differ from float64 in the last bits), and
#   such flips spread like the rounding itself; so the bound is the size of that
#   rounding's own effect on this model and these tokens, measured on the plain
#   model as max |rounded - exact| (the engine stays at a third of it or below).
TOL = {"float32": 2e-5}
BF16_NOISE_FACTOR = 1.0

REQUEST_LENGTHS = {"a": 97, "b": 45, "c": 130, "d": 33, "e": 71, "f": 58}
PROMPT_LENGTHS = {"a": 60, "b": 12, "c": 101, "d": 30, "e": 2, "f": 41}
ROUNDED = plain.bf16_sites(("gemm_in", "kv_cache", "q"))


def make_requests(vocab, seed=7):
    return {r: random_tokens(n, vocab, seed + i) for i, (r, n) in enumerate(REQUEST_LENGTHS.items())}


_plain_cache = {}


def plain_logits(folder, requests, dtype, angles32=False):
    """({request: logits [T, V]}, tolerance) of the plain model for this dtype.  angles32: the plain model has
    the rotation's frequencies and angles in 32-bit like the engine (for contexts of thousands of tokens)."""
    key = (folder, angles32, tuple((r, tuple(t)) for r, t in sorted(requests.items())))
    for d in ("float32", "bfloat16"):
        if key + (d,) not in _plain_cache:
            cfg, w = read_folder(folder)
            rnd = ROUNDED if d == "bfloat16" else plain.no_rounding
            if angles32:
                rnd = plain.float32_angles(rnd)
            _plain_cache[key + (d,)] = {r: plain.forward(w, cfg, t, rnd) for r, t in requests.items()}
    want = _plain_cache[key + (dtype,)]
    if dtype == "float32":
        return want, TOL["float32"]
    exact = _plain_cache[key + ("float32",)]
    noise = max(float(np.abs(want[r] - exact[r]).max()) for r in want)
    return want, BF16_NOISE_FACTOR * noise


def replay(engine, trace):
    """Feed a trace through Engine.step; {request: [logits row per position]}."""
    from tinyinfer_amd.engine import StepEntry
    got = {}
    for step in trace:
        logits = engine.step([StepEntry(r, t, w) for r, t, w in step["entries"]])
        rows = None if logits is None else logits.cpu().numpy().astype(np.float64)     # None: nothing wanted
        i = 0
        for r, t, w in step["entries"]:
            for _ in w:
                got.setdefault(r, []).append(rows[i])
                i += 1
        for r in step["end"]:
            engine.release(r)
        engine.cache.check()
    return {r: np.stack(v) for r, v in got.items()}


def build_engine(folder, dtype, max_tokens, page_size=16):
    import tinyinfer_amd  # noqa: F401
    from tinyinfer_amd.engine import Engine
    return Engine.from_folder(folder, dtype, page_size=page_size, max_tokens=max_tokens, max_requests=4,
                              max_seq=max_tokens)


def worst(got, want):
    w = 0.0
    where = None
    for r in want:
        assert got[r].shape == want[r].shape, (r, got[r].shape, want[r].shape)
        d = np.abs(got[r] - want[r]).max(axis=1)
        if d.max() > w:
            w, where = float(d.max()), (r, int(d.argmax()))
    return w, where


def make_trace(mode, requests):
    if mode == "whole":
        return traces.whole(requests)
    if mode == "tail":
        return traces.tail_one_by_one(requests, 32)
    if mode == "portions":
        return traces.portions(requests)
    return traces.mixed(requests, PROMPT_LENGTHS, live=4)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,sharp,page_size", [("A", False, 16), ("B", False, 4), ("B", True, 16), ("C", True, 16), ("D", True, 16), ("D", True, 32)])
@pytest.mark.parametrize("mode", ["whole", "tail", "portions", "mixed"])
def test_engine_matches_plain(model_folders, name, sharp, page_size, dtype, mode):
    folder = model_folders(name, "bfloat16", sharp)
    requests = make_requests(CONFIGS[name]["vocab_size"])
    want, tol = plain_logits(folder, requests, dtype)
    trace = make_trace(mode, requests)
    # the tightest pool that holds the trace, so that pages given back are handed out again
    n_tok = traces.max_pages(trace, page_size) * page_size
    assert n_tok <= traces.max_tokens(trace)
    engine = build_engine(folder, dtype, n_tok, page_size)
    got = replay(engine, trace)
    assert not engine.cache.live_requests()
    for _, g in engine.cache.paged_groups():
        assert g.pool.num_free == g.pool.num_pages            # every page came back
    if mode == "mixed":
        for _, g in engine.cache.paged_groups():
            assert g.pool.taken_total > g.pool.num_pages      # pages were handed out again
    err, where = worst(got, want)
    print(f"\n[{name} sharp={sharp} P={page_size} {dtype} {mode}] max |engine - plain| = {err:.3e} at {where}"
          f" (allowed {tol:.3e})")
    assert err < tol, (err, tol, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(ODD_CONFIGS))
def test_shapes_at_the_edges_match_plain(tmp_path_factory, name, dtype):
    """Head sizes 16, 80, 112 and 256, one and seventeen heads a group, a window on every layer, widths that are
    multiples of 8 only: mixed steps in a tight pool (which kernels serve such a shape differs; the logits do not)."""
    from tinyinfer_amd.weights import write_model_folder
    cfg = ODD_CONFIGS[name]
    folder = str(tmp_path_factory.mktemp("odd"))
    write_model_folder(folder, cfg, seed=99, dtype="bfloat16")
    sharpen_folder(folder)
    requests = make_requests(cfg["vocab_size"])
    want, tol = plain_logits(folder, requests, dtype)
    trace = make_trace("mixed", requests)
    engine = build_engine(folder, dtype, traces.max_pages(trace, 16) * 16, 16)
    got = replay(engine, trace)
    assert not engine.cache.live_requests()
    err, where = worst(got, want)
    assert err < tol, (err, tol, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prompt_of_5000_tokens_in_portions_then_decoding(tmp_path_factory, dtype):
    """Beyond every other test's contexts: 5,000 tokens fed as portions of 2,048, 2,048 and 884 (the later ones
    attend through thousands of cached keys, in runs), then 20 tokens one by one behind them (block-table rows
    of 300 and more pages), beside a second short request; config D's shapes (a head of 64, windows of 37 on two
    layers, full attention on one).  The last rows of every portion and every decoded row are the plain model's."""
    from tinyinfer_amd.weights import write_model_folder
    cfg = dict(CONFIGS["D"], max_position_embeddings=8192)
    folder = str(tmp_path_factory.mktemp("long"))
    write_model_folder(folder, cfg, seed=5, dtype="bfloat16")
    sharpen_folder(folder)
    requests = {"a": random_tokens(5020, cfg["vocab_size"], 70), "b": random_tokens(40, cfg["vocab_size"], 71)}
    # thousands of tokens in, an angle computed in 32-bit is some 1e-4 off (the plain model with
    # `float32_angles` shows it): the engine's table of cosines and sines comes from angles in double precision
    want, tol = plain_logits(folder, requests, dtype)
    a, b = requests["a"], requests["b"]
    trace = [{"entries": [("a", a[:2048], [0, 2047])], "end": []},
             {"entries": [("a", a[2048:4096], [0, 1000, 2047]), ("b", b[:20], [19])], "end": []},
             {"entries": [("a", a[4096:5000], [0, 500, 903]), ("b", b[20:21], [0])], "end": []}]
    for k in range(19):
        trace.append({"entries": [("b", b[21 + k:22 + k], [0]), ("a", a[5000 + k:5001 + k], [0])], "end": []})
    trace.append({"entries": [("a", a[5019:5020], [0])], "end": ["a", "b"]})
    engine = build_engine(folder, dtype, 5120 + 64)
    got = replay(engine, trace)
    places = {"a": [0, 2047, 2048, 3048, 4095, 4096, 4596, 4999] + list(range(5000, 5020)), "b": [19] + list(range(20, 40))}
    worst_err = 0.0
    for r, at in places.items():
        assert got[r].shape[0] == len(at), (r, got[r].shape)
        worst_err = max(worst_err, float(np.abs(got[r] - want[r][at]).max()))
    assert worst_err < tol, (worst_err, tol)


@pytest.mark.parametrize("seed", [1, 2, 3])
@pytest.mark.parametrize("name,dtype,page_size,graph", [("B", "float32", 4, False), ("D", "float32", 16, True),
                                                        ("B", "bfloat16", 16, True), ("D", "bfloat16", 32, False)])
def test_steps_drawn_at_random_match_plain(model_folders, name, dtype, page_size, graph, seed):
    """Steps cut at random: which live requests a step feeds, in which order, how many tokens each,
    which places are wanted; the pool as tight as the trace allows; with graphs, the shapes that
    repeat are replayed.  Only the wanted places come back, and each is the plain model's."""
    folder = model_folders(name, "bfloat16", True)
    requests = make_requests(CONFIGS[name]["vocab_size"])
    want, tol = plain_logits(folder, requests, dtype)
    trace = traces.at_random(requests, seed)
    assert any(len(s["entries"]) >= 3 for s in trace) and any(len(t) == 1 for s in trace for _, t, _ in s["entries"])
    engine = build_engine(folder, dtype, traces.max_pages(trace, page_size) * page_size, page_size)
    from tinyinfer_amd.engine import StepEntry
    fed = {r: 0 for r in requests}
    worst_err, where = 0.0, None
    for k, step in enumerate(trace):
        entries = [StepEntry(r, t, w) for r, t, w in step["entries"]]
        logits = (engine.step_graph(entries) if graph else engine.step(entries)).cpu().numpy().astype(np.float64)
        i = 0
        for r, t, w in step["entries"]:
            for place in w:
                err = float(np.abs(logits[i] - want[r][fed[r] + place]).max())
                if err > worst_err:
                    worst_err, where = err, (k, r, fed[r] + place)
                i += 1
            fed[r] += len(t)
        assert i == logits.shape[0]
        for r in step["end"]:
            engine.release(r)
        engine.cache.check()
    assert not engine.cache.live_requests()
    assert fed == {r: len(t) for r, t in requests.items()}
    print(f"\n[{name} {dtype} P={page_size} graph={graph} seed={seed}] {len(trace)} steps, max |engine - plain| = "
          f"{worst_err:.3e} at {where} (allowed {tol:.3e})")
    assert worst_err < tol, (worst_err, tol, where)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_float32_weights_stay_32bit(model_folders, dtype):
    """A folder stored in float32: the float32 engine uses every bit of it."""
    folder = model_folders("A", "float32")
    requests = {"a": random_tokens(40, 256, 3)}
    cfg, w = read_folder(folder)
    exact = plain.forward(w, cfg, requests["a"])
    if dtype == "bfloat16":
        w = {k: (plain.round_bf16(v) if v.ndim == 2 else v) for k, v in w.items()}
        want = plain.forward(w, cfg, requests["a"], ROUNDED)
        tol = BF16_NOISE_FACTOR * np.abs(want - exact).max()
    else:
        want, tol = exact, TOL["float32"]
    engine = build_engine(folder, dtype, 64)
    got = replay(engine, traces.whole(requests))
    assert np.abs(got["a"] - want).max() < tol


def test_first_tokens_and_long_decoding(model_folders):
    """The first tokens of a sequence one by one from an empty cache, then a long
    run of single-token steps across many pages."""
    folder = model_folders("B", "bfloat16", True)
    toks = random_tokens(400, 1000, 11)
    cfg, w = read_folder(folder)
    want = plain.forward(w, cfg, toks)
    engine = build_engine(folder, "float32", 448, page_size=16)
    trace = [{"entries": [("r", [t], [0])], "end": []} for t in toks]
    trace[-1]["end"] = ["r"]
    got = replay(engine, trace)
    assert np.abs(got["r"] - want).max() < TOL["float32"]


def test_cuts_agree_bitwise_in_float32(model_folders):
    """In 32-bit every output element is reduced in an order that does not depend
    on the batch, so different cuts give the same bits, not just close ones."""
    folder = model_folders("B", "bfloat16", True)
    requests = make_requests(1000)
    results = []
    for mode in ("whole", "portions", "mixed"):
        trace = make_trace(mode, requests)
        engine = build_engine(folder, "float32", traces.max_tokens(trace), 4)
        results.append(replay(engine, trace))
    for r in requests:
        assert np.array_equal(results[0][r], results[1][r]), r
        assert np.array_equal(results[0][r], results[2][r]), r


def test_norm_inside_the_product_changes_no_bit(model_folders):
    """Steps of few tokens run the norm before a projection inside the projection's
    kernel.  With that switched off the same steps give the same bits."""
    folder = model_folders("A", "bfloat16")
    requests = {r: t for r, t in make_requests(CONFIGS["A"]["vocab_size"]).items() if r in ("a", "b")}
    trace = traces.tail_one_by_one(requests, 32)
    results = []
    for fused in (True, False):
        engine = build_engine(folder, "bfloat16", traces.max_tokens(trace))
        engine.ops.use_fused_norm = fused            # the switches are the engine's own
        assert engine.ops.can_fuse_norm(1, torch.bfloat16) == fused
        results.append(replay(engine, trace))
    for r in requests:
        assert np.array_equal(results[0][r], results[1][r]), r


def test_prepared_decode_attention_changes_only_rounding(model_folders):
    """Steps of single tokens norm, rotate and cache inside the attention kernel.  With that
    switched off the same steps give the same logits up to the rounding of a different order
    of summation (config D: head size 64, one kv head, a window)."""
    folder = model_folders("D", "bfloat16", True)
    requests = {r: t for r, t in make_requests(CONFIGS["D"]["vocab_size"]).items() if r in ("a", "c")}
    trace = traces.tail_one_by_one(requests, 48)
    results = []
    for fused in (True, False):
        engine = build_engine(folder, "bfloat16", traces.max_tokens(trace))
        engine.ops.use_fused_qk_decode = fused
        results.append(replay(engine, trace))
    _, tol = plain_logits(folder, make_requests(CONFIGS["D"]["vocab_size"]), "bfloat16")
    for r in requests:
        assert np.abs(results[0][r] - results[1][r]).max() < tol, r
        assert not np.array_equal(results[0][r][:1], results[0][r][1:2])


@pytest.mark.parametrize("config,fused", [("D", True), ("D", False), ("B", True)])
def test_page_ids_fetched_beside_the_position_change_no_bit(model_folders, config, fused):
    """In a step of single tokens the decode attention fetches a row's page ids beside its position
    instead of behind it (row m of the step is row m of the block tables).  With that switched off
    the same steps give the same bits: requests that start in different steps, so that rows and
    block-table rows are told apart, with pages that are used again."""
    folder = model_folders(config, "bfloat16", True)
    V = CONFIGS[config]["vocab_size"]
    requests = {r: random_tokens(n, V, 50 + i) for i, (r, n) in enumerate((("a", 90), ("b", 41), ("c", 70), ("d", 55)))}
    first = {"a": 50, "b": 21, "c": 30, "d": 35}                      # fed whole; the rest one token a step
    trace = [{"entries": [(r, requests[r][:first[r]], [first[r] - 1]) for r in ("a", "b", "c")], "end": []}]
    fed = dict(first)
    live = ["a", "b", "c"]
    for k in range(40):
        if k == 20:                                                   # b is over; d takes its pages
            trace.append({"entries": [("d", requests["d"][:first["d"]], [first["d"] - 1])], "end": []})
            live = ["d", "c", "a"]
        order = live[k % 3:] + live[:k % 3]                           # the rows of a step in changing order
        trace.append({"entries": [(r, requests[r][fed[r]:fed[r] + 1], [0]) for r in order], "end": ["b"] if k == 19 else []})
        for r in order:
            fed[r] += 1
    trace[-1]["end"] = list(live)
    assert fed == {"a": 90, "b": 41, "c": 70, "d": 55}
    results = []
    for early in (True, False):
        engine = build_engine(folder, "bfloat16", 256)
        engine.ops.use_early_page_ids = early
        engine.ops.use_fused_qk_decode = fused
        results.append(replay(engine, trace))
    for r in requests:
        assert np.array_equal(results[0][r], results[1][r]), r
        assert len(results[0][r]) == len(requests[r]) - first[r] + 1


def test_prepared_qkv_product_changes_no_bit(model_folders):
    """Steps of many tokens prepare q and write the cache in the epilogue of the q/k/v product.
    With that switched off the same steps give the same bits (config D, head size 64)."""
    folder = model_folders("D", "bfloat16", True)
    requests = {"a": random_tokens(300, CONFIGS["D"]["vocab_size"], 5), "b": random_tokens(90, CONFIGS["D"]["vocab_size"], 6)}
    trace = [{"entries": [("a", requests["a"][:200], [0, 199]), ("b", requests["b"][:70], [69])], "end": []},
             {"entries": [("a", requests["a"][200:], list(range(100))), ("b", requests["b"][70:71], [0])], "end": ["a", "b"]}]
    results = []
    for fused in (True, False):
        engine = build_engine(folder, "bfloat16", 512)
        engine.ops.use_fused_qkv_prefill = fused
        results.append(replay(engine, trace))
    for r in requests:
        assert np.array_equal(results[0][r], results[1][r]), r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_real_width_match_plain(model_folders, dtype):
    """Two layers with the widths of Qwen3-0.6B: a prompt of 540 tokens in portions (one of them
    beside another request's decoded token), then 24 tokens one by one (a context long enough for
    the decode attention to split it over workgroups), against the plain model.  These widths take
    other kernels than the tiny configurations do."""
    folder = model_folders("E", "bfloat16", True)
    V = CONFIGS["E"]["vocab_size"]
    requests = {"a": random_tokens(564, V, 31), "b": random_tokens(40, V, 32)}
    want, tol = plain_logits(folder, requests, dtype)
    a, b = requests["a"], requests["b"]
    trace = [{"entries": [("a", a[:200], [0, 100, 199]), ("b", b[:39], [38])], "end": []},
             {"entries": [("b", b[39:40], [0]), ("a", a[200:540], list(range(0, 340, 31)))], "end": ["b"]}]
    trace += [{"entries": [("a", a[i:i + 1], [0])], "end": []} for i in range(540, 564)]
    trace[-1]["end"] = ["a"]
    engine = build_engine(folder, dtype, 704)
    got = replay(engine, trace)
    rows = {"a": [0, 100, 199] + [200 + i for i in range(0, 340, 31)] + list(range(540, 564)), "b": [38, 39]}
    # The 32-bit bound of the tiny models (2e-5 for logits of order 1) is kept relative to the size
    # of the logits here: sums run over 1,024 to 3,072 terms instead of 64 to 224.
    scale = max(1.0, max(float(np.abs(want[r]).max()) for r in requests))
    if dtype == "float32":
        tol = TOL["float32"] * scale
    for r in requests:
        err = np.abs(got[r] - want[r][rows[r]]).max()
        print(f"\n[E {dtype} {r}] max |engine - plain| = {err:.3e} (allowed {tol:.3e}, logits up to {scale:.1f})")
        assert err < tol, (r, err, tol)


def test_a_layer_of_another_real_width_matches_plain(model_folders):
    """One layer with the widths of Qwen3-4B in bfloat16: a prompt of 2,048 tokens whole (its o and down
    projections take tiles of 128 x 160), seven short requests beside its first decoded token, then six steps
    of all eight (products of 8 rows under weights of 2,560 and 9,728 columns), against the plain model."""
    folder = model_folders("F", "bfloat16", True)
    V = CONFIGS["F"]["vocab_size"]
    requests = {"a": random_tokens(2055, V, 61)}
    requests.update({f"s{i}": random_tokens(9, V, 70 + i) for i in range(7)})
    want, tol = plain_logits(folder, requests, "bfloat16")
    a = requests["a"]
    shorts = [r for r in requests if r != "a"]
    trace = [{"entries": [("a", a[:2048], [0, 1000, 2047])], "end": []},
             {"entries": [("a", a[2048:2049], [0])] + [(r, requests[r][:3], [2]) for r in shorts], "end": []}]
    for k in range(6):
        trace.append({"entries": [("a", a[2049 + k:2050 + k], [0])] + [(r, requests[r][3 + k:4 + k], [0]) for r in shorts], "end": []})
    trace[-1]["end"] = list(requests)
    from tinyinfer_amd.engine import Engine
    engine = Engine.from_folder(folder, "bfloat16", page_size=16, max_tokens=2048 + 64 + 7 * 16, max_requests=8, max_seq=2112)
    got = replay(engine, trace)
    rows = {"a": [0, 1000, 2047] + list(range(2048, 2055))}
    rows.update({r: list(range(2, 9)) for r in shorts})
    for r in requests:
        err = np.abs(got[r] - want[r][rows[r]]).max()
        print(f"\n[F bfloat16 {r}] max |engine - plain| = {err:.3e} (allowed {tol:.3e})")
        assert err < tol, (r, err, tol)


def test_steps_of_17_to_64_tokens_at_real_width(model_folders):
    """Steps of 17 to 64 tokens at the widths of Qwen3-0.6B: the products into the residual split
    K over workgroups and leave their partial sums to the norm that follows (the last one to a
    kernel of their own, before the final norm of the wanted rows).  A prompt in portions of 40,
    17, 64 and 33 tokens, one of them beside another request's token, then a step that wants
    nothing: against the plain model; with the sums added at once the bits are the same, and
    with the kernels without MFMA the logits agree within the same bound."""
    folder = model_folders("E", "bfloat16", True)
    V = CONFIGS["E"]["vocab_size"]
    requests = {"a": random_tokens(154, V, 41), "b": random_tokens(3, V, 42)}
    want, tol = plain_logits(folder, requests, "bfloat16")
    a, b = requests["a"], requests["b"]
    trace = [{"entries": [("a", a[:40], [0, 39])], "end": []},
             {"entries": [("a", a[40:57], [16])], "end": []},
             {"entries": [("b", b[:2], []), ("a", a[57:119], [0, 61])], "end": []},
             {"entries": [("a", a[119:152], [])], "end": []},                   # wants nothing
             {"entries": [("a", a[152:154], [0, 1]), ("b", b[2:3], [0])], "end": ["a", "b"]}]
    rows = {"a": [0, 39, 56, 57, 118, 152, 153], "b": [2]}
    results = {}
    for how in ("left to the norm", "added at once", "without MFMA"):
        engine = build_engine(folder, "bfloat16", 256)
        engine.ops.use_deferred_add = how == "left to the norm"
        engine.ops.use_split_k_add = how != "without MFMA"
        results[how] = replay(engine, trace)
        assert engine.ops._pending is None
    for r in requests:
        got = results["left to the norm"][r]
        err = np.abs(got - want[r][rows[r]]).max()
        print(f"\n[E 17..64 tokens {r}] max |engine - plain| = {err:.3e} (allowed {tol:.3e})")
        assert err < tol, (r, err, tol)
        assert np.array_equal(got, results["added at once"][r]), r
        assert np.abs(results["without MFMA"][r] - want[r][rows[r]]).max() < tol, r
    assert not np.array_equal(results["left to the norm"]["a"], results["without MFMA"]["a"]), \
        "the switch did not change the kernel"


def test_step_refuses_what_it_cannot_run(model_folders):
    from tinyinfer_amd.engine import StepEntry, EngineError
    from tinyinfer_amd.cache import OutOfPages
    engine = build_engine(model_folders("A"), "float32", 64)
    with pytest.raises(EngineError):
        engine.step([StepEntry("x", [1, 2, 999], [0])])           # token outside the vocabulary
    with pytest.raises(EngineError):
        engine.step([StepEntry("x", [1, 2], [2])])                # wanted place outside the entry
    with pytest.raises(EngineError):
        engine.step([StepEntry("x", [1], []), StepEntry("x", [2], [])])
    engine.step([StepEntry("x", list(range(60)), [59])])
    free = engine.cache.num_free_pages()
    with pytest.raises(OutOfPages):
        engine.step([StepEntry("y", list(range(10)), [0])])       # the pool is full
    assert engine.cache.num_free_pages() == free and not engine.cache.has("y")
    engine.cache.check()
