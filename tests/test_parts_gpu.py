"""Each part alone against its plain function, and parts that are defined here,
in the test: a mixer with state of its own, a feed-forward with routing, another
position encoding, a block arrangement, an architecture.  They are registered,
built, loaded and stepped without a change to the framework's files."""
import json
import math
import os

import numpy as np
import pytest
import torch

from helpers import random_tokens, read_folder
from plain import qwen3_plain as plain

pytestmark = pytest.mark.gpu

DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


class PartCtx:
    """The least a part that keeps no cache needs of a step context."""

    def __init__(self, dtype, positions=None):
        import tinyinfer_amd  # noqa: F401
        from tinyinfer_amd.ops.kernels import get_ops
        self.ops = get_ops()
        self.dtype = dtype
        self.act_dtype = DT[dtype]
        self.f32 = torch.float32
        self.positions = positions
        self._b = {}

    def buf(self, name, shape, dtype):
        self._b[name] = torch.empty(tuple(shape), dtype=dtype, device="cuda")
        return self._b[name]


def build(family, kind, params, tensors, dtype, prefix="p"):
    """Build a part through the registry and load `tensors` (float64 numpy by name)."""
    from tinyinfer_amd import build_part, PartSpec
    part = build_part(family, PartSpec(kind, params), prefix)
    need = part.tensors()
    assert set(need) >= set(tensors), (sorted(need), sorted(tensors))
    loaded = {}
    for n, t in tensors.items():
        assert tuple(t.shape) == need[n].shape
        dt = DT[dtype] if need[n].role == "matrix" else torch.float32
        loaded[n] = torch.tensor(t, dtype=torch.float64).to(dt).cuda()
    part.load(loaded)
    return part


def f64(t):
    return t.detach().cpu().to(torch.float64).numpy()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_norm_part(dtype):
    r = np.random.default_rng(1)
    x, w = r.normal(size=(5, 72)) * 2, 1 + 0.1 * r.normal(size=72)
    part = build("norm", "rmsnorm", {"dim": 72, "eps": 3e-5}, {"p.weight": w}, dtype)
    out = part.forward(PartCtx(dtype), torch.tensor(x, dtype=torch.float32).cuda())
    want = plain.rms_norm(np.float32(x), np.float32(w), 3e-5)
    assert out.dtype == DT[dtype]
    assert np.abs(f64(out) - want).max() < (1e-5 if dtype == "float32" else 3e-2)


def test_position_encoding_part():
    r = np.random.default_rng(2)
    q, k = r.normal(size=(6, 3, 48)), r.normal(size=(6, 1, 48))
    pos = [0, 1, 2, 50, 51, 1000]
    part = build("pos", "rope_neox", {"head_dim": 48, "theta": 5e5}, {}, "float32").to("cuda")
    ctx = PartCtx("float32", torch.tensor(pos, dtype=torch.int32).cuda())
    qd, kd = (torch.tensor(a, dtype=torch.float32).cuda() for a in (q, k))
    part.apply(ctx, qd, kd)
    assert np.abs(f64(qd) - plain.rope_neox(np.float32(q), pos, 5e5)).max() < 2e-4
    assert np.abs(f64(kd) - plain.rope_neox(np.float32(k), pos, 5e5)).max() < 2e-4
    assert part.fused_rotation()["inv_freq"].shape == (24,)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_feed_forward_part(dtype):
    r = np.random.default_rng(3)
    H, F, M = 40, 104, 9
    w = {"p.gate_proj.weight": r.normal(size=(F, H)) * 0.2, "p.up_proj.weight": r.normal(size=(F, H)) * 0.2,
         "p.down_proj.weight": r.normal(size=(H, F)) * 0.2}
    part = build("ffn", "swiglu", {"hidden": H, "intermediate": F}, w, dtype)
    h, x = r.normal(size=(M, H)), r.normal(size=(M, H))
    hd = torch.tensor(h).to(DT[dtype]).cuda()
    xd = torch.tensor(x, dtype=torch.float32).cuda()
    part.forward(PartCtx(dtype), hd, xd)
    wr = {k: f64(torch.tensor(v).to(DT[dtype])) for k, v in w.items()}
    rnd = plain.bf16_sites(("gemm_in",)) if dtype == "bfloat16" else plain.no_rounding
    want = np.float32(x) + plain.ffn_block(f64(hd), wr, "p", rnd)        # it adds into the residual stream
    assert np.abs(f64(xd) - want).max() < (1e-5 if dtype == "float32" else 2e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tied", [True, False])
def test_embedding_and_head_parts(dtype, tied):
    r = np.random.default_rng(4)
    V, H = 117, 24
    E, L = r.normal(size=(V, H)), r.normal(size=(V, H))
    emb = build("embedding", "table", {"vocab": V, "dim": H}, {"e.weight": E}, dtype, prefix="e")
    tensors = {"e.weight": E} if tied else {"h.weight": L}
    head = build("head", "linear", {"vocab": V, "dim": H, "tied": tied, "tied_to": "e.weight"}, tensors, dtype, "h")
    ctx = PartCtx(dtype)
    toks = torch.tensor([5, 0, 116, 5], dtype=torch.int32).cuda()
    x = torch.empty(4, H, device="cuda")
    emb.forward(ctx, toks, x)
    Er = f64(torch.tensor(E).to(DT[dtype]))
    assert np.array_equal(f64(x), Er[[5, 0, 116, 5]])
    h = torch.tensor(r.normal(size=(3, H))).to(DT[dtype]).cuda()
    logits = head.forward(ctx, h)
    Wr = Er if tied else f64(torch.tensor(L).to(DT[dtype]))
    assert logits.dtype == torch.float32
    assert np.abs(f64(logits) - f64(h) @ Wr.T).max() < 1e-4


# ------------------------------------------------ parts defined in this test
def register_toys():
    import tinyinfer_amd as ti
    from tinyinfer_amd.parts import Part
    from tinyinfer_amd.parts.base import join
    from tinyinfer_amd.spec import LayerSpec, ModelSpec, PagedRowsNeed, PartSpec, StateNeed, TensorNeed

    class DecayMixer(Part):
        """A mixer with state of its own: s_t = decay * s_{t-1} + h_t W^T; out_t = s_t.
        The state is one vector per request and layer, kept in the request's slot."""
        family = "mixer"

        def __init__(self, prefix, hidden, decay):
            super().__init__(prefix)
            self.hidden, self.decay = hidden, decay

        def tensors(self):
            return {join(self.prefix, "w"): TensorNeed((self.hidden, self.hidden), "matrix", ("normal", 0.0, 0.2))}

        def load(self, tensors):
            self.w = tensors[join(self.prefix, "w")]

        def cache_need(self):
            return StateNeed((self.hidden,))

        def forward(self, ctx, h, x):
            group, layer = ctx.binding(self)
            state = ctx.state(group, layer)
            u = h.float() @ self.w.float().T
            for row0, n, start, slot in ctx.entries:
                s = state[slot]
                for t in range(row0, row0 + n):
                    s = self.decay * s + u[t]
                    x[t] += s
                state[slot] = s

    class WindowMean(Part):
        """A mixer with pages of its own: every token keeps u_t = h_t W^T (one row of 32-bit numbers per
        token and layer, in pages the cache manager hands out and takes back); out_t is the mean of
        the rows of the last `window` tokens."""
        family = "mixer"

        def __init__(self, prefix, hidden, window):
            super().__init__(prefix)
            self.hidden, self.window = hidden, window

        def tensors(self):
            return {join(self.prefix, "w"): TensorNeed((self.hidden, self.hidden), "matrix", ("normal", 0.0, 0.2))}

        def load(self, tensors):
            self.w = tensors[join(self.prefix, "w")]

        def cache_need(self):
            return PagedRowsNeed((self.hidden,), float32=True, window=self.window)

        def forward(self, ctx, h, x):
            group, layer = ctx.binding(self)
            pool = ctx.page_pool(group, layer)               # [pages, P, hidden] float32
            view = ctx.cache_view(group)
            P = view.page_size
            u = h.float() @ self.w.float().T
            for e, (row0, n, start, slot) in enumerate(ctx.entries):
                table = view.table[e].tolist()
                for i in range(n):
                    p = start + i
                    assert table[p // P] >= 0
                    pool[table[p // P], p % P] = u[row0 + i]
                    rows = [pool[table[q // P], q % P] for q in range(max(0, p - self.window + 1), p + 1)]
                    x[row0 + i] += torch.stack(rows).mean(0)

    class BareBlock(Part):
        """An arrangement with a mixer and nothing else: x += mixer(cast(x))."""
        family = "block"
        slots = {"mixer": "mixer"}

        def __init__(self, prefix, mixer):
            super().__init__(prefix)
            self.mixer = mixer

        def children(self):
            return [self.mixer]

        def forward(self, ctx, x):
            self.mixer.forward(ctx, x.to(ctx.act_dtype, copy=True), x)

    class RoutedFFN(Part):
        """A feed-forward with routing: the expert with the largest router logit takes the
        token, out = softmax(router)[e] * W2[e] relu(W1[e] h).  Router logits in 32-bit."""
        family = "ffn"

        def __init__(self, prefix, hidden, inner, experts):
            super().__init__(prefix)
            self.hidden, self.inner, self.experts = hidden, inner, experts

        def tensors(self):
            H, F, E = self.hidden, self.inner, self.experts
            return {join(self.prefix, "router"): TensorNeed((E, H), "vector", ("normal", 0.0, 0.5)),
                    join(self.prefix, "w1"): TensorNeed((E, F, H), "matrix", ("normal", 0.0, 0.2)),
                    join(self.prefix, "w2"): TensorNeed((E, H, F), "matrix", ("normal", 0.0, 0.2))}

        def load(self, tensors):
            self.router = tensors[join(self.prefix, "router")]
            self.w1 = tensors[join(self.prefix, "w1")]
            self.w2 = tensors[join(self.prefix, "w2")]

        def forward(self, ctx, h, x):
            hf = h.float()
            prob = torch.softmax(hf @ self.router.T, dim=-1)
            top = prob.argmax(dim=-1)
            for e in range(self.experts):
                rows = (top == e).nonzero().flatten()
                if rows.numel():
                    y = torch.relu(hf[rows] @ self.w1[e].float().T) @ self.w2[e].float().T
                    x[rows] += prob[rows, e:e + 1] * y

    class PairRotary(Part):
        """Another position encoding: neighbours (2i, 2i + 1) rotate together.  It has no fused
        form, so the attention part calls `apply` on its 32-bit projections."""
        family = "pos"

        def __init__(self, prefix, head_dim, theta):
            super().__init__(prefix)
            self.head_dim, self.theta = head_dim, theta

        def apply(self, ctx, q, k):
            half = self.head_dim // 2
            inv = self.theta ** (-torch.arange(half, dtype=torch.float64, device=q.device) * 2 / self.head_dim)
            ang = ctx.positions.double()[:, None] * inv[None, :]
            cos, sin = ang.cos().float()[:, None, :], ang.sin().float()[:, None, :]
            for t in (q, k):
                if t is None:
                    continue
                a, b = t[..., 0::2].clone(), t[..., 1::2].clone()
                t[..., 0::2] = a * cos - b * sin
                t[..., 1::2] = a * sin + b * cos

    def read(d):
        return dict(d)

    def spec_of(c):
        H = c["hidden"]
        attn = PartSpec("attention", {"hidden": H, "heads": c["heads"], "kv_heads": c["kv_heads"],
                                      "head_dim": c["head_dim"], "qk_norm": c["qk_norm"], "eps": c["eps"],
                                      "window": c.get("window"),
                                      "pos": PartSpec("rope_neox", {"head_dim": c["head_dim"], "theta": c["theta"]})
                                      if c["rotate"] else None}, "attn")
        pair_attn = PartSpec("attention", {"hidden": H, "heads": c["heads"], "kv_heads": c["kv_heads"],
                                           "head_dim": c["head_dim"], "qk_norm": c["qk_norm"], "eps": c["eps"],
                                           "window": c.get("window"),
                                           "pos": PartSpec("toy_pair_rotary", {"head_dim": c["head_dim"],
                                                                               "theta": c["theta"]})}, "attn")
        layers = []
        for i, kind in enumerate(c["layers"]):
            if kind == "routed":
                layers.append(LayerSpec(f"l.{i}", PartSpec("pre_norm"), {
                    "norm1": PartSpec("rmsnorm", {"dim": H, "eps": c["eps"]}, "n1"), "mixer": pair_attn,
                    "norm2": PartSpec("rmsnorm", {"dim": H, "eps": c["eps"]}, "n2"),
                    "ffn": PartSpec("toy_routed", {"hidden": H, "inner": c["ff"], "experts": c["experts"]}, "moe")}))
            elif kind == "decay":
                layers.append(LayerSpec(f"l.{i}", PartSpec("bare"), {
                    "mixer": PartSpec("toy_decay", {"hidden": H, "decay": c["decay"]}, "mix")}))
            elif kind == "memory":
                layers.append(LayerSpec(f"l.{i}", PartSpec("bare"), {
                    "mixer": PartSpec("toy_window_mean", {"hidden": H, "window": c["memory_window"]}, "mem")}))
            elif kind == "bare_attention":
                layers.append(LayerSpec(f"l.{i}", PartSpec("bare"), {"mixer": attn}))
            else:
                layers.append(LayerSpec(f"l.{i}", PartSpec("pre_norm"), {
                    "norm1": PartSpec("rmsnorm", {"dim": H, "eps": c["eps"]}, "n1"), "mixer": attn,
                    "norm2": PartSpec("rmsnorm", {"dim": H, "eps": c["eps"]}, "n2"),
                    "ffn": PartSpec("swiglu", {"hidden": H, "intermediate": c["ff"]}, "ffn")}))
        return ModelSpec("ToyLM", c["vocab"], H, PartSpec("table", {"vocab": c["vocab"], "dim": H}, "emb"), layers,
                         PartSpec("rmsnorm", {"dim": H, "eps": c["eps"]}, "norm"),
                         PartSpec("linear", {"vocab": c["vocab"], "dim": H, "tied": True, "tied_to": "emb.weight"}, "head"),
                         schedule=c.get("schedule"))

    ti.register_part("mixer", "toy_decay", DecayMixer)
    ti.register_part("mixer", "toy_window_mean", WindowMean)
    ti.register_part("ffn", "toy_routed", RoutedFFN)
    ti.register_part("pos", "toy_pair_rotary", PairRotary)
    ti.register_part("block", "bare", BareBlock)
    ti.register_architecture("ToyLM", read, spec_of)


TOY = dict(architectures=["ToyLM"], vocab=90, hidden=32, heads=2, kv_heads=1, head_dim=16, ff=48, eps=1e-5,
           theta=1e4, decay=0.8, qk_norm=True, rotate=True, layers=["decay", "full", "decay"])


def pair_rotation(x, theta):
    """x [T, heads, hd]: dims (2i, 2i + 1) of position t rotate by t * theta^(-2i/hd)."""
    T, _, hd = x.shape
    ang = np.arange(T)[:, None] * theta ** (-np.arange(hd // 2) * 2.0 / hd)[None, :]
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = np.empty_like(x)
    out[..., 0::2] = x[..., 0::2] * cos - x[..., 1::2] * sin
    out[..., 1::2] = x[..., 0::2] * sin + x[..., 1::2] * cos
    return out


def toy_plain(cfg, w, toks):
    """The toy model, whole sequence, numpy."""
    x = plain.embed(w["emb.weight"], toks)
    T = len(toks)
    order = cfg.get("schedule") or range(len(cfg["layers"]))
    for i in order:
        kind = cfg["layers"][i]
        p = f"l.{i}"
        if kind == "decay":
            u = x @ w[p + ".mix.w"].T
            s = np.zeros(cfg["hidden"])
            out = np.zeros_like(x)
            for t in range(T):
                s = cfg["decay"] * s + u[t]
                out[t] = s
            x = x + out
        elif kind == "memory":
            u = x @ w[p + ".mem.w"].T
            out = np.stack([u[max(0, t - cfg["memory_window"] + 1):t + 1].mean(0) for t in range(T)])
            x = x + out
        else:
            full = kind in ("full", "routed")
            h = plain.rms_norm(x, w[p + ".n1.weight"], cfg["eps"]) if full else x
            a = p + ".attn"
            q = plain.linear(h, w[a + ".q_proj.weight"]).reshape(T, cfg["heads"], cfg["head_dim"])
            k = plain.linear(h, w[a + ".k_proj.weight"]).reshape(T, cfg["kv_heads"], cfg["head_dim"])
            v = plain.linear(h, w[a + ".v_proj.weight"]).reshape(T, cfg["kv_heads"], cfg["head_dim"])
            if cfg["qk_norm"]:
                q = plain.qk_norm(q, w[a + ".q_norm.weight"], cfg["eps"])
                k = plain.qk_norm(k, w[a + ".k_norm.weight"], cfg["eps"])
            if kind == "routed":
                q, k = pair_rotation(q, cfg["theta"]), pair_rotation(k, cfg["theta"])
            elif cfg["rotate"]:
                q, k = plain.rope_neox(q, range(T), cfg["theta"]), plain.rope_neox(k, range(T), cfg["theta"])
            o = plain.attention(q, k, v, cfg.get("window")).reshape(T, -1)
            x = x + plain.linear(o, w[a + ".o_proj.weight"])
            if kind == "routed":
                h = plain.rms_norm(x, w[p + ".n2.weight"], cfg["eps"])
                logit = h @ w[p + ".moe.router"].T
                prob = np.exp(logit - logit.max(-1, keepdims=True))
                prob /= prob.sum(-1, keepdims=True)
                out = np.zeros_like(x)
                for t in range(T):
                    e = int(prob[t].argmax())
                    out[t] = prob[t, e] * (w[p + ".moe.w2"][e] @ np.maximum(w[p + ".moe.w1"][e] @ h[t], 0.0))
                x = x + out
            elif full:
                h = plain.rms_norm(x, w[p + ".n2.weight"], cfg["eps"])
                x = x + plain.ffn_block(h, w, p + ".ffn", plain.no_rounding)
    return plain.linear(plain.rms_norm(x, w["norm.weight"], cfg["eps"]), w["emb.weight"])


def toy_engine(tmp_path, cfg, max_tokens=256, **kw):
    import tinyinfer_amd as ti
    from tinyinfer_amd.weights import write_model_folder
    register_toys()
    d = str(tmp_path / "toy")
    write_model_folder(d, cfg, seed=9, dtype="float32")
    _, w = read_folder(d)
    engine = ti.Engine.from_folder(d, "float32", page_size=4, max_tokens=max_tokens, max_requests=2, max_seq=128, **kw)
    return engine, w


def test_toy_mixer_with_state_is_registered_built_and_stepped(tmp_path):
    import tinyinfer_amd as ti
    engine, w = toy_engine(tmp_path, TOY)
    kinds = [type(b.mixer).__name__ for b in engine.model.blocks]
    assert kinds == ["DecayMixer", "Attention", "DecayMixer"]
    # the two decay layers share a state group with two cache layers; attention has pages
    needs = [type(n).__name__ for n, _ in engine.model.cache_groups]
    assert sorted(needs) == ["PagedKVNeed", "StateNeed"]
    reqs = {r: random_tokens(n, 90, 5 + i) for i, (r, n) in enumerate({"a": 23, "b": 40, "c": 17}.items())}
    want = {r: toy_plain(TOY, w, t) for r, t in reqs.items()}

    def feed(r, lo, hi):
        return ti.StepEntry(r, reqs[r][lo:hi], list(range(hi - lo)))

    got = {r: [] for r in reqs}

    def run(entries):
        logits = engine.step(entries).cpu().numpy()
        i = 0
        for e in entries:
            got[e.request].append(logits[i:i + len(e.tokens)])
            i += len(e.tokens)

    # portions of a beside portions and single tokens of b; then c takes a's slot, whose
    # state must start from zero again
    run([feed("a", 0, 9), feed("b", 0, 2)])
    run([feed("a", 9, 10), feed("b", 2, 30)])
    run([feed("b", 30, 31), feed("a", 10, 23)])
    engine.release("a")
    run([feed("c", 0, 5), feed("b", 31, 40)])
    run([feed("c", 5, 17)])
    assert engine.cache.slot("c") == 0                      # the slot a held
    for r in reqs:
        assert np.abs(np.concatenate(got[r]) - want[r]).max() < 2e-4, r
    # parts from outside the library read token ids only: such an engine offers no token feedback,
    # and a token that names a row of it is refused like any id outside the vocabulary
    from tinyinfer_amd.engine import EngineError
    assert engine.feedback_rows == 0
    with pytest.raises(EngineError, match="outside the vocabulary"):
        engine.step([ti.StepEntry("c", [ti.token_from_feedback(0)], [0])])


def test_toy_mixer_with_pages_of_its_own(tmp_path):
    """A mixer that keeps a row of its own per token in pages (neither keys nor values) behind a window:
    registered in this file, built, stepped in portions beside another request, with so few pages that
    the ones the window has passed are handed out again; against the whole-sequence numpy model."""
    import tinyinfer_amd as ti
    cfg = dict(TOY, layers=["memory", "full", "memory"], memory_window=6)
    engine, w = toy_engine(tmp_path, cfg, max_tokens=72)
    needs = sorted(type(n).__name__ for n, _ in engine.model.cache_groups)
    assert needs == ["PagedKVNeed", "PagedRowsNeed"]
    groups = {type(n).__name__: i for i, (n, _) in enumerate(engine.model.cache_groups)}
    mem = groups["PagedRowsNeed"]
    assert engine.page_pool(mem, 1).shape == (18, 4, 32) and engine.page_pool(mem, 1).dtype == torch.float32
    reqs = {"a": random_tokens(50, 90, 3), "b": random_tokens(21, 90, 4)}
    want = {r: toy_plain(cfg, w, t) for r, t in reqs.items()}
    got = {r: [] for r in reqs}

    def run(entries):
        logits = engine.step(entries).cpu().numpy()
        i = 0
        for e in entries:
            got[e.request].append(logits[i:i + len(e.tokens)])
            i += len(e.tokens)

    def feed(r, lo, hi):
        return ti.StepEntry(r, reqs[r][lo:hi], list(range(hi - lo)))
    free_before = engine.cache.groups[mem].pool.num_free
    run([feed("a", 0, 13), feed("b", 0, 2)])
    run([feed("a", 13, 14), feed("b", 2, 21)])
    engine.release("b")
    for t in range(14, 30):
        run([feed("a", t, t + 1)])
    run([feed("a", 30, 50)])
    # behind the window of 6 the memory's pages have gone back: a request of 50 tokens holds at most 3 of them
    assert len([p for p in engine.cache.table(mem, "a") if p >= 0]) <= 3
    engine.cache.check()
    for r in reqs:
        assert np.abs(np.concatenate(got[r]) - want[r]).max() < 2e-4, r
    engine.release("a")
    assert engine.cache.groups[mem].pool.num_free == free_before


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("qk_norm,rotate,window", [(True, True, None), (False, False, None), (True, True, 9)])
def test_attention_part_alone(tmp_path, dtype, qk_norm, rotate, window):
    """The attention part by itself in a block of its own (no norms, no
    feed-forward), with and without per-head norm and rotation: without either it
    is plain softmax attention."""
    import tinyinfer_amd as ti
    from tinyinfer_amd.weights import write_model_folder
    register_toys()
    cfg = dict(TOY, layers=["bare_attention"], qk_norm=qk_norm, rotate=rotate, window=window, heads=4, kv_heads=2,
               head_dim=32 if dtype == "bfloat16" else 16, hidden=64)
    d = str(tmp_path / "attn")
    write_model_folder(d, cfg, seed=3, dtype="bfloat16")
    _, w = read_folder(d)
    if not qk_norm:
        assert not any("q_norm" in k for k in w)
    engine = ti.Engine.from_folder(d, dtype, page_size=16, max_tokens=128, max_requests=1, max_seq=128)
    toks = random_tokens(45, 90, 1)
    got = np.concatenate([engine.step([ti.StepEntry("r", toks[a:b], list(range(b - a)))]).cpu().numpy()
                          for a, b in ((0, 20), (20, 21), (21, 45))])
    want = toy_plain(cfg, w, toks)
    assert np.abs(got - want).max() < (2e-4 if dtype == "float32" else 5e-2)


def test_run_order_may_name_a_layer_twice(tmp_path):
    """layers [decay, full] run as 0, 1, 0, 1: every run keeps a cache of its own."""
    import tinyinfer_amd as ti
    cfg = dict(TOY, layers=["decay", "full"], schedule=[0, 1, 0, 1])
    engine, w = toy_engine(tmp_path, cfg)
    assert sorted(n for _, n in engine.model.cache_groups) == [2, 2]
    toks = random_tokens(30, 90, 2)
    got = np.concatenate([engine.step([ti.StepEntry("r", toks[a:b], list(range(b - a)))]).cpu().numpy()
                          for a, b in ((0, 11), (11, 12), (12, 30))])
    assert np.abs(got - toy_plain(cfg, w, toks)).max() < 2e-4


def test_toy_routed_feed_forward_and_another_position_encoding(tmp_path):
    """A feed-forward that routes tokens to experts and a position encoding that rotates
    neighbouring dims (no fused form: the attention part applies it to its 32-bit
    projections), defined above in this file, beside the built-in parts: portions and single
    tokens of two requests in one batch against the whole-sequence numpy model."""
    import tinyinfer_amd as ti
    cfg = dict(TOY, layers=["routed", "full", "routed"], experts=3, ff=40, heads=4, kv_heads=2)
    engine, w = toy_engine(tmp_path, cfg)
    assert [type(b.ffn).__name__ for b in engine.model.blocks] == ["RoutedFFN", "SwiGLU", "RoutedFFN"]
    assert type(engine.model.blocks[0].mixer.pos).__name__ == "PairRotary"
    reqs = {"a": random_tokens(37, 90, 21), "b": random_tokens(26, 90, 22)}
    want = {r: toy_plain(cfg, w, t) for r, t in reqs.items()}
    # every expert is used by some token (else the routing is not tested)
    got = {r: [] for r in reqs}

    def run(*cuts):
        entries = [ti.StepEntry(r, reqs[r][lo:hi], list(range(hi - lo))) for r, lo, hi in cuts]
        logits = engine.step(entries).cpu().numpy()
        i = 0
        for e in entries:
            got[e.request].append(logits[i:i + len(e.tokens)])
            i += len(e.tokens)

    run(("a", 0, 18), ("b", 0, 1))
    run(("a", 18, 19), ("b", 1, 20))
    run(("b", 20, 21), ("a", 19, 37))
    run(("b", 21, 26))
    for r in reqs:
        assert np.abs(np.concatenate(got[r]) - want[r]).max() < 2e-4, r
