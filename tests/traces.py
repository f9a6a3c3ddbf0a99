"""Ways of cutting the same requests into steps.

A trace is a list of steps; a step is `{"entries": [(request, tokens, want)], "end": [requests]}`.
Every generator wants the logits of every token it feeds, so that each position
of each request can be compared with the plain implementation, whatever the cut.
`max_tokens(trace)` is the pool size the replay tool is given: the most tokens
live requests hold at any time, each request's count rounded up to 64.
"""
from typing import Dict, List, Sequence


def whole(requests: Dict[str, Sequence[int]]):
    """Each request alone and whole, one step each."""
    steps = []
    for rid, toks in requests.items():
        steps.append({"entries": [(rid, list(toks), list(range(len(toks))))], "end": [rid]})
    return steps


def tail_one_by_one(requests: Dict[str, Sequence[int]], tail: int = 32):
    """Most of a request in one step, then its last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        head = max(1, len(toks) - tail)
        steps.append({"entries": [(rid, toks[:head], list(range(head)))], "end": []})
        for i in range(head, len(toks)):
            steps.append({"entries": [(rid, [toks[i]], [0])], "end": []})
        steps[-1]["end"] = [rid]
    return steps


PORTIONS = (7, 5, 3, 2, 2, 11, 1, 4, 2, 13, 2, 6)


def portions(requests: Dict[str, Sequence[int]], sizes: Sequence[int] = PORTIONS):
    """Each request alone, in portions of changing size, down to two tokens (and one)."""
    steps = []
    for rid, toks in requests.items():
        toks = list(toks)
        i = k = 0
        while i < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - i)
            steps.append({"entries": [(rid, toks[i:i + n], list(range(n)))], "end": []})
            i += n
            k += 1
        steps[-1]["end"] = [rid]
    return steps


def mixed(requests: Dict[str, Sequence[int]], prompt_len: Dict[str, int], live: int = 4,
          sizes: Sequence[int] = PORTIONS):
    """Up to `live` requests at a time.  A request is fed in portions up to its
    `prompt_len`, then token by token; portions of some requests stand beside
    single tokens of others; a request that is done ends and the next one in
    line starts in the following step, so its pages go to the newcomer.  Every
    third step one live request sits out."""
    waiting = list(requests)
    fed = {r: 0 for r in requests}
    active: List[str] = []
    steps = []
    k = 0
    while waiting or active:
        while waiting and len(active) < live:
            active.append(waiting.pop(0))
        entries = []
        ended = []
        for j, rid in enumerate(list(active)):
            toks = list(requests[rid])
            if len(active) > 1 and k % 3 == 2 and j == (k // 3) % len(active):
                continue                         # left out of this step, goes on later
            i = fed[rid]
            if i < prompt_len[rid]:
                n = min(sizes[(k + j) % len(sizes)], prompt_len[rid] - i)
            else:
                n = 1
            entries.append((rid, toks[i:i + n], list(range(n))))
            fed[rid] = i + n
            if fed[rid] == len(toks):
                ended.append(rid)
        for rid in ended:
            active.remove(rid)
        if entries:
            steps.append({"entries": entries, "end": ended})
        k += 1
    return steps


def at_random(requests: Dict[str, Sequence[int]], seed: int, live: int = 4):
    """Up to `live` requests at a time, drawn from a seed: which of them a step feeds (at least one;
    the others sit out), how many tokens each gets (1 most often, else 2 to 40), and which of those
    places are wanted (the last one always, so that a request can be followed; others at random, so
    that the rows a step leaves out lie at changing places).  A request that is done ends at once;
    the next in line takes its place in a later step."""
    import random
    rng = random.Random(seed)
    waiting = list(requests)
    rng.shuffle(waiting)
    fed = {r: 0 for r in requests}
    active: List[str] = []
    steps = []
    while waiting or active:
        while waiting and len(active) < live and (not active or rng.random() < 0.6):
            active.append(waiting.pop(0))
        chosen = [r for r in active if rng.random() < 0.7] or [rng.choice(active)]
        rng.shuffle(chosen)                                  # the rows of a step in changing order
        entries, ended = [], []
        for rid in chosen:
            toks = list(requests[rid])
            left = len(toks) - fed[rid]
            n = 1 if rng.random() < 0.55 else rng.choice((2, 2, 3, 5, 8, 13, 16, 17, 31, 40))
            n = min(n, left)
            want = sorted(set([n - 1] + [i for i in range(n - 1) if rng.random() < 0.3]))
            entries.append((rid, toks[fed[rid]:fed[rid] + n], want))
            fed[rid] += n
            if fed[rid] == len(toks):
                ended.append(rid)
        for rid in ended:
            active.remove(rid)
        steps.append({"entries": entries, "end": ended})
    return steps


def max_tokens(trace) -> int:
    held: Dict[str, int] = {}
    worst = 0
    for step in trace:
        for rid, toks, _ in step["entries"]:
            held[rid] = held.get(rid, 0) + len(toks)
        worst = max(worst, sum(-(-n // 64) * 64 for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return worst


def max_pages(trace, page_size: int) -> int:
    """The fewest pages that hold the trace: the most pages live requests need at any time."""
    held: Dict[str, int] = {}
    worst = 0
    for step in trace:
        for rid, toks, _ in step["entries"]:
            held[rid] = held.get(rid, 0) + len(toks)
        worst = max(worst, sum(-(-n // page_size) for n in held.values()))
        for rid in step["end"]:
            held.pop(rid, None)
    return worst


def to_jsonl(trace) -> str:
    import json
    lines = []
    for i, step in enumerate(trace):
        lines.append(json.dumps({
            "step": i,
            "entries": [{"id": r, "tokens": list(t), "want": list(w)} for r, t, w in step["entries"]],
            "end": list(step["end"])}))
    return "\n".join(lines) + "\n"
