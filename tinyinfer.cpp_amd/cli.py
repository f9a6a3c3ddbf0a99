"""Command line in the manner of the reference's `tinyinfer`
(/root/reference/src/main.cpp:86-162, README.md:88-98):

    tinyinfer -m MODEL_DIR -n max_tokens -p "prompt" [-p "prompt2" ...] [-f prompts.txt]
              [-t temp] [--top-k K] [--top-p P] [--seed S] [--max-seq N] [--cuda-graph] [--verbose]
              [--dtype D] [--page-size P] [--num-pages N] [--chunk N] [--max-batched-tokens N] [--random-weights]

-m is a model folder (config.json and safetensors) instead of a GGUF file; with
--random-weights a config.json alone is enough, and the weights are drawn on the device from --seed.  A
prompt is a list of token ids ("1,2,3" or "1 2 3"); if the folder holds a
`tokenizer.json`, any other prompt is text and is tokenized with it, and outputs
are printed as text too.  `-f` reads one prompt per non-empty line.  Results go
to stdout in the reference's format, timings to stderr.
"""
from __future__ import annotations

import os
import sys
import time
from typing import List, Optional


USAGE = """usage: {prog} -m model_dir -n max_tokens -p "prompt" [-p "prompt2" ...] [-f prompts.txt]
  [-t temp] [--top-k K] [--top-p P] [--seed S] [--max-seq N] [--cuda-graph] [--verbose]
  [--dtype bfloat16|float32] [--page-size P] [--num-pages N] [--chunk N] [--max-batched-tokens N]
  [--random-weights]
  --random-weights: -m needs a config.json only; the weights are drawn on the device from --seed
  --num-pages: pages in the cache pool (default: enough for --max-seq tokens of every prompt)
  a prompt is a list of token ids ("1,2,3"), or text if the model folder has a tokenizer.json
  --cuda-graph (alias --graph): replay decode steps, and other steps whose shape repeats, from captured graphs (off by default)
"""


def _read_prompts_file(path: str) -> List[str]:
    out = []
    with open(path, "rb") as f:
        for line in f.read().decode("utf-8").split("\n"):
            if line.endswith("\r"):
                line = line[:-1]
            if line:
                out.append(line)
    return out


def _as_ids(text: str) -> Optional[List[int]]:
    parts = text.replace(",", " ").split()
    try:
        return [int(p) for p in parts] if parts else None
    except ValueError:
        return None


def main(argv: Optional[List[str]] = None) -> int:
    argv = list(sys.argv if argv is None else argv)
    prog, args = argv[0], argv[1:]
    if os.environ.get("TINY_SELFTEST") == "1":
        # every kernel against a CPU computation; the exit code counts the failures
        # (the reference's QWEN_SELFTEST=1: /root/reference/src/main.cpp:123-125)
        from .selftest import run_selftest
        return run_selftest()
    model = None
    prompts: List[str] = []
    n_predict, temp, top_k, top_p, seed, max_seq = 128, 0.0, 0, 1.0, 42, 2048
    graph = verbose = chat = False
    dtype, page_size, chunk, budget = "bfloat16", 16, 512, 2048
    num_pages, random_weights = None, False

    def usage() -> int:
        sys.stderr.write(USAGE.format(prog=os.path.basename(prog)))
        return 1

    i = 0
    try:
        while i < len(args):
            a = args[i]
            has = i + 1 < len(args)
            if a == "-m" and has:
                model = args[i + 1]; i += 2
            elif a == "-n" and has:
                n_predict = int(args[i + 1]); i += 2
            elif a == "-p" and has:
                prompts.append(args[i + 1]); i += 2
            elif a == "-f" and has:
                try:
                    prompts.extend(_read_prompts_file(args[i + 1]))
                except OSError:
                    sys.stderr.write(f"main: cannot read prompts file {args[i + 1]}\n")
                    return 1
                i += 2
            elif a == "-t" and has:
                temp = float(args[i + 1]); i += 2
            elif a == "--top-k" and has:
                top_k = int(args[i + 1]); i += 2
            elif a == "--top-p" and has:
                top_p = float(args[i + 1]); i += 2
            elif a == "--seed" and has:
                seed = int(args[i + 1]); i += 2
            elif a == "--max-seq" and has:
                max_seq = int(args[i + 1]); i += 2
            elif a in ("--cuda-graph", "--graph"):
                graph = True; i += 1
            elif a == "--verbose":
                verbose = True; i += 1
            elif a == "--chat":
                chat = True; i += 1
            elif a == "--dtype" and has:
                dtype = args[i + 1]; i += 2
            elif a == "--page-size" and has:
                page_size = int(args[i + 1]); i += 2
            elif a == "--num-pages" and has:
                num_pages = int(args[i + 1]); i += 2
            elif a == "--random-weights":
                random_weights = True; i += 1
            elif a == "--chunk" and has:
                chunk = int(args[i + 1]); i += 2
            elif a == "--max-batched-tokens" and has:
                budget = int(args[i + 1]); i += 2
            else:
                return usage()
    except ValueError:
        return usage()
    if not model or not prompts:
        return usage()
    if dtype not in ("bfloat16", "float32"):
        return usage()

    tokenizer = None
    tok_path = os.path.join(model, "tokenizer.json")
    if os.path.isfile(tok_path):
        from tokenizers import Tokenizer
        tokenizer = Tokenizer.from_file(tok_path)
    ids: List[List[int]] = []
    for p in prompts:
        t = None if chat else _as_ids(p)
        if t is None:
            if tokenizer is None:
                sys.stderr.write("main: a prompt that is not a list of token ids needs a tokenizer.json "
                                 "in the model folder\n")
                return 1
            text = p
            if chat:
                # the reference's chat wrapping, thinking switched off: src/main.cpp:188-193
                text = ("<|im_start|>user\n" + p + "<|im_end|>\n<|im_start|>assistant\n<think>\n\n</think>\n\n")
            t = tokenizer.encode(text, add_special_tokens=False).ids
        if not t:
            sys.stderr.write("main: empty prompts\n")
            return 1
        ids.append(t)

    import tinyinfer_amd as ti
    from tinyinfer_amd.weights import WeightsError, FileError
    try:
        n_req = max(1, min(len(ids), 64))
        llm = ti.LLM(model, dtype=dtype, max_seq=max_seq, max_requests=n_req, page_size=page_size,
                     chunk_size=chunk, max_batched_tokens=budget, use_graph=graph, num_pages=num_pages,
                     random_seed=seed if random_weights else None)
    except (ti.ConfigError, WeightsError, FileError, FileNotFoundError) as e:
        sys.stderr.write(f"main: {e}\n")
        return 1
    if verbose:
        for s, t in enumerate(ids):
            sys.stderr.write(f"prompt {s} tokens: {len(t)}\n")

    def show_logits(s, row):
        # the first five logits and the five largest behind each prompt, as the reference's --verbose prints them
        # (/root/reference/src/main.cpp:233-249)
        import numpy as np
        top = np.lexsort((np.arange(row.shape[0]), -row))[:5]            # descending, the lowest id first among equals
        piece = (lambda t: tokenizer.id_to_token(int(t)) or "") if tokenizer is not None else (lambda t: "")
        sys.stderr.write(f"prefill logits seq {s} (first 5, top 5):" + "".join(f" {v:.3f}" for v in row[:5]) + " | top5:" +
                         "".join(f" {int(t)}({piece(t)}):{row[t]:.3f}" for t in top) + "\n")

    t0 = time.perf_counter()
    try:
        outs = llm.generate(ids, max_new_tokens=n_predict, temperature=temp, top_k=top_k, top_p=top_p, seed=seed,
                            on_prompt_logits=show_logits if verbose else None)
    except RuntimeError as e:
        sys.stderr.write(f"main: {e}\n")
        return 1
    wall = (time.perf_counter() - t0) * 1e3
    for s, (p, o) in enumerate(zip(prompts, outs)):
        print(f"==================== prompt {s} ====================")
        print(f"[prompt] {p}")
        if tokenizer is not None and _as_ids(p) is None:
            print(f"[output] {tokenizer.decode(o)}")
        else:
            print("[output] " + " ".join(str(t) for t in o))
    st = llm.last_stats
    sys.stderr.write(f"main: prefill: {st.prefill_ms:.1f} ms ({st.prefill_tokens} tokens)\n")
    rate = st.decode_tokens / (st.decode_ms / 1000.0) if st.decode_ms > 0 else 0.0
    sys.stderr.write(f"main: decode: {st.decode_ms:.1f} ms, {st.decode_tokens} tokens, {rate:.1f} tok/s "
                     f"[hip-graph: {'on' if graph else 'off'}] (wall {wall:.1f} ms, {st.steps} steps, "
                     f"{st.preemptions} preemptions)\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
