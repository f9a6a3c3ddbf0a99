"""Random weights from a configuration and a seed, and a model folder written
from them.

Matrices and the embedding ~ N(0, 0.02); every RMSNorm weight (input,
post-attention, per-head q/k, final) = 1 + N(0, 0.1), so that a norm weight
that is forgotten or put in the wrong place changes the logits.  The
distribution of each tensor is the one its part declares; a tensor's values are
a pure function of the seed, its name and the element's index
(weights/weights.cpp `host_random`; the device draws the same in
csrc/core.hip), so a seed fixes every bit.  The reference has no such mode (it
loads GGUF files only).
"""
from __future__ import annotations

import json
from typing import Mapping

from .. import native
from ..models.model import Model
from ..registry import config_and_spec


def write_model_folder(path: str, config: Mapping, seed: int, dtype: str = "bfloat16") -> None:
    """Write `path/config.json` and `path/model.safetensors` for the architecture that `config` (a
    config.json dict) names.  `dtype` is how matrices are stored.  A head tied to the embedding (or
    left open with `tie_word_embeddings` absent) stores no `lm_head.weight`."""
    if dtype not in ("bfloat16", "float32"):
        raise ValueError(f"dtype must be bfloat16 or float32, got {dtype!r}")
    cfg, spec = config_and_spec(config)
    model = Model(spec)
    out_cfg = cfg.to_dict() if hasattr(cfg, "to_dict") else dict(config)
    native.call("ti_model_write_random_folder", model._ptr, path.encode(), json.dumps(out_cfg).encode(), int(seed),
                dtype.encode())


def main(argv=None) -> int:
    """python -m tinyinfer_amd.weights.random_init CONFIG.json OUT_DIR [--seed S] [--dtype bfloat16|float32]"""
    import argparse
    ap = argparse.ArgumentParser(description="write a model folder (config.json, model.safetensors) with random "
                                             "weights from a configuration and a seed")
    ap.add_argument("config", help="a config.json of a registered architecture")
    ap.add_argument("out", help="folder to write")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16",
                    help="how matrices are stored (norm weights are stored in float32)")
    args = ap.parse_args(argv)
    with open(args.config, "r", encoding="utf-8") as f:
        config = json.load(f)
    write_model_folder(args.out, config, args.seed, args.dtype)
    print(f"wrote {args.out}: seed {args.seed}, matrices in {args.dtype}")
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())
