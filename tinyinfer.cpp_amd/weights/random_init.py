"""Random weights from a configuration and a seed, and a model folder written
from them.

Matrices and the embedding ~ N(0, 0.02); every RMSNorm weight (input,
post-attention, per-head q/k, final) = 1 + N(0, 0.1), so that a norm weight
that is forgotten or put in the wrong place changes the logits.  The
distribution of each tensor is the one its part declares; tensors are drawn in
the model's own fixed order from one generator, so a seed fixes every bit.
The reference has no such mode (it loads GGUF files only).
"""
from __future__ import annotations

import json
import os
from typing import Dict, Mapping

import torch

from .safetensors_io import write_safetensors
from ..models.model import Model
from ..registry import config_and_spec


def random_tensors(model: Model, seed: int, matrix_dtype: torch.dtype = torch.bfloat16,
                   device: str = "cpu") -> Dict[str, torch.Tensor]:
    """name -> tensor for every tensor the model requires.  Values are drawn in
    float32 and rounded once to `matrix_dtype` (matrices) or kept in float32
    (vectors).  Optional tensors are not written."""
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out: Dict[str, torch.Tensor] = {}
    for name, need in model.tensors().items():
        if need.optional:
            continue
        kind, a, b = need.init
        if need.role == "table":
            t = torch.randint(int(a), int(b), need.shape, generator=gen, device=device, dtype=torch.int32)
        elif kind == "normal":
            t = torch.randn(need.shape, generator=gen, device=device, dtype=torch.float32) * b + a
        elif kind == "uniform":
            t = torch.rand(need.shape, generator=gen, device=device, dtype=torch.float32) * (b - a) + a
        elif kind == "constant":
            t = torch.full(need.shape, float(a), device=device, dtype=torch.float32)
        else:
            raise ValueError(f"tensor '{name}': unknown init {need.init!r}")
        if need.role == "matrix":
            t = t.to(matrix_dtype)
        out[name] = t
    return out


def write_model_folder(path: str, config: Mapping, seed: int, dtype: str = "bfloat16") -> Dict[str, torch.Tensor]:
    """Write `path/config.json` and `path/model.safetensors` for the architecture
    that `config` (a config.json dict) names.  `dtype` is how matrices are stored.
    A head tied to the embedding (or left open with `tie_word_embeddings` absent)
    stores no `lm_head.weight`."""
    cfg, spec = config_and_spec(config)
    model = Model(spec)
    tensors = random_tensors(model, seed, {"bfloat16": torch.bfloat16, "float32": torch.float32}[dtype])
    os.makedirs(path, exist_ok=True)
    out_cfg = cfg.to_dict() if hasattr(cfg, "to_dict") else dict(config)
    out_cfg["torch_dtype"] = dtype
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(out_cfg, f, indent=1)
    write_safetensors(os.path.join(path, "model.safetensors"), tensors,
                      {"format": "pt", "seed": str(seed)})
    return tensors


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
    tensors = write_model_folder(args.out, config, args.seed, args.dtype)
    n = sum(t.numel() for t in tensors.values())
    print(f"wrote {args.out}: {len(tensors)} tensors, {n} parameters, seed {args.seed}, matrices in {args.dtype}")
    return 0


if __name__ == "__main__":
    import sys
    sys.exit(main())
