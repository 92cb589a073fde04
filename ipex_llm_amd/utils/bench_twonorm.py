"""Prefill / decode throughput of a decoder of two-norm parallel blocks
(Zoguzen layout: chunked grouped attention with mixed head weights, a layer
that borrows its keys and values, minGRU, windowed attention side by side with
gated linear attention; softmax-routed experts and a token-side input on every
layer) at layer sizes of a real model, beside the framework's closest existing
model -- the parallel-residual decoder with mixed-score grouped attention,
sigmoid-routed experts and the same token-side input (Masezen layout,
models/masezen.py: the same ragged serving steps, paged rows and state slots)
-- at equal width, attention sizes, expert count / size and as many layers.
Random bf16 weights, synthetic tokens.  Run through ``bench.py --twonorm``;
one JSON line.

Both models go through ``LLMEngine.feed``.  Prefill: one request of P tokens
in one step, tokens / s.  Decode: B sequences at context P, one token each per
step (hipGraph on both sides), tokens / s.
"""
from __future__ import annotations

import json
import sys
from typing import List

import torch

from .bench_prenorm import bench_model

SIZES = {
    # width, vocab; attention (heads, kv heads, dim, vdim, chunk, window, kept first tokens, rotated dims); taps of the
    # q / k / v convolutions; minGRU width; gated linear attention (heads, dim, vdim, decay rank, tau); experts
    # (count, top, ff); blocks of four layers.  The chunk does not divide the prompt lengths, so prompts end and
    # decoding runs inside a chunk
    "small": dict(width=1024, vocab=32000, attn=(8, 2, 128, 128, 768, 1024, 8, 64), taps=4, gru=2048,
                  gla=(8, 64, 128, 32, 8.0), moe=(8, 2, 1024), blocks=1),
    "base": dict(width=2048, vocab=32000, attn=(16, 4, 128, 128, 1536, 2048, 8, 64), taps=4, gru=4096,
                 gla=(16, 64, 128, 64, 8.0), moe=(16, 2, 1408), blocks=1),
}


def twonorm_config(sz: dict) -> dict:
    H, G, d, dv, chunk, win, keep, rd = sz["attn"]
    gh, gd, gv, rank, tau = sz["gla"]
    E, top, ff = sz["moe"]
    mlp = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": ff}}
    attn = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": sz["taps"], "scale": d ** -0.5, "softcap": 50.0,
            "mask": {"size": chunk}}
    left = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": sz["taps"], "scale": d ** -0.5,
            "mask": {"size": win, "keep_first": keep},
            "rot": {"base": 500000.0, "dims": rd, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    right = {"heads": gh, "dim": gd, "vdim": gv, "tau": tau, "rank": rank}
    layers = []
    for b in range(sz["blocks"]):
        layers += [{"type": "attention", "mixer": dict(attn), "mlp": mlp},
                   {"type": "mingru", "mixer": {"width": sz["gru"]}, "mlp": mlp},
                   {"type": "attention", "mixer": dict(attn, kv_from=4 * b), "mlp": mlp},
                   {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}]
    return {"architecture": "Zoguzen", "vocab": sz["vocab"], "width": sz["width"], "norm": {"eps": 1e-6},
            "token_side": {"dim": 64}, "logit_softcap": 50.0, "layers": layers}


def reference_config(sz: dict) -> dict:
    """mixed-score grouped attention of the same head sizes on every layer, experts of the same count and size
    (plus that design's shared expert), the same token-side input"""
    H, G, d, _, _, _, _, rd = sz["attn"]
    E, top, ff = sz["moe"]
    mixer = {"heads": H, "kv_heads": G, "dim": d, "vdim": d, "scale": d ** -0.5, "rot": {"base": 10000.0, "dims": rd}}
    mlp = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": ff, "limit": 7.0},
           "shared": {"ff": ff, "limit": 7.0}}
    return {"architecture": "Masezen", "vocab": sz["vocab"], "width": sz["width"], "norm": {"eps": 1e-6},
            "canon": {"taps": sz["taps"]}, "token_side": {"dim": 64},
            "layers": [{"type": "attention", "mixer": mixer, "mlp": mlp} for _ in range(4 * sz["blocks"])]}


def main(args) -> dict:
    from ..models import masezen as M, zoguzen as Z
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    out: List[dict] = []
    for name in args.twonorm_sizes.split(","):
        sz = SIZES[name]
        for P in [int(p) for p in args.twonorm_prompts.split(",")]:
            row = {"size": name, "prompt_len": P, "batch": args.batch}
            model = Z.random_model(Z.spec_from_config(twonorm_config(sz)), 0, torch.bfloat16, dev)
            row["twonorm"] = {k: round(v, 3) for k, v in bench_model(model, dev, P, args.batch, args.steps, args.warmup).items()}
            del model
            if not args.no_twonorm_ref:
                ref = M.random_model(M.spec_from_config(reference_config(sz)), 0, torch.bfloat16, dev)
                row["parallel_reference"] = {k: round(v, 3) for k, v in
                                             bench_model(ref, dev, P, args.batch, args.steps, args.warmup).items()}
                del ref
            torch.cuda.empty_cache()
            out.append(row)
            print(json.dumps(row), file=sys.stderr, flush=True)
    res = {"metric": "two-norm parallel-block decoder prefill / decode throughput (random weights, synthetic tokens)",
           "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "rows": out}
    print(json.dumps(res))
    return res
