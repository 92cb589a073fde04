"""Prefill / decode throughput of a pre-norm hybrid decoder (Vogolix layout:
chunked grouped attention with a sink, a layer that borrows its keys and
values, a state-space mixer, latent attention in a window; ReLU-gated
feed-forward) at layer sizes of a real model, beside the framework's closest
existing model -- the hybrid decoder of latent attention and mLSTM layers
(Zamelix layout, models/zamelix.py: paged rows + recurrent state slots, the
same ragged serving steps) -- at equal width, feed-forward and latent-attention
sizes and as many layers.  Random bf16 weights, synthetic tokens.
Run through ``bench.py --prenorm``; one JSON line.

Both models go through ``LLMEngine.feed``.  Prefill: one request of P tokens
in one step, tokens / s.  Decode: B sequences at context P, one token each per
step (hipGraph on both sides), tokens / s.
"""
from __future__ import annotations

import json
import sys
import time
from typing import Dict, List

import torch

SIZES = {
    # width, vocab, ff; attention (heads, kv heads, dim, vdim, rotated dims, chunk); state-space (heads, vdim, state,
    # groups, taps, norm groups); latent attention (heads, dim, rot, vdim, rank, window); mLSTM of the comparison
    # model (heads, dim, vdim); blocks of four layers.  The chunks do not divide the prompt lengths, so prompts end
    # and decoding runs inside a chunk (256 and 1024 keys in view)
    "small": dict(width=1024, vocab=32000, ff=2816, attn=(8, 2, 128, 128, 64, 768), ssm=(32, 64, 128, 1, 4, 1),
                  latent=(8, 64, 32, 64, 256, 1024), mlstm=(4, 64, 256), blocks=1),
    "base": dict(width=2048, vocab=32000, ff=5632, attn=(16, 4, 128, 128, 64, 1536), ssm=(64, 64, 128, 8, 4, 8),
                 latent=(16, 128, 64, 128, 512, 2048), mlstm=(4, 256, 512), blocks=1),
}


def prenorm_config(sz: dict) -> dict:
    H, G, d, dv, rd, chunk = sz["attn"]
    sh, sp, sn, sg, taps, ng = sz["ssm"]
    lh, ld, lr, lv, rank, win = sz["latent"]
    mlp = {"kind": "dense", "ff": sz["ff"]}
    attn = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5, "mask": {"size": chunk},
            "rot": {"base": 10000.0, "dims": rd}}
    layers = []
    for b in range(sz["blocks"]):
        layers += [{"type": "attention", "mixer": dict(attn), "mlp": mlp},
                   {"type": "mamba2", "mixer": {"heads": sh, "vdim": sp, "state": sn, "groups": sg, "conv": taps,
                                                "norm_groups": ng}, "mlp": mlp},
                   {"type": "attention", "mixer": dict(attn, kv_from=4 * b), "mlp": mlp},
                   {"type": "latent_attention",
                    "mixer": {"heads": lh, "dim": ld, "rot_dim": lr, "vdim": lv, "kv_rank": rank,
                              "scale": (ld + lr) ** -0.5, "mask": {"size": win}, "rot": {"base": 10000.0, "dims": lr}},
                    "mlp": mlp}]
    return {"architecture": "Vogolix", "vocab": sz["vocab"], "width": sz["width"], "norm": {"eps": 1e-6},
            "logit_scale": 1.0, "layers": layers}


def reference_config(sz: dict) -> dict:
    """latent attention of the same sizes (unbounded view) and mLSTM layers, a feed-forward on every layer"""
    lh, ld, lr, lv, rank, _ = sz["latent"]
    mh, md, mv = sz["mlstm"]
    mlp = {"kind": "dense", "ff": sz["ff"]}
    attn = {"type": "latent_attention",
            "mixer": {"heads": lh, "dim": ld, "rot_dim": lr, "vdim": lv, "kv_rank": rank, "scale": (ld + lr) ** -0.5,
                      "rot": {"base": 10000.0, "dims": lr}}, "mlp": mlp}
    rec = {"type": "mlstm", "mixer": {"heads": mh, "dim": md, "vdim": mv, "gate_cap": 15.0}, "mlp": mlp}
    return {"architecture": "Zamelix", "vocab": sz["vocab"], "width": sz["width"], "norm": {"eps": 1e-6},
            "residual_mult": 0.5, "layers": [attn, rec] * (2 * sz["blocks"])}


def _sync_time(fn, dev, reps: int) -> float:
    torch.cuda.synchronize(dev)
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize(dev)
    return (time.perf_counter() - t0) / reps


def bench_model(model, dev, prompt_len: int, batch: int, steps: int, warmup: int) -> Dict[str, float]:
    from ..serving.engine import LLMEngine
    total = prompt_len + warmup + steps + 8
    nblk = batch * (-(-total // 64))
    eng = LLMEngine(model, max_batch=batch, block_size=64, num_blocks=nblk, max_model_len=total,
                    max_prefill_tokens=1 << 30, use_graph=True, enable_prefix_caching=False)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, model.spec.vocab_size, (prompt_len,), generator=g).tolist() for _ in range(batch)]
    times = []
    for rep in range(3):
        rid = eng.open_stream()
        torch.cuda.synchronize(dev)
        t0 = time.perf_counter()
        eng.feed([(rid, prompts[0], [prompt_len - 1])])
        torch.cuda.synchronize(dev)
        times.append(time.perf_counter() - t0)
        eng.close_stream(rid)
    prefill_s = min(times[1:])
    rids = [eng.open_stream() for _ in range(batch)]
    eng.feed([(r, p, [prompt_len - 1]) for r, p in zip(rids, prompts)])
    tok = [[1 + i] for i in range(batch)]

    def step():
        eng.feed([(r, t, [0]) for r, t in zip(rids, tok)])
    for _ in range(warmup):
        step()
    decode_s = _sync_time(step, dev, steps)
    for r in rids:
        eng.close_stream(r)
    return {"prefill_tok_s": prompt_len / prefill_s, "prefill_ms": prefill_s * 1e3,
            "decode_tok_s": batch / decode_s, "decode_ms_per_step": decode_s * 1e3}


def main(args) -> dict:
    from ..models import vogolix as V, zamelix as Z
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    out: List[dict] = []
    for name in args.prenorm_sizes.split(","):
        sz = SIZES[name]
        for P in [int(p) for p in args.prenorm_prompts.split(",")]:
            row = {"size": name, "prompt_len": P, "batch": args.batch}
            model = V.random_model(V.spec_from_config(prenorm_config(sz)), 0, torch.bfloat16, dev)
            row["prenorm"] = {k: round(v, 3) for k, v in bench_model(model, dev, P, args.batch, args.steps, args.warmup).items()}
            del model
            if not args.no_prenorm_ref:
                ref = Z.random_model(Z.spec_from_config(reference_config(sz)), 0, torch.bfloat16, dev)
                row["hybrid_reference"] = {k: round(v, 3) for k, v in
                                           bench_model(ref, dev, P, args.batch, args.steps, args.warmup).items()}
                del ref
            torch.cuda.empty_cache()
            out.append(row)
            print(json.dumps(row), file=sys.stderr, flush=True)
    res = {"metric": "pre-norm hybrid decoder prefill / decode throughput (random weights, synthetic tokens)",
           "unit": "tokens/s", "dtype": "bf16", "data": "synthetic", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "rows": out}
    print(json.dumps(res))
    return res
