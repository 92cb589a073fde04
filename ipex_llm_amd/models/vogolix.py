"""Vogolix: a pre-norm hybrid decoder whose layers mix a state-space mixer,
latent attention in a sliding window and chunked grouped attention with a
softmax sink (optionally on an earlier layer's keys and values), read from
its own checkpoint layout.

A checkpoint folder holds ``config.json`` (``"architecture": "Vogolix"``) and
``model.safetensors`` (bf16 weights, linear weights stored [out, in]).  The
configuration lists the layers in order; each entry names its mixer type
(``mamba2``, ``latent_attention``, ``attention``), the mixer's sizes and its
feed-forward (``dense`` or none).  Tensor names: ``embed``, ``l<i>.norm1`` /
``norm2``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``, ``final.norm``, ``head``.
Every size and constant comes from the configuration; the building blocks are
the generic ones of ``models/hybrid.py``:

* ``mamba2``            -> ``SSMMixer`` (``in``, ``conv`` + ``conv.b``, ``dt_bias``, ``A_log``, ``D``, ``norm``, ``o``)
* ``latent_attention``  -> ``LatentAttention`` with a window (``mask.size``), half-split rotary pairs on the
                           shared rotated key and an element-wise output gate (``q``, ``dkv`` + ``dkv.norm``,
                           ``uk``, ``uv``, ``g``, ``o``)
* ``attention``         -> ``MaskedAttention``: biased projections, RMS norm over the whole q / k projection,
                           neighbouring rotary pairs on the first ``rot.dims`` values of a head, chunks of
                           ``mask.size`` positions, a sink per head; ``kv_from: j`` reads layer j's cache rows
                           (``q`` ``k`` ``v`` + ``.b``, ``q.norm`` ``k.norm``, ``sink``, ``o``)
* feed-forward          -> ``DenseFF`` with a ReLU gate
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

from .hybrid import (DenseFF, DenseFFSpec, HybridCausalLM, HybridSpec, LatentAttention, LatentAttentionSpec, LayerSpec,
                     MaskedAttention, MaskedAttentionSpec, MaskSpec, PreNormLayer, RotarySpec, SSMMixer, SSMSpec)

ARCHITECTURE = "Vogolix"


def spec_from_config(cfg: dict) -> HybridSpec:
    layers = []
    raw = cfg["layers"]
    for i, L in enumerate(raw):
        m, kind = L["mixer"], L["type"]
        if kind == "mamba2":
            mixer = SSMSpec(heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]), groups=int(m["groups"]),
                            taps=int(m["conv"]), norm_groups=int(m.get("norm_groups", 1)))
            name = "ssm"
        elif kind == "latent_attention":
            rot = m["rot"]
            mixer = LatentAttentionSpec(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]),
                                        vdim=int(m["vdim"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                                        rot=RotarySpec(int(rot["dims"]), float(rot["base"]), None, "half"),
                                        out_gate=True, gate="element", window=int(m["mask"]["size"]))
            if mixer.rot.dims > mixer.rot_dim or mixer.rot.dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
            if mixer.window < 1:
                raise ValueError(f"layer {i}: mask.size must be at least 1")
            name = "latent_attention"
        elif kind == "attention":
            rot = m["rot"]
            src = m.get("kv_from")
            mixer = MaskedAttentionSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]), dim=int(m["dim"]),
                                        vdim=int(m["vdim"]), scale=float(m["scale"]),
                                        rot=RotarySpec(int(rot["dims"]), float(rot["base"]), None, "pairs"),
                                        mask=MaskSpec("chunk", int(m["mask"]["size"])), qk_norm="whole", bias=True,
                                        sink=True, kv_from=None if src is None else int(src))
            if mixer.rot.dims > mixer.dim or mixer.rot.dims % 2:
                raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
            if mixer.kv_from is not None:
                j = mixer.kv_from
                if not 0 <= j < i or raw[j]["type"] != "attention" or raw[j]["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys of its own")
                o = raw[j]["mixer"]
                if (int(o["kv_heads"]), int(o["dim"]), int(o["vdim"])) != (mixer.kv_heads, mixer.dim, mixer.vdim):
                    raise ValueError(f"layer {i}: layer {j}'s key / value sizes differ")
            name = "masked_attention"
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = L.get("mlp")
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            mlp = DenseFFSpec(int(mlp["ff"]), act="relu")
        layers.append(LayerSpec(name, mixer, mlp))
    return HybridSpec(model_type="vogolix", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                      norm_eps=float(cfg["norm"]["eps"]), block="pre_norm", norm="rms",
                      logit_scale=float(cfg.get("logit_scale", 1.0)))


def tensor_shapes(spec: HybridSpec) -> Dict[str, tuple]:
    """name -> shape of every tensor of a checkpoint of ``spec``"""
    W = spec.hidden_size
    out = {"embed": (spec.vocab_size, W)}
    for i, L in enumerate(spec.layers):
        p, m = f"l{i}.", L.mixer
        out[p + "norm1"] = (W,)
        if L.kind == "ssm":
            inner, gn = m.heads * m.vdim, m.groups * m.state
            out.update({p + "mix.in": (2 * inner + 2 * gn + m.heads, W), p + "mix.conv": (inner + 2 * gn, m.taps),
                        p + "mix.conv.b": (inner + 2 * gn,), p + "mix.dt_bias": (m.heads,), p + "mix.A_log": (m.heads,),
                        p + "mix.D": (m.heads,), p + "mix.norm": (inner,), p + "mix.o": (W, inner)})
        elif L.kind == "latent_attention":
            out.update({p + "mix.q": (m.heads * (m.dim + m.rot_dim), W), p + "mix.dkv": (m.kv_rank + m.rot_dim, W),
                        p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                        p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.g": (m.heads * m.vdim, W),
                        p + "mix.o": (W, m.heads * m.vdim)})
        else:
            out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.q.b": (m.heads * m.dim,),
                        p + "mix.q.norm": (m.heads * m.dim,), p + "mix.sink": (m.heads,),
                        p + "mix.o": (W, m.heads * m.vdim)})
            if m.kv_from is None:
                out.update({p + "mix.k": (m.kv_heads * m.dim, W), p + "mix.k.b": (m.kv_heads * m.dim,),
                            p + "mix.k.norm": (m.kv_heads * m.dim,), p + "mix.v": (m.kv_heads * m.vdim, W),
                            p + "mix.v.b": (m.kv_heads * m.vdim,)})
        if L.mlp is not None:
            out.update({p + "norm2": (W,), p + "mlp.gate": (L.mlp.ff, W), p + "mlp.up": (L.mlp.ff, W),
                        p + "mlp.down": (W, L.mlp.ff)})
    out["final.norm"] = (W,)
    out["head"] = (spec.vocab_size, W)
    return out


def build(spec: HybridSpec, tensors: Dict[str, torch.Tensor], dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    """Assemble the model from name -> tensor (any float dtype; cast to ``dtype``)."""
    want = tensor_shapes(spec)
    for name, shape in want.items():
        if name not in tensors:
            raise KeyError(f"checkpoint lacks tensor {name!r}")
        if tuple(tensors[name].shape) != tuple(shape):
            raise ValueError(f"tensor {name!r}: shape {tuple(tensors[name].shape)}, configuration says {tuple(shape)}")

    def t(name):
        return tensors[name].to(device=device, dtype=dtype).contiguous()

    layers = []
    for i, L in enumerate(spec.layers):
        p = f"l{i}.mix."
        if L.kind == "ssm":
            mixer = SSMMixer(L.mixer, t(p + "in"), t(p + "conv"), t(p + "conv.b"), t(p + "dt_bias"), t(p + "A_log"),
                             t(p + "D"), t(p + "norm"), t(p + "o"))
        elif L.kind == "latent_attention":
            mixer = LatentAttention(L.mixer, t(p + "q"), t(p + "dkv"), t(p + "dkv.norm"), t(p + "uk"), t(p + "uv"),
                                    t(p + "g"), t(p + "o"))
        else:
            own = L.mixer.kv_from is None
            mixer = MaskedAttention(L.mixer, t(p + "q"), t(p + "k") if own else None, t(p + "v") if own else None,
                                    t(p + "q.b"), t(p + "k.b") if own else None, t(p + "v.b") if own else None,
                                    t(p + "q.norm"), t(p + "k.norm") if own else None, t(p + "sink"), t(p + "o"))
        mlp, n2 = None, None
        if L.mlp is not None:
            q = f"l{i}.mlp."
            mlp, n2 = DenseFF(t(q + "gate"), t(q + "up"), t(q + "down"), act=L.mlp.act), t(f"l{i}.norm2")
        layers.append(PreNormLayer(mixer, t(f"l{i}.norm1"), mlp, n2))
    return HybridCausalLM(spec, t("embed"), None, layers, t("final.norm"), t("head"), dtype).eval()


def load(path: str, dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    """Read ``config.json`` + ``model.safetensors`` of a checkpoint folder."""
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    spec = spec_from_config(cfg)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), "pt") as f:
        names = set(f.keys())
        for name in tensor_shapes(spec):
            if name in names:
                tensors[name] = f.get_tensor(name)
    model = build(spec, tensors, dtype, device)
    model.config = cfg
    return model


@torch.no_grad()
def random_tensors(spec: HybridSpec, seed: int = 0, std: Optional[float] = None) -> Dict[str, torch.Tensor]:
    """Random bf16 weights of ``spec``'s shapes (benchmarks and tests)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(spec).items():
        if name.endswith(("norm1", "norm2", "final.norm", "mix.norm", "dkv.norm", "q.norm", "k.norm", "mix.D")):
            w = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith(("dt_bias", "A_log")):
            w = -1.0 + 0.5 * torch.randn(shape, generator=g)
        elif name.endswith((".b", "sink")):
            w = 0.3 * torch.randn(shape, generator=g)
        elif name.endswith("mix.conv"):
            w = 0.5 * torch.randn(shape, generator=g)
        elif len(shape) == 2 and name != "embed":
            w = torch.randn(shape, generator=g) * (std if std is not None else shape[1] ** -0.5)
        else:
            w = torch.randn(shape, generator=g) * (std if std is not None else 1.0)
        out[name] = w.to(torch.bfloat16)
    return out


def random_model(spec: HybridSpec, seed: int = 0, dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    return build(spec, random_tensors(spec, seed), dtype, device)
