"""Zoguzen: a decoder of two-norm parallel blocks -- a token-shifted mixer
(minGRU, chunked grouped attention with mixed head weights, or a sliding-window
attention side by side with gated linear attention) beside softmax-routed
experts, then a token-side input -- read from its own checkpoint layout.

A checkpoint folder holds ``config.json`` (``"architecture": "Zoguzen"``) and
``model.safetensors`` (bf16 weights, linear weights stored [out, in]).  The
configuration lists the layers in order; each entry names its mixer type
(``mingru``, ``attention``, ``parallel``), the mixer's sizes and its
feed-forward (``moe`` or none).  Tensor names: ``embed`` (also the head),
``side.embed``, ``l<i>.norm1`` / ``norm2`` / ``shift``, ``l<i>.mix.<name>``,
``l<i>.mlp.e<k>.<name>`` / ``router``, ``l<i>.side.<name>``, ``final.norm``.
Every size and constant comes from the configuration (the rank of the decay
projection from its tensor); the building blocks are the generic ones of
``models/hybrid.py``:

* ``mingru``     -> ``MinGRU`` (``z`` ``x`` + ``.b``, ``g``, ``o``)
* ``attention``  -> ``MaskedAttention``: biased projections, short convolutions on q / k / v, RMS norm per head,
                    no rotation, capped scores, chunks of ``mask.size`` positions, a sink of score 0, the heads'
                    weights mixed by ``talk`` after the softmax; ``kv_from: j`` reads layer j's cache rows
* ``parallel``   -> ``SideBySide`` of ``MaskedAttention`` (``left``: convolutions, neighbouring rotary pairs with
                    the Llama 3.1 wavelength rule, a window of ``mask.size`` that keeps the first
                    ``mask.keep_first`` tokens, sigmoid gate) and ``GatedLinearAttention`` (``right``)
* feed-forward   -> ``SoftmaxMoE``
"""
from __future__ import annotations

import json
import os
from typing import Dict, Optional

import torch

from .hybrid import (ExpertSpec, GatedLinearAttention, GatedLinearAttentionSpec, HybridCausalLM, HybridSpec, LayerSpec,
                     MaskedAttention, MaskedAttentionSpec, MaskSpec, MinGRU, MinGRUSpec, MoESpec, RotarySpec,
                     SideBySide, SideBySideSpec, SoftmaxMoE, TokenSide, TwoNormParallelLayer)

ARCHITECTURE = "Zoguzen"


def _heads(m: dict, i: int):
    H, G = int(m["heads"]), int(m.get("kv_heads", m["heads"]))
    if H < 1 or G < 1 or H % G:
        raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
    return H, G


def _chunk_attention(m: dict, i: int, raw) -> MaskedAttentionSpec:
    H, G = _heads(m, i)
    src = m.get("kv_from")
    s = MaskedAttentionSpec(heads=H, kv_heads=G, dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                            rot=None, mask=MaskSpec("chunk", int(m["mask"]["size"])), qk_norm="head", bias=True,
                            sink=False, kv_from=None if src is None else int(src), taps=int(m.get("conv") or 0),
                            softcap=float(m.get("softcap") or 0.0), sink_score=0.0, talk=True)
    if s.mask.size < 1:
        raise ValueError(f"layer {i}: mask.size must be at least 1")
    if s.kv_from is not None:
        j = s.kv_from
        if not 0 <= j < i or raw[j]["type"] != "attention" or raw[j]["mixer"].get("kv_from") is not None:
            raise ValueError(f"layer {i}: kv_from must name an earlier attention layer with keys of its own")
        o = raw[j]["mixer"]
        if (int(o.get("kv_heads", o["heads"])), int(o["dim"]), int(o["vdim"])) != (s.kv_heads, s.dim, s.vdim):
            raise ValueError(f"layer {i}: layer {j}'s key / value sizes differ")
    return s


def _window_attention(m: dict, i: int) -> MaskedAttentionSpec:
    H, G = _heads(m, i)
    rot = m.get("rot")
    rs = None
    if rot and int(rot.get("dims", 0)):
        rs = RotarySpec(int(rot["dims"]), float(rot["base"]), rot.get("scaling") or None, "pairs")
        if rs.dims > int(m["dim"]) or rs.dims % 2:
            raise ValueError(f"layer {i}: rot.dims must be even and at most dim")
    mask = MaskSpec("window", int(m["mask"]["size"]), int(m["mask"].get("keep_first") or 0))
    if mask.size < 1 or mask.keep_first < 0:
        raise ValueError(f"layer {i}: mask.size must be at least 1")
    return MaskedAttentionSpec(heads=H, kv_heads=G, dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
                               rot=rs, mask=mask, qk_norm="none", bias=False, sink=False, taps=int(m.get("conv") or 0),
                               out_gate=True)


def spec_from_config(cfg: dict, decay_rank: Optional[Dict[int, int]] = None) -> HybridSpec:
    """``decay_rank``: layer -> rank of its decay projection (a checkpoint's tensor gives it; otherwise the
    mixer's ``rank`` entry)"""
    layers = []
    raw = cfg["layers"]
    for i, L in enumerate(raw):
        m, kind = L["mixer"], L["type"]
        if kind == "mingru":
            mixer, name = MinGRUSpec(int(m["width"])), "mingru"
        elif kind == "attention":
            mixer, name = _chunk_attention(m, i, raw), "masked_attention"
        elif kind == "parallel":
            r = m["right"]
            rank = (decay_rank or {}).get(i) or r.get("rank")
            if not rank:
                raise ValueError(f"layer {i}: the rank of the decay projection is not known")
            right = GatedLinearAttentionSpec(heads=int(r["heads"]), dim=int(r["dim"]), vdim=int(r["vdim"]),
                                             tau=float(r["tau"]), rank=int(rank))
            mixer, name = SideBySideSpec(_window_attention(m["left"], i), right), "side_by_side"
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = L.get("mlp")
        if mlp is not None:
            if mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
            r = mlp["router"]
            mlp = MoESpec(experts=int(r["experts"]), top=int(r["top"]), expert=ExpertSpec(ff=int(mlp["expert"]["ff"])))
            if not 1 <= mlp.top <= mlp.experts:
                raise ValueError(f"layer {i}: router.top must be 1..experts")
        layers.append(LayerSpec(name, mixer, mlp))
    return HybridSpec(model_type="zoguzen", vocab_size=int(cfg["vocab"]), hidden_size=int(cfg["width"]), layers=layers,
                      norm_eps=float(cfg["norm"]["eps"]), block="parallel2", norm="layer_norm",
                      final_softcap=float(cfg.get("logit_softcap") or 0.0), tied_head=True,
                      side_dim=int((cfg.get("token_side") or {}).get("dim", 0)))


def _attention_shapes(out: dict, p: str, m: MaskedAttentionSpec, W: int):
    own = m.kv_from is None
    out.update({p + "q": (m.heads * m.dim, W), p + "o": (W, m.heads * m.vdim)})
    if own:
        out.update({p + "k": (m.kv_heads * m.dim, W), p + "v": (m.kv_heads * m.vdim, W)})
    if m.bias:
        out[p + "q.b"] = (m.heads * m.dim,)
        if own:
            out.update({p + "k.b": (m.kv_heads * m.dim,), p + "v.b": (m.kv_heads * m.vdim,)})
    if m.taps >= 1:
        out[p + "q.conv"] = (m.heads * m.dim, m.taps)
        if own:
            out.update({p + "k.conv": (m.kv_heads * m.dim, m.taps), p + "v.conv": (m.kv_heads * m.vdim, m.taps)})
    if m.qk_norm == "head":
        out[p + "q.norm"] = (m.dim,)
        if own:
            out[p + "k.norm"] = (m.dim,)
    if m.talk:
        out[p + "talk"] = (m.heads, m.heads)
    if m.out_gate:
        out[p + "g"] = (m.heads * m.vdim, W)


def tensor_shapes(spec: HybridSpec) -> Dict[str, tuple]:
    """name -> shape of every tensor of a checkpoint of ``spec``"""
    W = spec.hidden_size
    out = {"embed": (spec.vocab_size, W)}
    if spec.side_dim:
        out["side.embed"] = (spec.vocab_size, spec.side_dim * spec.num_layers)
    for i, L in enumerate(spec.layers):
        p, m = f"l{i}.", L.mixer
        out.update({p + "norm1": (W,), p + "shift": (W,)})
        if L.kind == "mingru":
            n = m.width
            out.update({p + "mix.z": (n, W), p + "mix.z.b": (n,), p + "mix.x": (n, W), p + "mix.x.b": (n,),
                        p + "mix.g": (n, W), p + "mix.o": (W, n)})
        elif L.kind == "masked_attention":
            _attention_shapes(out, p + "mix.", m, W)
        else:
            _attention_shapes(out, p + "mix.left.", m.left, W)
            r, q = m.right, p + "mix.right."
            out.update({q + "q": (r.heads * r.dim, W), q + "k": (r.heads * r.dim, W), q + "v": (r.heads * r.vdim, W),
                        q + "g": (r.heads * r.vdim, W), q + "o": (W, r.heads * r.vdim), q + "norm": (r.vdim,),
                        q + "a1": (r.rank, W), q + "a2": (r.heads * r.dim, r.rank), q + "a2.b": (r.heads * r.dim,),
                        p + "mix.left.out": (W,), p + "mix.right.out": (W,)})
        if L.mlp is not None:
            out[p + "norm2"] = (W,)
            for e in range(L.mlp.experts):
                q = f"{p}mlp.e{e}."
                out.update({q + "gate": (L.mlp.expert.ff, W), q + "up": (L.mlp.expert.ff, W),
                            q + "down": (W, L.mlp.expert.ff)})
            out[p + "mlp.router"] = (L.mlp.experts, W)
        if spec.side_dim:
            out.update({p + "side.gate": (spec.side_dim, W), p + "side.proj": (W, spec.side_dim), p + "side.norm": (W,)})
    out["final.norm"] = (W,)
    return out


def _attention(m: MaskedAttentionSpec, t, p: str) -> MaskedAttention:
    own = m.kv_from is None

    def opt(name, cond=True):
        return t(p + name) if cond else None

    conv = None
    if m.taps >= 1:
        conv = (t(p + "q.conv"), opt("k.conv", own), opt("v.conv", own))
    return MaskedAttention(m, t(p + "q"), opt("k", own), opt("v", own), opt("q.b", m.bias), opt("k.b", m.bias and own),
                           opt("v.b", m.bias and own), opt("q.norm", m.qk_norm == "head"),
                           opt("k.norm", m.qk_norm == "head" and own), None, t(p + "o"), conv=conv,
                           talk=opt("talk", m.talk), w_g=opt("g", m.out_gate))


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
        if L.kind == "mingru":
            mixer = MinGRU(L.mixer, t(p + "z"), t(p + "x"), t(p + "g"), t(p + "z.b"), t(p + "x.b"), t(p + "o"))
        elif L.kind == "masked_attention":
            mixer = _attention(L.mixer, t, p)
        else:
            q = p + "right."
            right = GatedLinearAttention(L.mixer.right, t(q + "q"), t(q + "k"), t(q + "v"), t(q + "g"), t(q + "a1"),
                                         t(q + "a2"), t(q + "a2.b"), t(q + "norm"), t(q + "o"))
            mixer = SideBySide(_attention(L.mixer.left, t, p + "left."), right, t(p + "left.out"), t(p + "right.out"))
        mlp, n2 = None, None
        if L.mlp is not None:
            q = f"l{i}.mlp."
            E = L.mlp.experts
            w_gu = torch.stack([torch.cat([t(f"{q}e{e}.gate"), t(f"{q}e{e}.up")], 0) for e in range(E)])
            w_down = torch.stack([t(f"{q}e{e}.down") for e in range(E)])
            mlp, n2 = SoftmaxMoE(L.mlp, t(q + "router"), w_gu, w_down), t(f"l{i}.norm2")
        side = None
        if spec.side_dim:
            r = f"l{i}.side."
            side = TokenSide(t(r + "gate"), t(r + "proj"), t(r + "norm"), i * spec.side_dim)
        layers.append(TwoNormParallelLayer(mixer, t(f"l{i}.norm1"), mlp, n2, shift=t(f"l{i}.shift"), side=side))
    return HybridCausalLM(spec, t("embed"), None, layers, t("final.norm"), None, dtype,
                          side_embed=t("side.embed") if spec.side_dim else None).eval()


def load(path: str, dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    """Read ``config.json`` + ``model.safetensors`` of a checkpoint folder."""
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    tensors = {}
    with safe_open(os.path.join(path, "model.safetensors"), "pt") as f:
        names = set(f.keys())
        rank = {i: int(f.get_slice(f"l{i}.mix.right.a1").get_shape()[0]) for i in range(len(cfg["layers"]))
                if f"l{i}.mix.right.a1" in names}
        spec = spec_from_config(cfg, rank)
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
        if name.endswith(("norm1", "norm2", "final.norm", ".norm", ".out")):
            w = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name.endswith("shift"):
            w = torch.rand(shape, generator=g)
        elif name.endswith("talk"):
            w = torch.eye(shape[0]) + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith(".conv"):
            w = 0.5 * torch.randn(shape, generator=g)
        elif name.endswith("a2.b"):
            w = 2.0 + torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            w = 0.3 * torch.randn(shape, generator=g)
        elif len(shape) == 2 and name not in ("embed", "side.embed"):
            w = torch.randn(shape, generator=g) * (std if std is not None else shape[1] ** -0.5)
        else:
            w = torch.randn(shape, generator=g) * (std if std is not None else 1.0)
        out[name] = w.to(torch.bfloat16)
    return out


def random_model(spec: HybridSpec, seed: int = 0, dtype=torch.bfloat16, device="cuda") -> HybridCausalLM:
    return build(spec, random_tensors(spec, seed), dtype, device)
