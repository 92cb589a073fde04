"""Hybrid decoders: a layer list that mixes attention over a paged cache with
recurrent layers over per-sequence state, driven by data (``HybridSpec``).

Building blocks (each usable by any design that lists it in its layer specs):

* ``LatentAttention``   low-rank latent attention: one cached row per token,
  ``[latent c (kv_rank) | shared rotated key (rot_dim)]``; per-head keys and
  values are ``W_uk c`` / ``W_uv c``, so scores and outputs are formed in the
  latent space with the up-projections absorbed (as models/mla.py does for
  the DeepSeek family):  q_lat[h] = W_uk[h]^T q_nope[h],
  s = (q_lat[h] . c + q_rot[h] . k_rot) scale,  o[h] = W_uv[h] (softmax(s) C).
  Interleaved-pair rotary positions with optional YaRN scaling, an optional
  per-head sigmoid output gate.
* ``MLSTM``             matrix-memory recurrence (xLSTM's mLSTM) with capped
  exponential gates, running-maximum stabiliser, per-head RMS norm and a
  sigmoid output gate; f32 state in the cache's slots.
* ``DenseFF``           gated feed-forward, tanh-GELU.
* ``GroupedAttention``  grouped-query attention over a paged cache of
  ``[keys | values]`` rows: per-head RMS norm of queries and keys, half-split
  rotary positions (optionally on part of the head, optional YaRN), the
  values are the key projection itself (before norm and rotation), the
  heads' scores are mixed by an [H, H] matrix before the softmax, an
  element-wise sigmoid output gate.
* ``ReluSqFF``          two-matrix feed-forward with a squared-ReLU activation.
* ``SigmoidMoE``        experts behind a sigmoid router: the chosen experts'
  scores weigh the experts' *inputs*; clamped GLU experts
  ``W_down (g sigmoid(alpha g) (u + 1))``; an optional shared expert.
* ``TokenSide``         a per-layer token input: a slice of a second
  embedding table, gated by the residual stream, projected, RMS-normed and
  added.
* ``SSMMixer``          state-space mixer (Mamba-2 form): one input
  projection ``[z | x | B | C | dt]``, a short causal convolution with SiLU
  over ``[x | B | C]`` (its last inputs are state), the selective scan
  S' = exp(-exp(A) dt) S + dt B x^T, y = S'^T C + D x over f32 state slots,
  then y silu(z), a group RMS norm and the output projection.
* ``MaskedAttention``   grouped-query attention over paged ``[keys | values]``
  rows with separate value size, optional projection biases, RMS norm of
  queries and keys per head or over the whole projection, rotary positions in
  either pair layout, a causal / sliding-window / chunked view of the past,
  an optional per-head sink in the softmax, and optionally the keys and
  values of an earlier layer (``kv_from``) instead of its own.
* ``LatentAttention`` also takes a sliding window, the half-split rotary layout
  (folded into the weights' row order) and an element-wise output gate.
* ``MaskedAttention`` also takes short causal convolutions on q / k / v right
  after the projection (their last inputs are state), a tanh cap on the
  scores, a sink of a fixed score, a window that keeps the sequence's first
  tokens visible, an [H, H] mixing of the heads' weights *after* the softmax,
  a sigmoid output gate, and the wavelength rule of Llama 3.1 for its rotary
  frequencies.
* ``MinGRU``            minGRU: gates that read only the current token,
  S' = (1 - z) S + z c element by element over f32 state, SiLU output gate.
* ``GatedLinearAttention``  per head S' = diag(alpha) S + k v^T, o = S'^T q with
  a decay per key channel alpha = sigmoid(low-rank(h))^(1 / tau), per-head RMS
  norm and a SiLU output gate; f32 state.
* ``SideBySide``        two mixers on the same input (one fused projection),
  each result RMS-normed over the width, then their mean.
* ``SoftmaxMoE``        experts whose weights are the softmax over the chosen
  router logits and multiply the experts' *outputs*; SiLU-gated experts.

Block layouts.  ``pre_norm`` (``PreNormLayer``): x += mixer(norm1(x)),
x += ff(norm2(x)) with vector RMS norms; each sublayer's result is added by
the launch that also forms the next norm.  ``post_norm`` (``HybridLayer``): the sublayers read the
residual stream ``x`` itself and their *output* is normalised:
x += mult * LN(mixer(x)), x += mult * LN(ff(x)).  ``parallel``
(``ParallelLayer``): one norm, both sublayers read it, their scaled results
are summed and added: h = norm(x), x += ls1 * mixer(h + conv(h)) + ls2 * ff(h),
with an optional short causal convolution in front of the mixer (its last
inputs are per-sequence state) and an optional token-side input afterwards.
``parallel2`` (``TwoNormParallelLayer``): two LayerNorms of the same x, the
mixer's input shifted towards the previous token's:
h = LN1(x), x += mixer(h + (h_prev - h) * mu) + ff(LN2(x)), then the token-side
input.
The residual stream is f32 throughout; projections run in the model's
activation dtype through the vendor GEMM, everything else in the kernels of
``ops/seqmix.py`` and ``ops/blockmix.py``.

``forward_tokens`` takes a *ragged* step (``AttnMeta.cu_q`` ...): sequences
bring different numbers of new tokens, prompt portions beside single decoded
tokens, and is what ``serving.engine.LLMEngine`` drives for these models.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops import blockmix as BM
from ..ops import gatedmix as GM
from ..ops import maskattn as MA
from ..ops import seqmix as SM
from ..ops import ssm as SSM
from .decoder import AttnMeta


# ---------------------------------------------------------------------- specs
@dataclass
class RotarySpec:
    dims: int
    base: float = 10000.0
    scaling: Optional[dict] = None          # YaRN: factor, original, fast, slow | Llama 3.1: factor, low, high, original
    layout: Optional[str] = None            # "pairs" (2i, 2i+1) | "half" (i, i + dims/2); None: the mixer's own


@dataclass
class MaskSpec:
    kind: str = "causal"                    # "causal" | "window" (itself and size - 1 before) | "chunk" (aligned blocks)
    size: int = 0
    keep_first: int = 0                     # window: the sequence's first keep_first tokens stay visible as well


@dataclass
class LatentAttentionSpec:
    heads: int
    dim: int                                # unrotated query / key size per head
    rot_dim: int                            # rotated part (one key shared by all heads)
    vdim: int
    kv_rank: int
    scale: float
    rot: RotarySpec = None
    out_gate: bool = True
    gate: str = "head"                      # "head": one gate per head | "element": one per value of the joined heads
    window: int = 0                         # > 0: a token sees itself and the window - 1 tokens before it


@dataclass
class SSMSpec:
    heads: int
    vdim: int                               # values per head (inner = heads * vdim)
    state: int                              # N
    groups: int                             # B / C groups; head h reads group h // (heads / groups)
    taps: int                               # of the convolution over [x | B | C]
    norm_groups: int = 1


@dataclass
class MaskedAttentionSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[RotarySpec] = None        # on the first rot.dims values of every head
    mask: MaskSpec = None
    qk_norm: str = "whole"                  # "none" | "head" (weights [dim]) | "whole" (weights [heads dim])
    bias: bool = True                       # q / k / v projections carry biases
    sink: bool = True                       # a learned number per head in the softmax's denominator
    kv_from: Optional[int] = None           # read this layer's cache rows instead of projecting keys and values
    taps: int = 0                           # >= 1: causal per-channel convolutions on q / k / v right after the projection
    softcap: float = 0.0                    # > 0: score <- softcap tanh(score / softcap)
    sink_score: Optional[float] = None      # a sink of this fixed score (no tensor) instead of a learned one
    talk: bool = False                      # [H, H] mixing of the heads' weights after the softmax
    out_gate: bool = False                  # element-wise sigmoid gate on the joined heads


@dataclass
class MinGRUSpec:
    width: int


@dataclass
class GatedLinearAttentionSpec:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int                               # of the low-rank decay projection


@dataclass
class SideBySideSpec:
    left: object                            # (kind, spec) pairs of MIXERS
    right: object
    left_kind: str = "masked_attention"
    right_kind: str = "gated_linear_attention"


@dataclass
class MLSTMSpec:
    heads: int
    dim: int
    vdim: int
    gate_cap: float = 15.0


@dataclass
class DenseFFSpec:
    ff: int
    act: str = "gelu_tanh"                  # "gelu_tanh" | "relu" | "silu" on the gate rows


@dataclass
class GroupedAttentionSpec:
    heads: int
    kv_heads: int
    dim: int                                # query / key size per head; the values are the keys as projected
    scale: float
    rot: RotarySpec = None                  # half-split pairs on the first rot.dims values of a head
    qk_norm: bool = True
    talk: bool = True                       # [H, H] mixing of the heads' scores before the softmax
    out_gate: bool = True                   # element-wise sigmoid gate on the concatenated heads


@dataclass
class ReluSqFFSpec:
    ff: int


@dataclass
class ExpertSpec:
    ff: int
    limit: float = float("inf")
    alpha: float = 1.702


@dataclass
class MoESpec:
    experts: int
    top: int
    expert: ExpertSpec = None
    shared: Optional[ExpertSpec] = None


@dataclass
class LayerSpec:
    kind: str                               # key of MIXERS
    mixer: object
    mlp: Optional[object] = None            # DenseFFSpec | ReluSqFFSpec | MoESpec


@dataclass
class BigramSpec:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class HybridSpec:
    model_type: str
    vocab_size: int
    hidden_size: int
    layers: List[LayerSpec]
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    bigram: Optional[BigramSpec] = None
    final_softcap: float = 0.0              # read by the engines' shared helpers
    logit_scale: float = 1.0                # the logits are multiplied by it
    block: str = "post_norm"                # "post_norm" | "parallel" | "parallel2" | "pre_norm"
    norm: str = "layer_norm"                # "layer_norm" | "rms_scalar" (one number) | "rms" (a vector)
    layer_scale: bool = False               # parallel blocks: per-coordinate scales on both sublayers' results
    canon_taps: int = 0                     # parallel blocks: taps of the convolution in front of the mixer (0: none)
    side_dim: int = 0                       # per-layer slice of the token-side table (0: none)
    tied_head: bool = False                 # the logits are products with the embedding table

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def _spec_list(c) -> list:
    """a mixer's cache request (one entry, a list of entries or None) as a list"""
    return list(c) if isinstance(c, list) else [c]


# ---------------------------------------------------------------------- mixers
class LatentAttention(nn.Module):
    cache_kind = "rows"

    def __init__(self, s: LatentAttentionSpec, w_q, w_dkv, dkv_norm, w_uk, w_uv, w_g, w_o):
        super().__init__()
        self.s = s
        H, r = s.heads, s.kv_rank
        if s.rot is not None and s.rot.layout == "half":
            # half-split pairs (i, i + dims / 2) -> the kernels' neighbouring pairs (2 i, 2 i + 1): the same
            # reordering of the rotated rows of W_q (every head) and of W_dkv leaves every score unchanged
            n = s.rot.dims
            perm = torch.arange(s.rot_dim)
            perm[:n] = torch.stack([torch.arange(n // 2), torch.arange(n // 2) + n // 2], 1).reshape(-1)
            w_q = w_q.view(H, s.dim + s.rot_dim, -1)
            w_q = torch.cat([w_q[:, :s.dim], w_q[:, s.dim:][:, perm.to(w_q.device)]], 1).reshape(H * (s.dim + s.rot_dim), -1)
            w_dkv = torch.cat([w_dkv[:r], w_dkv[r:][perm.to(w_dkv.device)]], 0)
        if s.out_gate and s.gate not in ("head", "element"):
            raise ValueError(f"unknown gate kind {s.gate!r}")
        # one projection launch: [q | dkv | gate] rows
        parts = [w_q, w_dkv] + ([w_g] if w_g is not None else [])
        self.w_in = nn.Parameter(torch.cat(parts, 0).contiguous(), requires_grad=False)
        self.n_q, self.n_dkv = w_q.shape[0], w_dkv.shape[0]
        self.dkv_norm = nn.Parameter(dkv_norm, requires_grad=False)
        self.w_uk = nn.Parameter(w_uk.view(H, s.dim, r).contiguous(), requires_grad=False)               # [H, dim, r]
        self.w_uv_t = nn.Parameter(w_uv.view(H, s.vdim, r).transpose(1, 2).contiguous(), requires_grad=False)  # [H, r, dv]
        self.w_o = nn.Parameter(w_o, requires_grad=False)
        self.table: Optional[torch.Tensor] = None

    def cache_spec(self):
        return ("rows", self.s.kv_rank + self.s.rot_dim)

    def ensure_table(self, max_pos: int):
        if self.table is None or self.table.shape[0] < max_pos or self.table.device != self.w_o.device:
            n = max(256, 1 << (max_pos - 1).bit_length())
            self.table = SM.rope_table(n, self.s.rot.dims, self.s.rot.base, self.s.rot.scaling).to(self.w_o.device)
        return self.table

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H = xa.shape[0], s.heads
        y = F.linear(xa, self.w_in)
        q = y[:, :self.n_q].reshape(T, H, s.dim + s.rot_dim).contiguous()
        dkv = y[:, self.n_q:self.n_q + self.n_dkv]
        gate = y[:, self.n_q + self.n_dkv:] if s.out_gate else None
        head_gate = gate if s.gate == "head" else None
        table = self.table
        SM.latent_kv_store(dkv, self.dkv_norm, eps, s.kv_rank, table, pos, slots, cache.rows[li])
        SM.rope_rows_(q, s.dim, table, pos)
        # absorbed up-projection of the keys: per-head [T, dim] x [dim, r]
        q_lat = torch.bmm(q[..., :s.dim].transpose(0, 1), self.w_uk).transpose(0, 1)
        o_lat = SM.latent_attention(q_lat, q[..., s.dim:], cache.rows[li], meta.block_tables, meta.seq_of, pos,
                                    s.scale, head_gate, meta.q_lens_host, meta.seq_lens_host, xa.dtype,
                                    window=s.window)
        o = torch.bmm(o_lat.transpose(0, 1), self.w_uv_t).transpose(0, 1).reshape(T, H * s.vdim)
        if gate is not None and s.gate == "element":
            o = MA.sigmoid_gate(o, gate)
        return BM.linear(o, self.w_o)


class MLSTM(nn.Module):
    cache_kind = "state"

    def __init__(self, s: MLSTMSpec, w_q, w_k, w_v, w_g, w_i, w_f, b_i, b_f, norm, w_o):
        super().__init__()
        self.s = s
        self.w_in = nn.Parameter(torch.cat([w_q, w_k, w_v, w_g, w_i, w_f], 0).contiguous(), requires_grad=False)
        self.b_i = nn.Parameter(b_i.float(), requires_grad=False)
        self.b_f = nn.Parameter(b_f.float(), requires_grad=False)
        self.norm = nn.Parameter(norm, requires_grad=False)
        self.w_o = nn.Parameter(w_o, requires_grad=False)

    def cache_spec(self):
        s = self.s
        return ("state", {"S": (s.heads, s.dim, s.vdim), "n": (s.heads, s.dim), "m": (s.heads,)})

    def ensure_table(self, max_pos: int):
        return None

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H = xa.shape[0], s.heads
        nqk, nv = H * s.dim, H * s.vdim
        y = F.linear(xa, self.w_in)
        q, k = y[:, :nqk].reshape(T, H, s.dim), y[:, nqk:2 * nqk].reshape(T, H, s.dim)
        v = y[:, 2 * nqk:2 * nqk + nv].reshape(T, H, s.vdim)
        g = y[:, 2 * nqk + nv:2 * nqk + 2 * nv]
        ip, fp = y[:, 2 * nqk + 2 * nv:2 * nqk + 2 * nv + H], y[:, 2 * nqk + 2 * nv + H:]
        h = SM.mlstm_scan(q, k, v, ip, fp, self.b_i, self.b_f, s.gate_cap, cache.state[li], meta.cu_q,
                          meta.state_slots, pos, meta.q_lens_host)
        o = SM.head_rms_gate(h, self.norm, g, eps, xa.dtype)
        return F.linear(o, self.w_o)


class DenseFF(nn.Module):
    """``W_down (act(W_gate h) * (W_up h))``"""

    def __init__(self, w_gate, w_up, w_down, act: str = "gelu_tanh"):
        super().__init__()
        if act not in SM.GLU_ACTS:
            raise ValueError(f"unknown feed-forward activation {act!r}")
        self.act = act
        self.w_gu = nn.Parameter(torch.cat([w_gate, w_up], 0).contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(w_down, requires_grad=False)

    def forward(self, xa):
        if self.act == "gelu_tanh":
            return F.linear(SM.glu_gelu(F.linear(xa, self.w_gu)), self.w_down)
        return BM.linear(SM.glu_act(BM.linear(xa, self.w_gu), self.act), self.w_down)


class SSMMixer(nn.Module):
    """``w_in`` rows ``[z (inner) | x (inner) | B (G N) | C (G N) | dt (heads)]``; ``conv_w`` [inner + 2 G N, taps]
    (last column: the current token) with bias ``conv_b``; ``dt_bias`` / ``a_log`` / ``d_skip`` [heads]; ``norm``
    [inner]."""
    cache_kind = "state"

    def __init__(self, s: SSMSpec, w_in, conv_w, conv_b, dt_bias, a_log, d_skip, norm, w_o):
        super().__init__()
        if s.heads % s.groups:
            raise ValueError("heads must be a multiple of groups")
        if (s.heads * s.vdim) % s.norm_groups:
            raise ValueError("heads * vdim must split into norm_groups equal parts")
        if s.taps < 1 or s.taps > 16:
            raise ValueError("1 <= conv taps <= 16")
        if s.state > SSM.SCAN_MAX_STATE:
            raise ValueError(f"state size above {SSM.SCAN_MAX_STATE}")
        self.s = s
        self.inner, self.chan = s.heads * s.vdim, s.heads * s.vdim + 2 * s.groups * s.state
        self.w_in = nn.Parameter(w_in, requires_grad=False)
        self.conv_w = nn.Parameter(conv_w.float().contiguous(), requires_grad=False)
        self.conv_b = nn.Parameter(conv_b.float().contiguous(), requires_grad=False)
        self.dt_bias = nn.Parameter(dt_bias.float().contiguous(), requires_grad=False)
        self.a_log = nn.Parameter(a_log.float().contiguous(), requires_grad=False)
        self.d_skip = nn.Parameter(d_skip.float().contiguous(), requires_grad=False)
        self.norm = nn.Parameter(norm, requires_grad=False)
        self.w_o = nn.Parameter(w_o, requires_grad=False)

    def cache_spec(self):
        s = self.s
        return ("state", {"S": (s.heads, s.state, s.vdim), "conv": (s.taps - 1, self.chan)})

    def ensure_table(self, max_pos: int):
        return None

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H, inner, GN = xa.shape[0], s.heads, self.inner, s.groups * s.state
        y = BM.linear(xa, self.w_in)
        z, u, dt = y[:, :inner], y[:, inner:inner + self.chan], y[:, inner + self.chan:]
        st = cache.state[li]
        xbc = SSM.conv_silu(u, self.conv_w, self.conv_b, st["conv"], meta.cu_q, meta.seq_of, meta.state_slots, pos,
                            meta.q_lens_host)
        yy = SSM.selective_scan(xbc[:, :inner].view(T, H, s.vdim), xbc[:, inner:inner + GN].view(T, s.groups, s.state),
                                xbc[:, inner + GN:].view(T, s.groups, s.state), dt, self.dt_bias, self.a_log,
                                self.d_skip, st["S"], meta.cu_q, meta.state_slots, pos, meta.q_lens_host)
        o = SSM.gated_group_norm(yy.view(T, inner), z, self.norm, s.norm_groups, eps, xa.dtype)
        return BM.linear(o, self.w_o)


class MaskedAttention(nn.Module):
    """``w_q`` [H d, W], ``w_k`` [G d, W], ``w_v`` [G dv, W] (``w_k`` / ``w_v`` None with ``kv_from``), biases or
    None, norm weights per ``qk_norm``, ``sink`` [H] or None, ``w_o`` [W, H dv]; optional ``conv`` = (q, k, v)
    weights [channels, taps] (k / v None with ``kv_from``), ``talk`` [H, H], ``w_g`` [H dv, W]."""
    cache_kind = "rows"

    def __init__(self, s: MaskedAttentionSpec, w_q, w_k, w_v, b_q, b_k, b_v, q_norm, k_norm, sink, w_o, conv=None,
                 talk=None, w_g=None):
        super().__init__()
        if s.heads % s.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if s.mask is None or s.mask.kind not in MA.MASKS or (s.mask.kind != "causal" and s.mask.size < 1):
            raise ValueError("mask: causal, or window / chunk with a size of at least 1")
        if s.mask.keep_first and s.mask.kind != "window":
            raise ValueError("keep_first belongs to a window")
        if s.qk_norm not in ("none", "head", "whole"):
            raise ValueError(f"unknown qk_norm {s.qk_norm!r}")
        self.s = s
        shared = s.kv_from is not None
        parts = [w_q] if shared else [w_q, w_k, w_v]
        self.n_qkv = sum(int(w.shape[0]) for w in parts)
        if s.out_gate:
            parts = parts + [w_g]
        self.w_in = nn.Parameter(torch.cat(parts, 0).contiguous(), requires_grad=False)
        self.b_in = None
        if s.bias:
            bs = [b_q] if shared else [b_q, b_k, b_v]
            if s.out_gate:
                bs = bs + [torch.zeros(w_g.shape[0], dtype=b_q.dtype, device=b_q.device)]
            self.b_in = nn.Parameter(torch.cat(bs, 0).contiguous(), requires_grad=False)
        self.conv = None
        if s.taps >= 1:
            cw = [conv[0]] if shared else list(conv)
            self.conv = nn.Parameter(torch.cat(cw, 0).float().contiguous(), requires_grad=False)      # [q | k | v] channels
        self.q_norm = nn.Parameter(q_norm, requires_grad=False) if q_norm is not None else None
        self.k_norm = nn.Parameter(k_norm, requires_grad=False) if k_norm is not None else None
        if s.sink_score is not None:
            sink = torch.full((s.heads,), float(s.sink_score), device=w_o.device)
        self.sink = nn.Parameter(sink.float().contiguous(), requires_grad=False) if sink is not None else None
        self.talk = nn.Parameter(talk.float().contiguous(), requires_grad=False) if s.talk else None
        self.w_o = nn.Parameter(w_o, requires_grad=False)
        self.table: Optional[torch.Tensor] = None

    def cache_spec(self):
        s = self.s
        out = [] if s.kv_from is not None else [("rows", s.kv_heads * (s.dim + s.vdim))]
        if self.conv is not None:
            out.append(("state", {"conv": (s.taps - 1, self.n_qkv)}))
        return out[0] if len(out) == 1 else (out or None)

    def ensure_table(self, max_pos: int):
        if self.s.rot is None or self.s.rot.dims == 0:
            return None
        if self.table is None or self.table.shape[0] < max_pos or self.table.device != self.w_o.device:
            n = max(256, 1 << (max_pos - 1).bit_length())
            self.table = SM.rope_table(n, self.s.rot.dims, self.s.rot.base, self.s.rot.scaling).to(self.w_o.device)
        return self.table

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        return self.mix(BM.linear(xa, self.w_in, self.b_in), pos, slots, meta, cache, li, eps)

    def mix(self, y, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        """``y``: this mixer's columns of the input projection, ``[q | k | v | gate]``"""
        s = self.s
        T, H, G, d, dv = y.shape[0], s.heads, s.kv_heads, s.dim, s.vdim
        act = y.dtype
        gate = y[:, self.n_qkv:] if s.out_gate else None
        if self.conv is not None:               # f32 result: the norm and the rotation read it unrounded
            y = GM.causal_conv(y[:, :self.n_qkv], self.conv, cache.state[li]["conv"], meta.cu_q, meta.seq_of,
                               meta.state_slots, pos, meta.q_lens_host)
        q = y[:, :H * d].view(T, H, d)
        layout = (s.rot.layout if s.rot is not None else None) or "half"
        table = self.table if s.rot is not None and s.rot.dims else None
        if s.kv_from is None:
            k = y[:, H * d:(H + G) * d].view(T, G, d)
            v = y[:, (H + G) * d:(H + G) * d + G * dv].view(T, G, dv)
            rows = cache.rows[li]
            qf = MA.qkv_norm_rope_store(q, k, v, self.q_norm, self.k_norm, s.qk_norm == "whole", eps, table,
                                        layout, pos, slots, rows)
        else:
            rows = cache.rows[s.kv_from]
            qf = MA.qkv_norm_rope_store(q, None, None, self.q_norm, None, s.qk_norm == "whole", eps, table,
                                        layout, pos, slots, None)
        o = MA.masked_attention(qf, rows, G, dv, meta.block_tables, meta.seq_of, pos, s.scale, s.mask.kind, s.mask.size,
                                self.sink, meta.q_lens_host, meta.seq_lens_host, act, softcap=s.softcap,
                                keep_first=s.mask.keep_first, talk=self.talk)
        if gate is not None:
            o = MA.sigmoid_gate(o, gate)
        return BM.linear(o, self.w_o)


class MinGRU(nn.Module):
    """``w_z`` / ``w_x`` / ``w_g`` [width, W], ``b_z`` / ``b_x`` [width], ``w_o`` [W, width]: z = sigmoid(W_z h + b_z),
    u = W_x h + b_x, candidate u + 1/2 (u >= 0) or sigmoid(u) (u < 0), S' = (1 - z) S + z c, W_o (S' silu(W_g h))."""
    cache_kind = "state"

    def __init__(self, s: MinGRUSpec, w_z, w_x, w_g, b_z, b_x, w_o):
        super().__init__()
        self.s = s
        self.w_in = nn.Parameter(torch.cat([w_z, w_x, w_g], 0).contiguous(), requires_grad=False)
        self.b_in = nn.Parameter(torch.cat([b_z, b_x, torch.zeros_like(b_x)], 0).contiguous(), requires_grad=False)
        self.w_o = nn.Parameter(w_o, requires_grad=False)

    def cache_spec(self):
        return ("state", {"gru": (self.s.width,)})

    def ensure_table(self, max_pos: int):
        return None

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        return self.mix(BM.linear(xa, self.w_in, self.b_in), pos, slots, meta, cache, li, eps)

    def mix(self, y, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        o = GM.mingru_scan(y, self.s.width, cache.state[li]["gru"], meta.cu_q, meta.state_slots, pos, meta.q_lens_host)
        return BM.linear(o, self.w_o)


class GatedLinearAttention(nn.Module):
    """``w_q`` / ``w_k`` [H d, W], ``w_v`` / ``w_g`` [H dv, W], ``w_a1`` [rank, W], ``w_a2`` [H d, rank] with bias
    ``b_a2``, ``norm`` [dv], ``w_o`` [W, H dv]."""
    cache_kind = "state"

    def __init__(self, s: GatedLinearAttentionSpec, w_q, w_k, w_v, w_g, w_a1, w_a2, b_a2, norm, w_o):
        super().__init__()
        if s.tau <= 0:
            raise ValueError("tau must be positive")
        self.s = s
        self.w_in = nn.Parameter(torch.cat([w_q, w_k, w_v, w_g, w_a1], 0).contiguous(), requires_grad=False)
        self.b_in = None
        self.w_a2 = nn.Parameter(w_a2, requires_grad=False)
        self.b_a2 = nn.Parameter(b_a2, requires_grad=False)
        self.norm = nn.Parameter(norm, requires_grad=False)
        self.w_o = nn.Parameter(w_o, requires_grad=False)

    def cache_spec(self):
        s = self.s
        return ("state", {"gla": (s.heads, s.dim, s.vdim)})

    def ensure_table(self, max_pos: int):
        return None

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        return self.mix(BM.linear(xa, self.w_in), pos, slots, meta, cache, li, eps)

    def mix(self, y, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H, d, dv = y.shape[0], s.heads, s.dim, s.vdim
        nqk, nv = H * d, H * dv
        q, k = y[:, :nqk].view(T, H, d), y[:, nqk:2 * nqk].view(T, H, d)
        v = y[:, 2 * nqk:2 * nqk + nv].view(T, H, dv)
        g = y[:, 2 * nqk + nv:2 * nqk + 2 * nv]
        a = BM.linear(y[:, 2 * nqk + 2 * nv:].contiguous(), self.w_a2, self.b_a2).view(T, H, d)
        o = GM.gla_scan(q, k, v, a, s.tau, d ** -0.5, cache.state[li]["gla"], meta.cu_q, meta.state_slots, pos,
                        meta.q_lens_host)
        return BM.linear(GM.head_rms_silu(o, self.norm, g, eps, y.dtype), self.w_o)


class SideBySide(nn.Module):
    """Two mixers reading the same input: one projection launch over both mixers' input rows, then
    ``(rms_norm(left) * out_l + rms_norm(right) * out_r) / 2`` over the model width."""
    cache_kind = "both"

    def __init__(self, left: nn.Module, right: nn.Module, out_l, out_r):
        super().__init__()
        self.left, self.right = left, right
        ws, bs = [left.w_in, right.w_in], [left.b_in, right.b_in]
        self.n_left = int(left.w_in.shape[0])
        self.w_in = nn.Parameter(torch.cat([w.data for w in ws], 0).contiguous(), requires_grad=False)
        self.b_in = None
        if any(b is not None for b in bs):
            bs = [b.data if b is not None else torch.zeros(w.shape[0], dtype=w.dtype, device=w.device)
                  for w, b in zip(ws, bs)]
            self.b_in = nn.Parameter(torch.cat(bs, 0).contiguous(), requires_grad=False)
        left.w_in = right.w_in = None                  # the fused copy is the one that runs
        left.b_in = right.b_in = None
        self.out_l = nn.Parameter(out_l, requires_grad=False)
        self.out_r = nn.Parameter(out_r, requires_grad=False)

    def cache_spec(self):
        out = []
        for m in (self.left, self.right):
            c = m.cache_spec()
            out += c if isinstance(c, list) else ([c] if c is not None else [])
        return out

    def ensure_table(self, max_pos: int):
        self.left.ensure_table(max_pos)
        self.right.ensure_table(max_pos)

    @property
    def table(self):
        return getattr(self.left, "table", None)

    @table.setter
    def table(self, v):
        for m in (self.left, self.right):
            if hasattr(m, "table"):
                m.table = v

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        y = BM.linear(xa, self.w_in, self.b_in)
        a = self.left.mix(y[:, :self.n_left], pos, slots, meta, cache, li, eps)
        b = self.right.mix(y[:, self.n_left:], pos, slots, meta, cache, li, eps)
        return GM.rms_pair_mean(a, b, self.out_l, self.out_r, eps, xa.dtype)


class GroupedAttention(nn.Module):
    cache_kind = "rows"

    def __init__(self, s: GroupedAttentionSpec, w_q, w_k, q_norm, k_norm, talk, w_g, w_o):
        super().__init__()
        if s.heads % s.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        self.s = s
        parts = [w_q, w_k] + ([w_g] if w_g is not None else [])
        self.w_in = nn.Parameter(torch.cat(parts, 0).contiguous(), requires_grad=False)      # [q | k | gate] rows
        self.q_norm = nn.Parameter(q_norm, requires_grad=False) if q_norm is not None else None
        self.k_norm = nn.Parameter(k_norm, requires_grad=False) if k_norm is not None else None
        self.talk = nn.Parameter(talk.float().contiguous(), requires_grad=False) if talk is not None else None
        self.w_o = nn.Parameter(w_o, requires_grad=False)
        self.table: Optional[torch.Tensor] = None

    def cache_spec(self):
        return ("rows", 2 * self.s.kv_heads * self.s.dim)

    def ensure_table(self, max_pos: int):
        if self.table is None or self.table.shape[0] < max_pos or self.table.device != self.w_o.device:
            n = max(256, 1 << (max_pos - 1).bit_length())
            if self.s.rot is None or self.s.rot.dims == 0:     # no rotation: one pair turned by the angle 0
                self.table = torch.tensor([1.0, 0.0]).repeat(n, 1, 1).contiguous().to(self.w_o.device)
            else:
                self.table = SM.rope_table(n, self.s.rot.dims, self.s.rot.base, self.s.rot.scaling).to(self.w_o.device)
        return self.table

    def forward(self, xa, pos, slots, meta: AttnMeta, cache, li: int, eps: float):
        s = self.s
        T, H, G, d = xa.shape[0], s.heads, s.kv_heads, s.dim
        y = BM.linear(xa, self.w_in)
        q = y[:, :H * d].view(T, H, d)
        k = y[:, H * d:(H + G) * d].view(T, G, d)
        gate = y[:, (H + G) * d:] if s.out_gate else None
        qf = BM.qk_norm_rope_store(q, k, self.q_norm, self.k_norm, eps, self.table, pos, slots, cache.rows[li])
        o = BM.talk_attention(qf, cache.rows[li], meta.block_tables, meta.seq_of, pos, s.scale, self.talk, gate, G,
                              meta.q_lens_host, meta.seq_lens_host, xa.dtype)
        return BM.linear(o, self.w_o)


class ReluSqFF(nn.Module):
    def __init__(self, w_up, w_down):
        super().__init__()
        self.w_up = nn.Parameter(w_up, requires_grad=False)
        self.w_down = nn.Parameter(w_down, requires_grad=False)

    def forward(self, xa, x32=None):
        return BM.linear(BM.relu_sq(BM.linear(xa, self.w_up)), self.w_down), None


class SigmoidMoE(nn.Module):
    """``w_gu`` [E, 2 ff, W] (every expert's gate rows, then its up rows),
    ``w_down`` [E, W, ff]; the router runs in f32 on the f32 input."""

    def __init__(self, s: MoESpec, router, w_gu, w_down, shared_gu=None, shared_down=None):
        super().__init__()
        self.s = s
        self.router = nn.Parameter(router.float().contiguous(), requires_grad=False)
        self.w_gu = nn.Parameter(w_gu.contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(w_down.contiguous(), requires_grad=False)
        self.shared_gu = nn.Parameter(shared_gu, requires_grad=False) if shared_gu is not None else None
        self.shared_down = nn.Parameter(shared_down, requires_grad=False) if shared_down is not None else None

    def forward(self, xa, x32):
        s = self.s
        idx, wts = BM.moe_route(F.linear(x32, self.router), s.top)
        y = BM.moe_experts(xa, idx, wts, self.w_gu, self.w_down, s.expert.limit, s.expert.alpha)
        ys = None
        if self.shared_gu is not None:
            ys = BM.linear(BM.glu_clamp(BM.linear(xa, self.shared_gu), s.shared.limit, s.shared.alpha), self.shared_down)
        return y, ys


class SoftmaxMoE(nn.Module):
    """``w_gu`` [E, 2 ff, W] (every expert's gate rows, then its up rows), ``w_down`` [E, W, ff].  The router's
    logits are f32 products with the input; the ``top`` largest win, their weights are the softmax over the chosen
    logits only and multiply the experts' *outputs*; experts ``W_down (silu(W_gate h) * (W_up h))``."""

    def __init__(self, s: MoESpec, router, w_gu, w_down):
        super().__init__()
        self.s = s
        self.router = nn.Parameter(router.float().contiguous(), requires_grad=False)
        self.w_gu = nn.Parameter(w_gu.contiguous(), requires_grad=False)
        self.w_down = nn.Parameter(w_down.contiguous(), requires_grad=False)

    def forward(self, xa, x32=None):
        s = self.s
        idx, wts = BM.moe_route(F.linear(xa.float() if x32 is None else x32, self.router), s.top, "softmax")
        y = BM.moe_experts(xa, idx, wts, self.w_gu, self.w_down, float("inf"), 1.0, 0.0, "output")
        return y, None


class TokenSide(nn.Module):
    """x += rms_norm(W_proj (gelu_tanh(W_gate x) * e)) * w, with e the layer's
    slice of the token-side table's row of the token."""

    def __init__(self, w_gate, w_proj, norm, offset: int):
        super().__init__()
        self.w_gate = nn.Parameter(w_gate, requires_grad=False)
        self.w_proj = nn.Parameter(w_proj, requires_grad=False)
        self.norm = nn.Parameter(norm, requires_grad=False)
        self.offset = offset

    def forward(self, x, xa, ids, table, eps: float, act):
        g = BM.side_gate(BM.linear(xa, self.w_gate), table, ids, self.offset)
        return BM.add_rms_norm_(x, BM.linear(g, self.w_proj), self.norm, eps, act)


class HybridLayer(nn.Module):
    def __init__(self, mixer: nn.Module, norm1: torch.Tensor, mlp: Optional[DenseFF], norm2: Optional[torch.Tensor]):
        super().__init__()
        self.mixer, self.mlp = mixer, mlp
        self.norm1 = nn.Parameter(norm1, requires_grad=False)
        self.norm2 = nn.Parameter(norm2, requires_grad=False) if norm2 is not None else None

    def cache_specs(self):
        return _spec_list(self.mixer.cache_spec())

    def forward(self, x, xa, ids, pos, slots, meta, cache, li: int, model):
        s, act = model.spec, model.dtype
        y = self.mixer(xa, pos, slots, meta, cache, li, s.norm_eps)
        xa = SM.add_scaled_layer_norm_(x, y, self.norm1, s.norm_eps, s.residual_mult, act)
        if self.mlp is not None:
            xa = SM.add_scaled_layer_norm_(x, self.mlp(xa), self.norm2, s.norm_eps, s.residual_mult, act)
        return xa


class PreNormLayer(nn.Module):
    """x += mixer(norm1(x)); x += ff(norm2(x)).  ``carry`` is the previous sublayer's result that is not yet in
    ``x`` (None at the first layer): the launch that forms a norm adds it first, and the layer hands its own last
    result on the same way (the model adds the final one with its own norm)."""

    def __init__(self, mixer: nn.Module, norm1: torch.Tensor, mlp: Optional[nn.Module], norm2: Optional[torch.Tensor]):
        super().__init__()
        self.mixer, self.mlp = mixer, mlp
        self.norm1 = nn.Parameter(norm1, requires_grad=False)
        self.norm2 = nn.Parameter(norm2, requires_grad=False) if norm2 is not None else None

    def cache_specs(self):
        return _spec_list(self.mixer.cache_spec())

    def forward(self, x, carry, ids, pos, slots, meta, cache, li: int, model):
        s, act = model.spec, model.dtype
        h = BM.add_rms_norm_rows_(x, carry, self.norm1, s.norm_eps, act)
        y = self.mixer(h, pos, slots, meta, cache, li, s.norm_eps)
        if self.mlp is None:
            return y
        h = BM.add_rms_norm_rows_(x, y, self.norm2, s.norm_eps, act)
        return self.mlp(h)


class ParallelLayer(nn.Module):
    """h = norm(x);  x += ls1 * mixer(h + conv(h)) + ls2 * ff(h);  then the
    token-side input.  ``canon`` [W, taps] or None, ``ls1`` / ``ls2`` [W] or
    None, ``mlp`` returns (result, second result or None) and may be None."""

    def __init__(self, mixer: nn.Module, norm1: torch.Tensor, mlp: Optional[nn.Module], canon=None, ls1=None, ls2=None,
                 side: Optional[TokenSide] = None):
        super().__init__()
        self.mixer, self.mlp, self.side = mixer, mlp, side
        self.norm1 = nn.Parameter(norm1, requires_grad=False)
        self.canon = nn.Parameter(canon.float().contiguous(), requires_grad=False) if canon is not None else None
        self.ls1 = nn.Parameter(ls1.float(), requires_grad=False) if ls1 is not None else None
        self.ls2 = nn.Parameter(ls2.float(), requires_grad=False) if ls2 is not None else None

    def cache_specs(self):
        out = _spec_list(self.mixer.cache_spec())
        if self.canon is not None and self.canon.shape[1] > 1:
            out.append(("state", {"canon": (self.canon.shape[1] - 1, self.canon.shape[0])}))
        return out

    def forward(self, x, xa, ids, pos, slots, meta, cache, li: int, model):
        s, act = model.spec, model.dtype
        if self.canon is not None and self.canon.shape[1] > 1:
            h32, ha, hm = BM.norm_canon(x, self.norm1, s.norm_eps, self.canon, cache.state[li]["canon"], meta.cu_q,
                                        meta.seq_of, meta.state_slots, pos, meta.q_lens_host, act)
        else:
            h32, ha = BM.rms_norm_rows(x, self.norm1, s.norm_eps, act)
            hm = ha if self.canon is None else (h32 * (1.0 + self.canon[:, 0])).to(act)
        ym = self.mixer(hm, pos, slots, meta, cache, li, s.norm_eps)
        y2, y3 = self.mlp(ha, h32) if self.mlp is not None else (None, None)
        xa = BM.residual_add_scaled_(x, ym, self.ls1, y2, y3, self.ls2, act)
        if self.side is not None:
            xa = self.side(x, xa, ids, model.side_embed, s.norm_eps, act)
        return xa


class TwoNormParallelLayer(nn.Module):
    """h = LN1(x) shifted towards the previous token's (``shift`` [W] or None), x += mixer(h) + ff(LN2(x)); then the
    token-side input.  LayerNorms with a weight and no bias; the previous token's LN1(x) is per-sequence state.
    ``mlp`` returns (result, second result or None) and may be None."""

    def __init__(self, mixer: nn.Module, norm1: torch.Tensor, mlp: Optional[nn.Module], norm2: Optional[torch.Tensor],
                 shift: Optional[torch.Tensor] = None, side: Optional[TokenSide] = None):
        super().__init__()
        self.mixer, self.mlp, self.side = mixer, mlp, side
        self.norm1 = nn.Parameter(norm1, requires_grad=False)
        self.norm2 = nn.Parameter(norm2, requires_grad=False) if norm2 is not None else None
        self.shift = nn.Parameter(shift.float().contiguous(), requires_grad=False) if shift is not None else None

    def cache_specs(self):
        out = _spec_list(self.mixer.cache_spec())
        if self.shift is not None:
            out.append(("state", {"shift": (self.norm1.shape[0],)}))
        return out

    def forward(self, x, xa, ids, pos, slots, meta, cache, li: int, model):
        s, act = model.spec, model.dtype
        st = cache.state[li]["shift"] if self.shift is not None else None
        h1, h2 = GM.layer_norm_pair_shift(x, self.norm1, self.norm2 if self.mlp is not None else None, self.shift,
                                          s.norm_eps, st, meta.cu_q, meta.seq_of, meta.state_slots, pos,
                                          meta.q_lens_host, act)
        ym = self.mixer(h1, pos, slots, meta, cache, li, s.norm_eps)
        y2, y3 = self.mlp(h2, None) if self.mlp is not None else (None, None)
        xa = BM.residual_add_scaled_(x, ym, None, y2, y3, None, act)
        if self.side is not None:
            xa = self.side(x, xa, ids, model.side_embed, s.norm_eps, act)
        return xa


# name -> (spec class, module class): a design's config reader maps its layer
# types onto these
MIXERS: Dict[str, tuple] = {"latent_attention": (LatentAttentionSpec, LatentAttention), "mlstm": (MLSTMSpec, MLSTM),
                            "grouped_attention": (GroupedAttentionSpec, GroupedAttention),
                            "ssm": (SSMSpec, SSMMixer), "masked_attention": (MaskedAttentionSpec, MaskedAttention),
                            "mingru": (MinGRUSpec, MinGRU),
                            "gated_linear_attention": (GatedLinearAttentionSpec, GatedLinearAttention),
                            "side_by_side": (SideBySideSpec, SideBySide)}


# ---------------------------------------------------------------------- model
class HybridCausalLM(nn.Module):
    ragged_step = True              # forward_tokens takes sequences of unequal new-token counts
    native_lib = "seqmix"           # the kernels it needs (ops.require_seqmix)

    def __init__(self, spec: HybridSpec, embed: torch.Tensor, bigram: Optional[torch.Tensor],
                 layers: List[nn.Module], final_norm: torch.Tensor, head: torch.Tensor, dtype=torch.bfloat16,
                 side_embed: Optional[torch.Tensor] = None):
        super().__init__()
        self.spec, self.dtype = spec, dtype
        self.embed_tokens = nn.Parameter(embed, requires_grad=False)
        self.bigram = nn.Parameter(bigram, requires_grad=False) if bigram is not None else None
        self.side_embed = nn.Parameter(side_embed, requires_grad=False) if side_embed is not None else None
        self.layers = nn.ModuleList(layers)
        self.norm = nn.Parameter(final_norm, requires_grad=False)
        # a tied head (head None) is the embedding table itself
        self.lm_head = nn.Parameter(head, requires_grad=False) if head is not None else self.embed_tokens
        self.tp_group = None
        self.first_stage = self.last_stage = True
        self.capture_layers: Optional[list] = None      # debugging: residual stream after every layer

    @property
    def device(self):
        return self.norm.device

    @property
    def has_state(self) -> bool:
        return any(c is not None and c[0] == "state" for L in self.layers for c in L.cache_specs())

    def graph_max_batch(self) -> int:
        return 0                    # ragged steps are launched eagerly

    def ensure_rope_cache(self, max_pos: int):
        for L in self.layers:
            L.mixer.ensure_table(max_pos)

    def cache_bytes_per_token(self) -> int:
        eb = torch.empty(0, dtype=self.dtype).element_size()
        return sum(c[1] * eb for L in self.layers for c in L.cache_specs() if c is not None and c[0] == "rows")

    def make_cache(self, max_tokens: int, batch: int = 1, block_size: int = 64, kv_fp8: int = 0,
                   num_blocks: Optional[int] = None, num_slots: Optional[int] = None):
        from .cache import HybridCache
        if kv_fp8:
            raise ValueError("hybrid decoders keep their latent rows in the activation dtype (no fp8 cache)")
        nblk = num_blocks or batch * ((max_tokens + block_size - 1) // block_size)
        self.ensure_rope_cache(max_tokens + 1)
        return HybridCache([L.cache_specs() for L in self.layers], nblk, num_slots or batch, block_size,
                           self.dtype, self.device)

    @staticmethod
    def complete_meta(meta: AttnMeta, pos: torch.Tensor, T: int) -> AttnMeta:
        """fill the ragged fields of a uniform (B x Tq) step"""
        if meta.cu_q is None:
            dev = pos.device
            meta.cu_q = torch.arange(0, (meta.B + 1) * meta.Tq, meta.Tq, dtype=torch.int32, device=dev)
            meta.q_lens_host = [meta.Tq] * meta.B
            meta.seq_of = torch.arange(meta.B, dtype=torch.int32, device=dev).repeat_interleave(meta.Tq)
        if meta.seq_lens_host is None:
            meta.seq_lens_host = [int(v) for v in meta.seq_lens.tolist()]
        return meta

    def forward_tokens(self, ids: torch.Tensor, pos: torch.Tensor, slots: torch.Tensor, meta: AttnMeta, cache,
                       logits_idx: Optional[torch.Tensor] = None, return_hidden: bool = False,
                       hidden_in: Optional[torch.Tensor] = None):
        """ids / pos / slots [T] (sequence after sequence, ``meta.cu_q``);
        ``meta.prev_ids`` the token before each one (-1: none) when the model
        has a bigram table; ``meta.state_slots`` when it has recurrent layers.
        Returns f32 logits [len(logits_idx) or T, vocab]."""
        s = self.spec
        T = ids.shape[0]
        meta = self.complete_meta(meta, pos, T)
        if self.has_state and meta.state_slots is None:
            raise ValueError("a model with recurrent layers needs AttnMeta.state_slots")
        self.ensure_rope_cache(max(meta.seq_lens_host) + 1)
        act = self.dtype
        if hidden_in is not None:
            x = hidden_in.float().contiguous().clone()
        elif self.bigram is not None:
            if meta.prev_ids is None:
                raise ValueError("a model with a bigram table needs AttnMeta.prev_ids")
            b = s.bigram
            x = SM.embed_bigram(ids, meta.prev_ids, self.embed_tokens, self.bigram, b.mul_prev, b.mul_cur)
        else:
            x = F.embedding(ids, self.embed_tokens).float()
        pre = s.block == "pre_norm"         # ``xa`` is then the last sublayer's result, still to be added to x
        xa = None if pre else (x if act == torch.float32 else x.to(act))
        for li, L in enumerate(self.layers):
            xa = L(x, xa, ids, pos, slots, meta, cache, li, self)
            if self.capture_layers is not None:
                self.capture_layers.append(x + xa.float() if pre else x.clone())
        if not self.last_stage:
            return x.add_(xa.float()) if pre and xa is not None else x
        if logits_idx is not None:
            x = x.index_select(0, logits_idx)
            xa = xa.index_select(0, logits_idx) if pre and xa is not None else xa
        if pre:
            xn = BM.add_rms_norm_rows_(x, xa, self.norm, s.norm_eps, act)
        elif s.norm == "layer_norm":
            xn = SM.layer_norm_f32(x, self.norm, s.norm_eps, act)
        else:
            xn = BM.rms_norm_rows(x, self.norm, s.norm_eps, act)[1]
        if return_hidden:
            return xn
        logits = BM.linear(xn, self.lm_head).float()
        if s.final_softcap:
            return GM.softcap_(logits, s.final_softcap)
        return logits.mul_(s.logit_scale) if s.logit_scale != 1.0 else logits
