"""Ops of the parallel-residual hybrid blocks (models/hybrid.py): RMS norms
with one number or a vector, the short causal convolution in front of a
mixer, grouped-query attention whose heads' scores are mixed before the
softmax, clamped-GLU experts behind a sigmoid router, and the element-wise
steps around them.

Like ``ops/seqmix.py`` every op takes a *ragged step* (``T`` tokens laid out
sequence after sequence).  GPU tensors run the HIP kernels of
``csrc/hip/blockmix_*.hip``; CPU tensors run the torch forms below.

Precision (both paths): norms, the residual sum, rotary angles, attention
scores / mixing / softmax / weights, router logits and scores are f32
whatever the activation dtype is; projections, expert products and
activations may be 16-bit with f32 accumulation.
"""
from __future__ import annotations

import math
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from .seqmix import native, _mm_f32

__all__ = ["linear", "rms_norm_rows", "add_rms_norm_rows_", "canon_conv", "norm_canon", "qk_norm_rope_store", "talk_attention", "relu_sq", "glu_clamp",
           "residual_add_scaled_", "side_gate", "add_rms_norm_", "moe_route", "moe_experts"]


def _ops():
    return torch.ops.ipex_llm_amd


ROUTE_MODES = {"sigmoid": 0, "softmax": 1}


# ------------------------------------------------------------------ projections
def linear(x: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``x W^T (+ b)`` for rows ``x`` [T, K] and ``w`` [N, K]: decode-size steps (at most 16 rows, 16-bit) stream
    the weight once through the skinny-GEMM kernel the dense decoders use (csrc/hip/dense_gemv.hip), everything
    else is a library GEMM."""
    if x.is_cuda and x.dim() == 2 and x.shape[0] <= 16 and x.dtype == torch.bfloat16 and w.dtype == x.dtype and \
            x.shape[1] % 8 == 0 and w.is_contiguous() and native(x):
        return _ops().dense_linear(x, w, b)
    return F.linear(x, w, b)


# ------------------------------------------------------------------ norms
def rms_norm_rows(x: torch.Tensor, w: torch.Tensor, eps: float, act_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """``x / sqrt(mean(x^2) + eps) * w`` for f32 rows ``x`` [T, W]; ``w`` holds
    W numbers or ONE number for all coordinates.  Returns the result in f32 and
    in ``act_dtype`` (the same tensor when that is f32)."""
    if native(x):
        h, ha = _ops().bm_rms_norm_rows(x.contiguous(), w.reshape(-1), eps, act_dtype == torch.float32)
        return h, ha
    h = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w.float().reshape(-1)
    return h, (h if act_dtype == torch.float32 else h.to(act_dtype))


def add_rms_norm_(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, eps: float, act_dtype: torch.dtype) -> torch.Tensor:
    """``x += y / sqrt(mean(y^2) + eps) * w`` on the f32 residual rows in place;
    returns ``x`` in ``act_dtype``."""
    if native(x):
        return _ops().bm_add_rms_norm(x, y.contiguous(), w, eps, act_dtype == torch.float32)
    yf = y.float()
    x.add_(yf * torch.rsqrt((yf * yf).mean(-1, keepdim=True) + eps) * w.float())
    return x if act_dtype == torch.float32 else x.to(act_dtype)


def add_rms_norm_rows_(x: torch.Tensor, y: Optional[torch.Tensor], w: torch.Tensor, eps: float,
                       act_dtype: torch.dtype) -> torch.Tensor:
    """``x += y`` on the f32 residual rows in place (``y`` in the activation
    dtype, or None for nothing to add), then ``x / sqrt(mean(x^2) + eps) * w``
    (``w`` [W]) in ``act_dtype``: the residual sum of one sublayer and the norm
    in front of the next in one pass."""
    if native(x):
        return _ops().bm_add_rms_norm_rows(x, None if y is None else y.contiguous(), w, eps, act_dtype == torch.float32)
    if y is not None:
        x.add_(y.float())
    return (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w.float()).to(act_dtype)


def residual_add_scaled_(x: torch.Tensor, y1: torch.Tensor, s1: Optional[torch.Tensor], y2: Optional[torch.Tensor],
                         y3: Optional[torch.Tensor], s2: Optional[torch.Tensor], act_dtype: torch.dtype) -> torch.Tensor:
    """``x += s1 * y1 + s2 * (y2 + y3)`` on the f32 residual rows in place
    (``s1`` / ``s2``: per-coordinate scales or None for 1; ``y2`` / ``y3`` may be
    None; each ``y`` is f32 or the activation dtype).  The two sublayers' results
    are summed first and then added to ``x``.  Returns ``x`` in ``act_dtype``."""
    if native(x):
        return _ops().bm_residual_add_scaled(x, y1.contiguous(), s1, None if y2 is None else y2.contiguous(),
                                             None if y3 is None else y3.contiguous(), s2, act_dtype == torch.float32)
    d = y1.float() * (s1.float() if s1 is not None else 1.0)
    if y2 is not None or y3 is not None:
        f = (y2.float() if y2 is not None else 0.0) + (y3.float() if y3 is not None else 0.0)
        d = d + f * (s2.float() if s2 is not None else 1.0)
    x.add_(d)
    return x if act_dtype == torch.float32 else x.to(act_dtype)


# ------------------------------------------------------------------ short convolution
def canon_conv(h: torch.Tensor, w: torch.Tensor, state: torch.Tensor, cu: torch.Tensor, seq_of: torch.Tensor,
               state_slots: torch.Tensor, pos: torch.Tensor, q_lens: List[int], act_dtype: torch.dtype) -> torch.Tensor:
    """``h + conv(h)``: a causal per-channel convolution over time added to its
    own input.  ``h`` f32 [T, W], ``w`` [W, taps]:

        out_t = h_t + sum_j w[:, j] * h_(t - taps + 1 + j)

    with zeros before a sequence's start.  ``state`` f32 [slots, taps - 1, W]
    holds, per sequence, the inputs of its last ``taps - 1`` positions (oldest
    first); a portion that does not start at position 0 reads what lies before
    it from there, and every portion leaves its last inputs there."""
    taps = w.shape[1]
    if native(h):
        return _ops().bm_canon_conv(h.contiguous(), w, state, cu, seq_of, state_slots, pos, act_dtype == torch.float32)
    out = torch.empty_like(h)
    wf = w.float()
    slots, first = state_slots.tolist(), pos.tolist()
    t0 = 0
    for b, n in enumerate(q_lens):
        if n == 0:
            continue
        p0 = first[t0]
        hist = state[slots[b]].clone()                                   # positions p0 - taps + 1 .. p0 - 1
        if p0 < taps - 1:
            hist[:taps - 1 - p0] = 0.0
        ext = torch.cat([hist, h[t0:t0 + n]], 0)
        acc = h[t0:t0 + n].clone()
        for j in range(taps):
            acc += wf[:, j][None] * ext[j:j + n]
        out[t0:t0 + n] = acc
        state[slots[b]] = ext[n:]
        t0 += n
    return out if act_dtype == torch.float32 else out.to(act_dtype)


def norm_canon(x: torch.Tensor, norm_w: torch.Tensor, eps: float, w: torch.Tensor, state: torch.Tensor, cu: torch.Tensor,
               seq_of: torch.Tensor, state_slots: torch.Tensor, pos: torch.Tensor, q_lens: List[int],
               act_dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """``rms_norm_rows`` then ``canon_conv`` (one launch on the GPU; a step in which every sequence brings one
    token also advances the state in it).  Returns the norm's result in f32 and in ``act_dtype`` and
    ``h + conv(h)`` in ``act_dtype``."""
    if native(x):
        single = len(q_lens) == x.shape[0] and all(n == 1 for n in q_lens)
        return _ops().bm_norm_canon(x.contiguous(), norm_w.reshape(-1), eps, w, state, cu, seq_of, state_slots, pos,
                                    single, act_dtype == torch.float32)
    h, ha = rms_norm_rows(x, norm_w, eps, act_dtype)
    return h, ha, canon_conv(h, w, state, cu, seq_of, state_slots, pos, q_lens, act_dtype)


# ------------------------------------------------------------------ grouped attention with mixed scores
def _rot_half(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x f32 [..., dims]: value i is paired with value i + dims / 2; cs [..., dims / 2, 2]"""
    half = x.shape[-1] // 2
    u, v = x[..., :half], x[..., half:]
    c, s = cs[..., 0], cs[..., 1]
    return torch.cat([u * c - v * s, v * c + u * s], -1)


def qk_norm_rope_store(q: torch.Tensor, k: torch.Tensor, q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor],
                       eps: float, table: torch.Tensor, pos: torch.Tensor, slots: torch.Tensor,
                       rows: torch.Tensor) -> torch.Tensor:
    """Per-head RMS norm (weights of the head's size, shared by the heads) and
    half-split rotary positions on the first ``2 * table.shape[1]`` values of
    every head of ``q`` [T, H, d] and ``k`` [T, G, d] (strided views allowed).
    Writes one cache row per token at row index ``slots`` of the paged pool
    ``rows`` [blocks, bs, 2 G d]: ``[normed, rotated keys | keys as projected]``
    -- the second half is what the attention uses as values.  Returns the
    queries f32 [T, H, d]."""
    T, H, d = q.shape
    G = k.shape[1]
    if native(q):
        return _ops().bm_qk_norm_rope_store(q, k, q_norm, k_norm, eps, table, pos, slots, rows)
    dims = 2 * table.shape[1]
    cs = table[pos.long()][:, None]
    qf, kf = q.float(), k.float()
    if q_norm is not None:
        qf = qf * torch.rsqrt((qf * qf).mean(-1, keepdim=True) + eps) * q_norm.float()
    kn = kf
    if k_norm is not None:
        kn = kf * torch.rsqrt((kf * kf).mean(-1, keepdim=True) + eps) * k_norm.float()
    qf = torch.cat([_rot_half(qf[..., :dims], cs), qf[..., dims:]], -1)
    kn = torch.cat([_rot_half(kn[..., :dims], cs), kn[..., dims:]], -1)
    flat = rows.view(-1, rows.shape[-1])
    flat.index_copy_(0, slots.long(), torch.cat([kn.reshape(T, G * d), kf.reshape(T, G * d)], -1).to(rows.dtype))
    return qf.contiguous()


# GPU paths by portion length.  Decoded tokens and short portions: the one-pass kernel, a workgroup per token.
# 16-bit portions of at least MFMA_MIN_Q tokens, head sizes 64 / 128 and 4 / 8 / 16 heads: the matrix-core kernel,
# a workgroup per 16 tokens.  Other portions of at least GEMM_MIN_Q tokens (and every portion of sizes the one-pass
# kernel cannot hold): library products with the fused mixing softmax between them.
MFMA_MIN_Q = int(__import__("os").environ.get("ILLM_TALK_MFMA_MIN", "32"))
GEMM_MIN_Q = int(__import__("os").environ.get("ILLM_TALK_GEMM_MIN", "128"))
GEMM_Q_BLOCK = int(__import__("os").environ.get("ILLM_TALK_GEMM_BLOCK", "512"))


def talk_attention(q: torch.Tensor, rows: torch.Tensor, block_tables: torch.Tensor, seq_of: torch.Tensor,
                   pos: torch.Tensor, scale: float, talk: Optional[torch.Tensor], gate: Optional[torch.Tensor], G: int,
                   q_lens: List[int], ctx_lens: List[int], out_dtype: torch.dtype) -> torch.Tensor:
    """Causal grouped-query attention over paged rows ``[keys (G d) | values (G d)]``
    with the heads' scores mixed before the softmax.  For token t (position p)
    of a sequence, query head h (key / value head h // (H / G)) and key j <= p:

        s[h, j]  = (q[t, h] . key_j[h // rep]) * scale
        s'[h, j] = sum_g talk[h, g] s[g, j]
        out[t, h] = sum_j softmax_j(s'[h, :]) value_j[h // rep]

    then ``out * sigmoid(gate)`` element by element (gate [T, H d]).  ``q`` f32
    [T, H, d]; scores, mixing, softmax and the weighted sum are f32.  Returns
    [T, H d] in ``out_dtype``."""
    T, H, d = q.shape
    if native(q):
        return _talk_attention_gpu(q, rows, block_tables, seq_of, pos, float(scale), talk, gate, G, q_lens, ctx_lens,
                                   out_dtype)
    rep = H // G
    out = torch.empty(T, H, d, dtype=torch.float32, device=q.device)
    bs = rows.shape[1]
    t0 = 0
    for b, (n, L) in enumerate(zip(q_lens, ctx_lens)):
        if n == 0:
            continue
        nb = (L + bs - 1) // bs
        kv = rows[block_tables[b, :nb].long()].reshape(nb * bs, -1)[:L].float()
        kk = kv[:, :G * d].view(L, G, d).repeat_interleave(rep, 1)
        vv = kv[:, G * d:].view(L, G, d).repeat_interleave(rep, 1)
        sc = torch.einsum("thd,lhd->htl", q[t0:t0 + n], kk) * scale
        if talk is not None:
            sc = torch.einsum("hg,gtl->htl", talk.float(), sc)
        vis = torch.arange(L, device=sc.device)[None, :] <= pos[t0:t0 + n].long()[:, None]
        sc = sc.masked_fill(~vis[None], float("-inf"))
        out[t0:t0 + n] = torch.einsum("htl,lhd->thd", torch.softmax(sc, -1), vv)
        t0 += n
    out = out.reshape(T, H * d)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(out_dtype)


def _talk_attention_gemm(q, rows, table_row, pos, scale, talk, G: int, L: int, n: int) -> torch.Tensor:
    """one sequence's portion of n tokens ending at key count L -> f32 [n, H, d]: scores and weighted sums
    as library products per key / value head, the mixing + causal softmax fused in one kernel between them"""
    _, H, d = q.shape
    rep = H // G
    bs = rows.shape[1]
    nb = (L + bs - 1) // bs
    kv = rows[table_row[:nb].long()].reshape(nb * bs, -1)
    f32 = rows.dtype == torch.float32
    out = torch.empty(n, H, d, dtype=torch.float32, device=q.device)
    for t0 in range(0, n, GEMM_Q_BLOCK):
        t1 = min(n, t0 + GEMM_Q_BLOCK)
        nt = t1 - t0
        Lb = min(nb * bs, (L - n + t1 + 7) // 8 * 8)
        sc = torch.empty(nt, H, Lb, dtype=torch.float32, device=q.device)
        qb = q[t0:t1]
        for g in range(G):
            kg = kv[:Lb, g * d:(g + 1) * d]
            qg = qb[:, g * rep:(g + 1) * rep].reshape(nt * rep, d)
            if f32:
                s = qg @ kg.t()
            else:                                   # f32 queries against 16-bit keys: hi + lo halves of q
                qh = qg.to(rows.dtype)
                ql = (qg - qh.float()).to(rows.dtype)
                s = _mm_f32(qh, kg.t()) + _mm_f32(ql, kg.t())
            sc[:, g * rep:(g + 1) * rep] = s.view(nt, rep, Lb)
        hi, lo = _ops().bm_talk_softmax(sc.view(nt * H, Lb), pos[t0:t1].contiguous(), H, scale, talk, f32)
        hi = hi.view(nt, H, Lb)
        lo = lo.view(nt, H, Lb) if not f32 else None
        for g in range(G):
            vg = kv[:Lb, (G + g) * d:(G + g + 1) * d]
            hg = hi[:, g * rep:(g + 1) * rep].reshape(nt * rep, Lb)
            o = _mm_f32(hg, vg)
            if not f32:
                o += _mm_f32(lo[:, g * rep:(g + 1) * rep].reshape(nt * rep, Lb), vg)
            out[t0:t1, g * rep:(g + 1) * rep] = o.view(nt, rep, d)
    return out


def _talk_attention_gpu(q, rows, block_tables, seq_of, pos, scale, talk, gate, G, q_lens, ctx_lens, out_dtype):
    T, H, d = q.shape
    f32 = out_dtype == torch.float32
    fits = _ops().bm_talk_attention_fits(not f32, H, G, d) > 0
    mfma = not f32 and MFMA_MIN_Q > 0 and _ops().bm_talk_prefill_fits(H, G, d) > 0
    min_q = (min(MFMA_MIN_Q, GEMM_MIN_Q) if mfma else GEMM_MIN_Q) if fits else 1
    if all(n < min_q for n in q_lens):
        return _ops().bm_talk_attention(q.contiguous(), rows, block_tables, seq_of, pos, scale, talk, gate, G,
                                        max(ctx_lens), f32)
    q = q.contiguous()
    out = torch.empty(T, H * d, dtype=out_dtype, device=q.device)
    small, small_ctx, t0 = [], 1, 0
    for b, (n, L) in enumerate(zip(q_lens, ctx_lens)):
        if n >= min_q and mfma:
            _ops().bm_talk_prefill(q, rows, block_tables[b], pos, t0, n, L, scale, talk, gate, G, out)
        elif n >= min_q:
            o = _talk_attention_gemm(q[t0:t0 + n], rows, block_tables[b], pos[t0:t0 + n], scale, talk, G, L, n)
            o = o.view(n, H * d)
            if gate is not None:
                o = o * torch.sigmoid(gate[t0:t0 + n].float())
            out[t0:t0 + n] = o.to(out_dtype)
        elif n:
            small.append(torch.arange(t0, t0 + n, device=q.device))
            small_ctx = max(small_ctx, L)
        t0 += n
    if small:
        idx = torch.cat(small)
        o = _ops().bm_talk_attention(q[idx].contiguous(), rows, block_tables, seq_of[idx].contiguous(),
                                     pos[idx].contiguous(), scale, talk, gate[idx] if gate is not None else None, G,
                                     small_ctx, f32)
        out[idx] = o
    return out


# ------------------------------------------------------------------ feed-forward
def relu_sq(y: torch.Tensor) -> torch.Tensor:
    """``max(y, 0)^2`` (f32 math), same dtype."""
    if native(y):
        return _ops().bm_relu_sq(y.contiguous())
    r = torch.relu(y.float())
    return (r * r).to(y.dtype)


def glu_clamp(gu: torch.Tensor, limit: float, alpha: float = 1.702) -> torch.Tensor:
    """[T, 2 I] = [gate | up] -> ``g sigmoid(alpha g) (u + 1)`` with
    g = min(gate, limit), u = clamp(up, -limit, limit)  (f32 math)."""
    I = gu.shape[-1] // 2
    if native(gu):
        return _ops().bm_glu_clamp(gu.contiguous(), limit, alpha)
    g = gu[..., :I].float().clamp(max=limit)
    u = gu[..., I:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gu.dtype)


def side_gate(z: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, offset: int) -> torch.Tensor:
    """``gelu_tanh(z) * table[ids, offset : offset + z.shape[1]]`` (f32 math), z's dtype."""
    n = z.shape[1]
    if native(z):
        return _ops().bm_side_gate(z.contiguous(), table, ids, offset)
    zf = z.float()
    a = 0.5 * zf * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (zf + 0.044715 * zf * zf * zf)))
    return (a * table[ids.long(), offset:offset + n].float()).to(z.dtype)


# ------------------------------------------------------------------ experts
def moe_route(z: torch.Tensor, top: int, mode: str = "sigmoid") -> Tuple[torch.Tensor, torch.Tensor]:
    """Router logits ``z`` f32 [T, E] -> the ``top`` experts with the largest
    logits per token (int32 [T, top], lowest index first among equals) and
    their weights (f32 [T, top]): ``mode`` "sigmoid": ``sigmoid(z)`` of each
    chosen expert, not renormalised; "softmax": the softmax over the chosen
    logits only."""
    if mode not in ROUTE_MODES:
        raise ValueError(f"unknown router mode {mode!r}")
    if native(z) and z.shape[1] <= 512 and (mode == "sigmoid" or top <= 64):
        return _ops().bm_moe_route(z.contiguous(), top, ROUTE_MODES[mode])
    # (sizes past the kernel's: library sort)
    val, idx = torch.sort(z.float(), dim=-1, descending=True, stable=True)
    val = val[:, :top]
    w = torch.sigmoid(val) if mode == "sigmoid" else torch.softmax(val, -1)
    return idx[:, :top].to(torch.int32).contiguous(), w.contiguous()


def moe_experts(h: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, w_gu: torch.Tensor, w_down: torch.Tensor,
                limit: float, alpha: float = 1.702, up_shift: float = 1.0, weigh: str = "input") -> torch.Tensor:
    """Sum over a token's chosen experts.  ``weigh`` "input": ``expert_e(w h)``,
    the routing weight multiplies the expert's *input*; "output":
    ``w expert_e(h)``.  ``h`` [T, W] in the activation dtype, ``w_gu``
    [E, 2 ff, W] (gate rows, then up rows), ``w_down`` [E, W, ff]; expert:
    ``W_down (g sigmoid(alpha g) (u + up_shift))`` with g = min(gate, limit),
    u = clamp(up, -limit, limit) (``limit`` may be infinite; alpha = 1,
    up_shift = 0: the SiLU-gated unit).  Returns f32 [T, W]."""
    T, W = h.shape
    top = idx.shape[1]
    if weigh not in ("input", "output"):
        raise ValueError(f"unknown weighing {weigh!r}")
    if native(h):
        return _ops().bm_moe_experts(h.contiguous(), idx, wts, w_gu, w_down, limit, alpha, up_shift, weigh == "output")
    out = torch.zeros(T, W, dtype=torch.float32, device=h.device)
    E = w_gu.shape[0]
    I = w_gu.shape[1] // 2
    for k in range(top):
        xin = (h.float() * wts[:, k:k + 1]).to(h.dtype) if weigh == "input" else h
        for e in range(E):
            sel = (idx[:, k] == e).nonzero().squeeze(-1)
            if sel.numel() == 0:
                continue
            gu = F.linear(xin[sel], w_gu[e])
            g = gu[..., :I].float().clamp(max=limit)
            u = gu[..., I:].float().clamp(-limit, limit)
            y = (g * torch.sigmoid(alpha * g) * (u + up_shift)).to(h.dtype)
            r = F.linear(y, w_down[e]).float()
            out[sel] += r * wts[sel, k:k + 1] if weigh == "output" else r
    return out
