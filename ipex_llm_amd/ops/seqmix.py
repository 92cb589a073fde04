"""Sequence-mixing ops of the hybrid decoders (models/hybrid.py): latent
attention over a paged latent cache, the mLSTM matrix-memory recurrence over
per-sequence state slots, and the element-wise steps around them.

Every op works on a *ragged step*: ``T`` tokens laid out sequence after
sequence, sequence ``b`` bringing ``cu[b + 1] - cu[b]`` new tokens at
positions ``pos`` (prompt portions and single decoded tokens side by side).
GPU tensors run the HIP kernels of ``csrc/hip/seqmix.hip`` (the small
``_C_seqmix.so`` library, or the full ``_C.so`` which contains them too); CPU
tensors run the plain torch forms below, which are also what the kernels are
tested against.

Precision (both paths): positions / angles, attention scores and
weights, every norm, the residual sum, the recurrence with its gates and its
state are f32 whatever the activation dtype is; projections and the
activation of the feed-forward may be 16-bit with f32 accumulation.
"""
from __future__ import annotations

import math
from typing import List, Optional

import torch
import torch.nn.functional as F

__all__ = ["embed_bigram", "add_scaled_layer_norm_", "layer_norm_f32", "latent_kv_store", "rope_rows_",
           "latent_attention", "mlstm_scan", "head_rms_gate", "glu_gelu", "glu_act", "GLU_ACTS", "rope_table", "native"]


def native(t: torch.Tensor) -> bool:
    """True when ``t`` is a GPU tensor (the HIP kernels must then run)."""
    if not t.is_cuda:
        return False
    from . import require_seqmix
    require_seqmix()
    return True


def _ops():
    return torch.ops.ipex_llm_amd


# ------------------------------------------------------------------ rotary table
def rope_table(max_pos: int, dims: int, base: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """f32 ``[max_pos, dims / 2, 2]`` cos / sin of interleaved-pair rotary
    positions, angles formed in f64 on the host and rounded once.

    ``scaling`` (YaRN): keys ``factor``, ``original``, ``fast``, ``slow``.
    With d(t) = dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(d(fast)), 0),
    hi = min(ceil(d(slow)), dims - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 1e-3), 0, 1),
    pair i turns at f_i (1 - ramp_i) + f_i ramp_i / factor, and cos / sin carry
    the magnitude 0.1 ln(factor) + 1.

    ``scaling`` with the keys ``factor``, ``low``, ``high``, ``original`` (the
    rule of Llama 3.1) acts on wavelengths l = 2 pi / f instead: f is kept where
    l < original / high, divided by the factor where l > original / low, and in
    between blended with s = (original / l - low) / (high - low) as
    (1 - s) f / factor + s f."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if scaling and "low" in scaling:
        factor, low, high = float(scaling["factor"]), float(scaling["low"]), float(scaling["high"])
        orig = float(scaling["original"])
        wl = 2.0 * math.pi / f
        s = (orig / wl - low) / (high - low) if high != low else torch.zeros_like(f)
        f = torch.where(wl < orig / high, f, torch.where(wl > orig / low, f / factor, (1 - s) * f / factor + s * f))
    elif scaling:
        factor = float(scaling["factor"])

        def d_of(t):
            return dims * math.log(float(scaling["original"]) / (2 * math.pi * float(t))) / (2 * math.log(float(base)))
        lo = max(math.floor(d_of(scaling["fast"])), 0)
        hi = min(math.ceil(d_of(scaling["slow"])), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    a = torch.arange(max_pos, dtype=torch.float64)[:, None] * f[None]
    return torch.stack([a.cos() * mag, a.sin() * mag], -1).float().contiguous()


# ------------------------------------------------------------------ embedding
def embed_bigram(ids: torch.Tensor, prev_ids: torch.Tensor, embed: torch.Tensor, bigram: torch.Tensor,
                 mul_prev: int, mul_cur: int) -> torch.Tensor:
    """f32 ``[T, W]``: ``embed[id] + bigram[row]`` with row = (prev mul_prev +
    id mul_cur) mod buckets, and the table's last row (index ``buckets``) for a
    token without a predecessor (``prev_ids < 0``)."""
    buckets = bigram.shape[0] - 1
    if native(ids):
        return _ops().sm_embed_bigram(ids.contiguous(), prev_ids.contiguous(), embed, bigram, mul_prev, mul_cur)
    row = (prev_ids.long() * mul_prev + ids.long() * mul_cur) % buckets
    row = torch.where(prev_ids < 0, torch.full_like(row, buckets), row)
    return embed[ids].float() + bigram[row].float()


# ------------------------------------------------------------------ norms
def add_scaled_layer_norm_(x: torch.Tensor, y: torch.Tensor, w: torch.Tensor, eps: float, mult: float,
                           act_dtype: torch.dtype) -> torch.Tensor:
    """``x += mult * LN(y) * w`` on the f32 residual stream ``x`` in place
    (LN without bias, variance = mean squared deviation); returns ``x`` in
    ``act_dtype`` for the next projection (``x`` itself when that is f32)."""
    if native(x):
        return _ops().sm_add_scaled_layer_norm(x, y.contiguous(), w, eps, mult, act_dtype == torch.float32)
    yf = y.float()
    mu = yf.mean(-1, keepdim=True)
    d = yf - mu
    x.add_(d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w.float() * mult)
    return x if act_dtype == torch.float32 else x.to(act_dtype)


def layer_norm_f32(x: torch.Tensor, w: torch.Tensor, eps: float, act_dtype: torch.dtype) -> torch.Tensor:
    """bias-free LayerNorm of f32 rows, result in ``act_dtype``."""
    if native(x):
        return _ops().sm_layer_norm(x.contiguous(), w, eps, act_dtype == torch.float32)
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return (d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w.float()).to(act_dtype)


# ------------------------------------------------------------------ rotary
def _rot_pairs(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x f32 [..., dims] interleaved pairs, cs [..., dims / 2, 2]"""
    u, v = x[..., 0::2], x[..., 1::2]
    c, s = cs[..., 0], cs[..., 1]
    return torch.stack([u * c - v * s, v * c + u * s], -1).flatten(-2)


def rope_rows_(q: torch.Tensor, offset: int, table: torch.Tensor, pos: torch.Tensor) -> torch.Tensor:
    """Rotate, in place, the ``dims = 2 * table.shape[1]`` values of every head
    of ``q`` [T, H, D] that start at ``offset`` (interleaved pairs, f32 math)."""
    dims = 2 * table.shape[1]
    if native(q):
        _ops().sm_rope_rows_(q, offset, table, pos)
        return q
    cs = table[pos.long()][:, None]                                 # [T, 1, dims / 2, 2]
    q[..., offset:offset + dims] = _rot_pairs(q[..., offset:offset + dims].float(), cs).to(q.dtype)
    return q


def latent_kv_store(dkv: torch.Tensor, norm_w: torch.Tensor, eps: float, rank: int, table: torch.Tensor,
                    pos: torch.Tensor, slots: torch.Tensor, rows: torch.Tensor) -> None:
    """One cache row per token: ``[rms_norm(dkv[:rank]) * norm_w | rope(dkv[rank:])]``
    written at row index ``slots`` of the paged pool ``rows`` [blocks, bs, width]
    (the rotation covers the first ``2 * table.shape[1]`` values of the rotated part)."""
    if native(dkv):
        _ops().sm_latent_kv_store(dkv, norm_w, eps, rank, table, pos, slots, rows)
        return
    dims = 2 * table.shape[1]
    c = dkv[:, :rank].float()
    c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * norm_w.float()
    kr = dkv[:, rank:].float().clone()
    kr[:, :dims] = _rot_pairs(kr[:, :dims], table[pos.long()])
    flat = rows.view(-1, rows.shape[-1])
    flat.index_copy_(0, slots.long(), torch.cat([c, kr], -1).to(rows.dtype))


# ------------------------------------------------------------------ latent attention
def latent_attention(q_lat: torch.Tensor, q_rot: torch.Tensor, rows: torch.Tensor, block_tables: torch.Tensor,
                     seq_of: torch.Tensor, pos: torch.Tensor, scale: float, gate: Optional[torch.Tensor],
                     q_lens: List[int], ctx_lens: List[int], out_dtype: torch.dtype, window: int = 0) -> torch.Tensor:
    """Causal softmax attention in the latent space over the paged rows
    ``[latent (r) | rotated key (dr)]``: for token t of sequence b and head h

        s_j = (q_lat[t, h] . c_j + q_rot[t, h] . kr_j) * scale      for j <= pos[t]
        out[t, h] = sigmoid(gate[t, h]) * sum_j softmax(s)_j c_j     [r]

    (scores, softmax and the weighted sum in f32).  ``window`` > 0: only the
    keys pos[t] - window < j <= pos[t] count (the token itself and the
    window - 1 before it).  ``q_rot`` may be a strided view.  ``q_lens`` /
    ``ctx_lens``: host copies of every sequence's new-token count and key count."""
    T, H, r = q_lat.shape
    window = int(window or 0)
    if native(q_lat):
        return _latent_attention_gpu(q_lat, q_rot, rows, block_tables, seq_of, pos, float(scale), gate, q_lens,
                                     ctx_lens, out_dtype, window)
    out = torch.empty(T, H, r, dtype=torch.float32, device=q_lat.device)
    bs = rows.shape[1]
    t0 = 0
    for b, (n, L) in enumerate(zip(q_lens, ctx_lens)):
        if n == 0:
            continue
        nb = (L + bs - 1) // bs
        kv = rows[block_tables[b, :nb].long()].reshape(nb * bs, -1)[:L].float()
        c, kr = kv[:, :r], kv[:, r:]
        ql, qr = q_lat[t0:t0 + n].float(), q_rot[t0:t0 + n].float()
        sc = (torch.einsum("thr,lr->thl", ql, c) + torch.einsum("thd,ld->thl", qr, kr)) * scale
        j, p = torch.arange(L, device=sc.device)[None, :], pos[t0:t0 + n].long()[:, None]
        vis = (j <= p) & (j > p - window) if window > 0 else j <= p
        sc = sc.masked_fill(~vis[:, None, :], float("-inf"))
        out[t0:t0 + n] = torch.einsum("thl,lr->thr", torch.softmax(sc, -1), c)
        t0 += n
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[..., None]
    return out.to(out_dtype)


# Portions of at least this many tokens take the library-GEMM path on the GPU:
# scores and the weighted sum of latents are GEMM-shaped ([tokens x heads, r + dr]
# x [r + dr, keys] and [tokens x heads, keys] x [keys, r]) and go to the vendor
# GEMM with f32 results (as models/mla.py does for its latent attention), with
# the fused causal softmax kernel between them.  Shorter portions and decoded
# tokens run the one-pass flash kernel, which keeps everything in f32 registers.
GEMM_MIN_Q = int(__import__("os").environ.get("ILLM_LATENT_GEMM_MIN", "128"))
GEMM_Q_BLOCK = int(__import__("os").environ.get("ILLM_LATENT_GEMM_BLOCK", "1024"))
_mm_out_f32: Optional[bool] = None


def _mm_f32(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """a @ b with an f32 result (16-bit operands: f32 accumulation, no rounding of the result)"""
    global _mm_out_f32
    if a.dtype == torch.float32:
        return a @ b
    if _mm_out_f32 is None:
        try:
            torch.mm(a[:16, :16].contiguous(), a[:16, :16].contiguous(), out_dtype=torch.float32)
            _mm_out_f32 = True
        except (TypeError, RuntimeError):
            _mm_out_f32 = False
    if _mm_out_f32:
        return torch.mm(a, b, out_dtype=torch.float32)
    return a.float() @ b.float()


def _latent_attention_gemm(q_lat, q_rot, rows, table_row, pos, scale, L: int, n: int, window: int = 0) -> torch.Tensor:
    """one sequence's portion of n >= GEMM_MIN_Q tokens ending at key count L -> f32 [n, H, r]"""
    _, H, r = q_lat.shape
    bs = rows.shape[1]
    nb = (L + bs - 1) // bs
    kv = rows[table_row[:nb].long()].reshape(nb * bs, -1)           # this sequence's rows, in order
    out = torch.empty(n, H, r, dtype=torch.float32, device=q_lat.device)
    f32 = q_lat.dtype == torch.float32
    for t0 in range(0, n, GEMM_Q_BLOCK):
        t1 = min(n, t0 + GEMM_Q_BLOCK)
        Lb = min(nb * bs, (L - n + t1 + 7) // 8 * 8)                 # keys the block's last token sees (rows past L: weight 0)
        k0 = max(0, L - n + t0 - window + 1) // 8 * 8 if window > 0 else 0      # the first key its first token sees
        q2 = torch.cat([q_lat[t0:t1], q_rot[t0:t1]], -1).reshape((t1 - t0) * H, -1)
        sc = _mm_f32(q2, kv[k0:Lb].t()).contiguous()
        hi, lo = _ops().sm_causal_softmax(sc, pos[t0:t1].contiguous(), H, scale, f32, k0, window)
        c = kv[k0:Lb, :r]
        o = _mm_f32(hi, c)
        if not f32:
            o += _mm_f32(lo, c)
        out[t0:t1] = o.view(t1 - t0, H, r)
    return out


def _latent_attention_gpu(q_lat, q_rot, rows, block_tables, seq_of, pos, scale, gate, q_lens, ctx_lens, out_dtype,
                          window: int = 0):
    T, H, r = q_lat.shape
    f32 = out_dtype == torch.float32
    # sizes the flash kernel cannot hold in LDS / registers: every portion takes the library-product path
    min_q = GEMM_MIN_Q if _ops().sm_latent_attention_fits(not f32, H, r, q_rot.shape[-1]) > 0 else 1
    big = [b for b, n in enumerate(q_lens) if n >= min_q]
    if not big:
        return _ops().sm_latent_attention(q_lat.contiguous(), q_rot, rows, block_tables, seq_of, pos, scale, gate,
                                          max(ctx_lens), f32, window)
    out = torch.empty(T, H, r, dtype=out_dtype, device=q_lat.device)
    small, small_ctx, t0 = [], 1, 0
    for b, (n, L) in enumerate(zip(q_lens, ctx_lens)):
        if n >= min_q:
            o = _latent_attention_gemm(q_lat[t0:t0 + n], q_rot[t0:t0 + n], rows, block_tables[b], pos[t0:t0 + n], scale,
                                       L, n, window)
            if gate is not None:
                o = o * torch.sigmoid(gate[t0:t0 + n].float())[..., None]
            out[t0:t0 + n] = o.to(out_dtype)
        elif n:
            small.append(torch.arange(t0, t0 + n, device=q_lat.device))
            small_ctx = max(small_ctx, L)
        t0 += n
    if small:
        idx = torch.cat(small)
        o = _ops().sm_latent_attention(q_lat[idx].contiguous(), q_rot[idx], rows, block_tables,
                                       seq_of[idx].contiguous(), pos[idx].contiguous(), scale,
                                       gate[idx] if gate is not None else None, small_ctx, f32, window)
        out[idx] = o
    return out


# ------------------------------------------------------------------ mLSTM
def mlstm_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, i_pre: torch.Tensor, f_pre: torch.Tensor,
               i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float, state: dict, cu: torch.Tensor,
               state_slots: torch.Tensor, pos: torch.Tensor, q_lens: List[int]) -> torch.Tensor:
    """Matrix-memory recurrence, token by token, per sequence and head.

    q, k [T, H, d], v [T, H, dv], gate pre-activations [T, H]; ``state`` holds
    f32 ``S`` [slots, H, d, dv], ``n`` [slots, H, d], ``m`` [slots, H], read at
    ``state_slots[b]`` (a sequence whose first new token is at position 0
    starts from zero instead) and written back after the last token.  With
    i = cap tanh((i_pre + b_i) / cap), f = logsigmoid(cap tanh((f_pre + b_f) / cap)):

        m' = max(f + m, i);  a = exp(f + m - m');  b = exp(i - m')
        S' = a S + b k v^T;  n' = a n + b k
        h  = S'^T q' / (max(|n' . q'|, exp(-m')) + 1e-6),   q' = q d^-1/2

    Returns h f32 [T, H, dv]."""
    T, H, d = q.shape
    dv = v.shape[-1]
    if native(q) and d <= 256:          # (larger key sizes: the token loop below, on the device)
        return _mlstm_scan_gpu(q, k, v, i_pre, f_pre, i_bias, f_bias, float(cap), state, cu, state_slots, pos, q_lens)
    out = torch.empty(T, H, dv, dtype=torch.float32, device=q.device)
    ig = cap * torch.tanh((i_pre.float() + i_bias.float()) / cap)
    fg = F.logsigmoid(cap * torch.tanh((f_pre.float() + f_bias.float()) / cap))
    qf, kf, vf = q.float() * d ** -0.5, k.float(), v.float()
    slots = state_slots.tolist()
    first = pos.tolist()
    t0 = 0
    for b, nq in enumerate(q_lens):
        if nq == 0:
            continue
        sl = slots[b]
        if first[t0] == 0:
            S = torch.zeros(H, d, dv, device=q.device)
            n = torch.zeros(H, d, device=q.device)
            m = torch.zeros(H, device=q.device)
        else:
            S, n, m = state["S"][sl].clone(), state["n"][sl].clone(), state["m"][sl].clone()
        for t in range(t0, t0 + nq):
            mn = torch.maximum(fg[t] + m, ig[t])
            a, bb = torch.exp(fg[t] + m - mn), torch.exp(ig[t] - mn)
            S = a[:, None, None] * S + bb[:, None, None] * kf[t][:, :, None] * vf[t][:, None, :]
            n = a[:, None] * n + bb[:, None] * kf[t]
            m = mn
            den = torch.maximum((n * qf[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
            out[t] = torch.einsum("hdv,hd->hv", S, qf[t]) / den[:, None]
        state["S"][sl], state["n"][sl], state["m"][sl] = S, n, m
        t0 += nq
    return out


# Portions of at least MLSTM_CHUNK_MIN tokens take the chunk-parallel form on
# the GPU: the recurrence is linear in the state, so within a chunk of C tokens
#   m_t   = F_t + max(M, max_{s<=t}(i_s - F_s))            F: prefix sums of f in the chunk, M: m at its start
#   num_t = e^{F_t + M - m_t} q_t^T S + sum_{s<=t} e^{F_t - F_s + i_s - m_t} (q_t . k_s) v_s
# (and the same with n for the normaliser), every exponent <= 0.  The pairwise
# part of all chunks and the chunk-end state increments K^T diag(w) V are
# batched f32 products; only S_{c+1} = e^{..} S_c + U_c runs chunk after chunk.
# Everything is f32; the token-sequential kernel takes what is left over.
MLSTM_CHUNK = int(__import__("os").environ.get("ILLM_MLSTM_CHUNK", "128"))
# None: by state size -- 512 tokens for large states (d x dv >= 64 K, where the sequential kernel's token
# takes longest), 2048 otherwise (measured on MI355X: below these the one-launch kernel is faster)
MLSTM_CHUNK_MIN = (lambda e: int(e) if e else None)(__import__("os").environ.get("ILLM_MLSTM_CHUNK_MIN"))


def _chunk_min(d: int, dv: int) -> int:
    if MLSTM_CHUNK_MIN is not None:
        return max(MLSTM_CHUNK_MIN, MLSTM_CHUNK)
    return max(MLSTM_CHUNK, 512 if d * dv >= 65536 else 2048)


def mlstm_chunked(q, k, v, ig, fg, S0, n0, m0, C: int):
    """q (already scaled), k [n, H, d], v [n, H, dv], log gates ig, fg [n, H],
    all f32, n a multiple of C; S0 [H, d, dv], n0 [H, d], m0 [H].  Returns
    h [n, H, dv] and the state after the last token."""
    n, H, d = q.shape
    dv = v.shape[-1]
    NC = n // C
    Q = q.view(NC, C, H, d).permute(2, 0, 1, 3)
    K = k.view(NC, C, H, d).permute(2, 0, 1, 3)
    V = v.view(NC, C, H, dv).permute(2, 0, 1, 3)
    I = ig.view(NC, C, H).permute(2, 0, 1)
    F_ = fg.view(NC, C, H).permute(2, 0, 1).cumsum(-1)                # [H, NC, C]
    g = I - F_
    G = g.cummax(-1).values
    Ftot, Gtot = F_[..., -1], G[..., -1]                                # [H, NC]
    # m at every chunk start: M_{c+1} = Ftot_c + max(M_c, Gtot_c) (scalars per head: on the host)
    Fh, Gh = Ftot.cpu(), Gtot.cpu()
    Ms = torch.empty(H, NC + 1, dtype=torch.float32)
    Ms[:, 0] = m0.cpu()
    for c in range(NC):
        Ms[:, c + 1] = Fh[:, c] + torch.maximum(Ms[:, c], Gh[:, c])
    Ms = Ms.to(q.device)
    Mc, Mn = Ms[:, :-1], Ms[:, 1:]
    m = F_ + torch.maximum(Mc[..., None], G)                            # [H, NC, C]
    dec_in = torch.exp(F_ + Mc[..., None] - m)
    vis = torch.ones(C, C, dtype=torch.bool, device=q.device).tril()
    D = torch.exp(((F_ - m)[..., :, None] + g[..., None, :]).masked_fill(~vis, float("-inf")))
    A = torch.matmul(Q, K.transpose(-1, -2)) * D                        # [H, NC, C, C]
    w = torch.exp(Ftot[..., None] - F_ + I - Mn[..., None])             # weight of token s in the chunk-end state
    U = torch.matmul(K.transpose(-1, -2), w[..., None] * V)             # [H, NC, d, dv]
    un = torch.matmul(K.transpose(-1, -2), w[..., None]).squeeze(-1)    # [H, NC, d]
    dec = torch.exp(Ftot + Mc - Mn)
    S_all = torch.empty(H, NC + 1, d, dv, dtype=torch.float32, device=q.device)
    n_all = torch.empty(H, NC + 1, d, dtype=torch.float32, device=q.device)
    S_all[:, 0], n_all[:, 0] = S0, n0
    for c in range(NC):
        torch.addcmul(U[:, c], S_all[:, c], dec[:, c, None, None], out=S_all[:, c + 1])
        torch.addcmul(un[:, c], n_all[:, c], dec[:, c, None], out=n_all[:, c + 1])
    num = torch.matmul(A, V) + dec_in[..., None] * torch.matmul(Q, S_all[:, :-1])
    nq = A.sum(-1) + dec_in * torch.matmul(Q, n_all[:, :-1, :, None]).squeeze(-1)
    den = torch.maximum(nq.abs(), torch.exp(-m)) + 1e-6
    h = (num / den[..., None]).permute(1, 2, 0, 3).reshape(n, H, dv)
    return h, S_all[:, -1], n_all[:, -1], Ms[:, -1]


def _mlstm_scan_gpu(q, k, v, i_pre, f_pre, i_bias, f_bias, cap, state, cu, state_slots, pos, q_lens):
    T, H, d = q.shape
    dv = v.shape[-1]
    C = MLSTM_CHUNK
    cmin = _chunk_min(d, dv)
    if max(q_lens) < cmin:
        return _ops().sm_mlstm_scan(q, k, v, i_pre, f_pre, i_bias, f_bias, cap, state["S"], state["n"], state["m"],
                                    cu, state_slots, pos, max(q_lens))
    out = torch.empty(T, H, dv, dtype=torch.float32, device=q.device)
    slots = state_slots.tolist()
    rest, rest_lens, rest_slots, t0 = [], [], [], 0              # what the sequential kernel takes afterwards
    for b, nq in enumerate(q_lens):
        nfull = (nq // C) * C if nq >= cmin else 0
        if nfull:
            sl, r = slots[b], slice(t0, t0 + nfull)
            ig = cap * torch.tanh((i_pre[r].float() + i_bias) / cap)
            fg = F.logsigmoid(cap * torch.tanh((f_pre[r].float() + f_bias) / cap))
            fresh = int(pos[t0]) == 0
            S0 = torch.zeros(H, d, dv, device=q.device) if fresh else state["S"][sl]
            n0 = torch.zeros(H, d, device=q.device) if fresh else state["n"][sl]
            m0 = torch.zeros(H, device=q.device) if fresh else state["m"][sl]
            h, S1, n1, m1 = mlstm_chunked(q[r].float() * d ** -0.5, k[r].float(), v[r].float(), ig, fg, S0, n0, m0, C)
            out[r] = h
            state["S"][sl], state["n"][sl], state["m"][sl] = S1, n1, m1
        if nq - nfull:
            rest.append(torch.arange(t0 + nfull, t0 + nq, device=q.device))
            rest_lens.append(nq - nfull)
            rest_slots.append(slots[b])
        t0 += nq
    if rest:
        idx = torch.cat(rest)
        cu_r = torch.tensor([0] + list(__import__("itertools").accumulate(rest_lens)), dtype=torch.int32, device=q.device)
        ss_r = torch.tensor(rest_slots, dtype=torch.int32, device=q.device)
        out[idx] = _ops().sm_mlstm_scan(q[idx], k[idx], v[idx], i_pre[idx], f_pre[idx], i_bias, f_bias, cap, state["S"],
                                        state["n"], state["m"], cu_r, ss_r, pos[idx].contiguous(), max(rest_lens))
    return out


def head_rms_gate(h: torch.Tensor, norm_w: torch.Tensor, gate_pre: torch.Tensor, eps: float,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """h f32 [T, H, dv]: every head divided by its root mean square, then
    ``* norm_w`` (all heads' size) ``* sigmoid(gate_pre)`` -> [T, H * dv]."""
    T, H, dv = h.shape
    if native(h):
        return _ops().sm_head_rms_gate(h.contiguous(), norm_w, gate_pre, eps, out_dtype == torch.float32)
    y = h * torch.rsqrt((h * h).mean(-1, keepdim=True) + eps)
    y = y.reshape(T, H * dv) * norm_w.float() * torch.sigmoid(gate_pre.float())
    return y.to(out_dtype)


# ------------------------------------------------------------------ feed-forward
GLU_ACTS = {"gelu_tanh": 0, "relu": 1, "silu": 2}


def glu_act(gu: torch.Tensor, act: str) -> torch.Tensor:
    """[T, 2 I] = [gate | up] -> act(gate) * up  [T, I] (f32 math), ``act`` a key of ``GLU_ACTS``."""
    I = gu.shape[-1] // 2
    if native(gu):
        return _ops().sm_glu_act(gu.contiguous(), GLU_ACTS[act])
    g, u = gu[..., :I].float(), gu[..., I:].float()
    if act == "relu":
        a = torch.relu(g)
    elif act == "silu":
        a = F.silu(g)
    else:
        a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
    return (a * u).to(gu.dtype)


def glu_gelu(gu: torch.Tensor) -> torch.Tensor:
    """[T, 2 I] = [gate | up] -> gelu_tanh(gate) * up  [T, I] (f32 math)."""
    I = gu.shape[-1] // 2
    if native(gu):
        return _ops().sm_glu_gelu(gu.contiguous())
    g, u = gu[..., :I].float(), gu[..., I:].float()
    a = 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g * g * g)))
    return (a * u).to(gu.dtype)
