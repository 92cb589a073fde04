"""Grouped-query attention over paged ``[keys | values]`` rows with a bounded
view of the past (a sliding window or position-aligned chunks) and an optional
sink in the softmax, plus the fused step in front of it: RMS norm of queries
and keys (per head or over the whole projection), rotary positions in either
pair layout, and the cache append.  Used by ``models/hybrid.py``
``MaskedAttention``.

Every op takes a *ragged step* like ``ops/seqmix.py``.  GPU tensors run the
HIP kernels of ``csrc/hip/maskattn.hip``; CPU tensors run the torch forms
below, which are also what the kernels are tested against.

Precision (both paths): norms, angles, scores, the softmax with its sink and
the weighted sum are f32 whatever the activation dtype is; the queries leave
the first step as f32 and are never rounded.
"""
from __future__ import annotations

import os
from typing import List, Optional

import torch

from .seqmix import native

__all__ = ["MASKS", "LAYOUTS", "first_visible", "qkv_norm_rope_store", "masked_attention", "sigmoid_gate"]

MASKS = {"causal": 0, "window": 1, "chunk": 2}
LAYOUTS = {"pairs": 0, "half": 1}


def _ops():
    return torch.ops.ipex_llm_amd


def first_visible(pos: torch.Tensor, mask: str, size: int) -> torch.Tensor:
    """the first key position a query at ``pos`` sees: 0 (causal), pos - size + 1
    clamped at 0 (window: itself and the size - 1 tokens before it), or the start
    of pos's chunk (chunks of ``size`` positions counted from position 0)"""
    if mask == "causal":
        return torch.zeros_like(pos)
    if mask == "window":
        return (pos - (size - 1)).clamp(min=0)
    if mask == "chunk":
        return pos - pos % size
    raise ValueError(f"unknown mask {mask!r}")


def _turn(x: torch.Tensor, cs: torch.Tensor, layout: str) -> torch.Tensor:
    """rotate the first ``2 * cs.shape[-2]`` values of every head of x f32 [T, heads, n]; cs [T, 1, dims / 2, 2]"""
    dims = 2 * cs.shape[-2]
    c, s = cs[..., 0], cs[..., 1]
    out = x.clone()
    if layout == "half":
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    else:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    return out


def qkv_norm_rope_store(q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                        q_norm: Optional[torch.Tensor], k_norm: Optional[torch.Tensor], whole: bool, eps: float,
                        table: Optional[torch.Tensor], layout: str, pos: torch.Tensor, slots: torch.Tensor,
                        rows: Optional[torch.Tensor]) -> torch.Tensor:
    """RMS norm and rotary positions of ``q`` [T, H, d] and ``k`` [T, G, d]
    (strided views allowed), and one cache row per token.

    ``whole``: the norm runs over all heads of a token at once (weights of the
    whole projection's size, [H d] and [G d]); otherwise per head (weights [d],
    shared by the heads).  A missing weight means no norm.  The rotation turns
    the first ``2 * table.shape[1]`` values of every head, pairing value i with
    i + dims / 2 (``layout`` "half") or 2 i with 2 i + 1 ("pairs"); no table: no
    rotation.  When ``k`` is given, ``[keys (normed, rotated) | v as projected]``
    is written at row index ``slots`` of the paged pool ``rows``
    [blocks, bs, G d + G dv]; a layer that reads another layer's rows passes
    ``k = v = rows = None``.  Returns the queries f32 [T, H, d]."""
    T, H, d = q.shape
    if native(q):
        return _ops().ma_qkv_norm_rope_store(q, k, v, q_norm, k_norm, whole, eps, table, LAYOUTS[layout], pos, slots,
                                             rows)
    cs = table[pos.long()][:, None] if table is not None else None

    def prep(x, w):
        x = x.float()
        if w is not None:
            if whole:
                n = x.shape[1] * x.shape[2]
                flat = x.reshape(T, n)
                x = (flat * torch.rsqrt((flat * flat).mean(-1, keepdim=True) + eps) * w.float()).view(x.shape)
            else:
                x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w.float()
        return _turn(x, cs, layout) if cs is not None else x

    qf = prep(q, q_norm)
    if k is not None:
        kf = prep(k, k_norm)
        flat = rows.view(-1, rows.shape[-1])
        flat.index_copy_(0, slots.long(), torch.cat([kf.reshape(T, -1), v.float().reshape(T, -1)], -1).to(rows.dtype))
    return qf.contiguous()


# GPU paths by portion: decoded tokens and short pieces run the one-pass kernel, a workgroup per (token, key head).
# With chunks, a portion splits into pieces that each see only keys of their own chunk (the rest of the chunk the
# portion starts in, whole chunks, the start of a last chunk): pieces of at least GEMM_MIN_CHUNK queries run as
# batched library products, with the fused softmax (sink, causal mask inside the chunk) between them.
GEMM_MIN_CHUNK = int(os.environ.get("ILLM_MASKATTN_GEMM_MIN", "128"))
# Under a sliding window, portions of at least WINDOW_GEMM_MIN queries run the same way in blocks of WINDOW_Q_BLOCK
# queries: a block's keys are the kept first tokens and everything from its first query's window start on.
WINDOW_GEMM_MIN = int(os.environ.get("ILLM_MASKATTN_WINDOW_GEMM_MIN", "1536"))
WINDOW_Q_BLOCK = int(os.environ.get("ILLM_MASKATTN_WINDOW_BLOCK", "512"))


def masked_attention(q: torch.Tensor, rows: torch.Tensor, G: int, dv: int, block_tables: torch.Tensor,
                     seq_of: torch.Tensor, pos: torch.Tensor, scale: float, mask: str, size: int,
                     sink: Optional[torch.Tensor], q_lens: List[int], ctx_lens: List[int],
                     out_dtype: torch.dtype, softcap: float = 0.0, keep_first: int = 0,
                     talk: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Grouped-query attention over paged rows ``[keys (G d) | values (G dv)]``.
    For token t (position p), query head h (key / value head h // (H / G)) and
    the visible keys ``first_visible(p) <= j <= p`` (and, with ``keep_first``,
    the keys ``j < keep_first`` of the sequence's start as well):

        s_j = (q[t, h] . key_j) * scale;   softcap > 0:  s_j <- softcap tanh(s_j / softcap)
        w_j = exp(s_j) / (sum_visible exp(s_i) + exp(sink[h]))      (no sink: the plain softmax)
        talk [H, H] given:  w_j[h] <- sum_g talk[h, g] w_j[g]       (the heads' weights mixed after the softmax)
        out[t, h] = sum_j w_j value_j

    The sink is one more term of the denominator: it has no key and no value,
    is not scaled or capped, counts once and is not mixed.  ``q`` f32 [T, H, d];
    everything is f32.  Returns [T, H dv] in ``out_dtype``."""
    T, H, d = q.shape
    if native(q):
        return _masked_attention_gpu(q, rows, G, dv, block_tables, seq_of, pos, float(scale), mask, int(size), sink,
                                     q_lens, ctx_lens, out_dtype, float(softcap), int(keep_first), talk)
    rep = H // G
    out = torch.empty(T, H, dv, dtype=torch.float32, device=q.device)
    bs = rows.shape[1]
    t0 = 0
    for b, (n, L) in enumerate(zip(q_lens, ctx_lens)):
        if n == 0:
            continue
        nb = (L + bs - 1) // bs
        kv = rows[block_tables[b, :nb].long()].reshape(nb * bs, -1)[:L].float()
        kk = kv[:, :G * d].view(L, G, d).repeat_interleave(rep, 1)
        vv = kv[:, G * d:].view(L, G, dv).repeat_interleave(rep, 1)
        p = pos[t0:t0 + n].long()
        sc = torch.einsum("thd,lhd->htl", q[t0:t0 + n], kk) * scale
        j = torch.arange(L, device=sc.device)[None, :]
        if softcap > 0:
            sc = softcap * torch.tanh(sc / softcap)
        vis = (j <= p[:, None]) & ((j >= first_visible(p, mask, size)[:, None]) | (j < keep_first))
        sc = sc.masked_fill(~vis[None], float("-inf"))
        top = sc.max(-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink.float()[:, None, None])
        e = torch.exp(sc - top)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink.float()[:, None, None] - top)
        wts = e / den
        if talk is not None:
            wts = torch.einsum("hg,gtl->htl", talk.float(), wts)
        out[t0:t0 + n] = torch.einsum("htl,lhd->thd", wts, vv)
        t0 += n
    return out.reshape(T, H * dv).to(out_dtype)


def _pieces_gemm(q, rows, table_row, G, dv, scale, sink, t0, lo, nc, nk, nq, out, softcap=0.0, talk=None):
    """``nc`` pieces of chunks of one sequence: piece i holds the ``nk`` keys from position ``lo + i nk`` (a chunk's
    first position) on, and its queries are its last ``nq`` positions (whole chunks: nq == nk == the chunk size;
    one piece with nq < nk: a portion that starts inside a chunk); the step's token ``t0`` is the first query.
    Scores and weighted sums are batched products over (piece, key head), the sink softmax is fused between them."""
    _, H, d = q.shape
    rep = H // G
    bs = rows.shape[1]
    f32 = rows.dtype == torch.float32
    # the pieces' rows in position order (gathered through the block table)
    p = torch.arange(lo, lo + nc * nk, device=q.device)
    ridx = table_row.long()[p // bs] * bs + p % bs
    kv = rows.view(-1, rows.shape[-1]).index_select(0, ridx)
    kk = kv[:, :G * d].reshape(nc, nk, G, d).permute(0, 2, 3, 1).reshape(nc * G, d, nk)
    vv = kv[:, G * d:].reshape(nc, nk, G, dv).permute(0, 2, 1, 3).reshape(nc * G, nk, dv)
    n = nc * nq
    qq = q[t0:t0 + n].view(nc, nq, G, rep, d).permute(0, 2, 1, 3, 4).reshape(nc * G, nq * rep, d)
    if f32:
        sc = torch.bmm(qq, kk)
        w = _ops().ma_chunk_softmax(sc.view(nc * G * nq * rep, nk), nq, G, rep, scale, sink, True, softcap, True, 0, 0, 0, 0, 0)
        if talk is not None:
            w = _ops().ma_talk_mix(w, talk, nq, G, rep, True)
        o = torch.bmm(w.view(nc * G, nq * rep, nk), vv)
    else:
        # f32 queries against 16-bit keys, f32 weights against 16-bit values: hi + lo halves side by side along the
        # summed axis, the keys / values twice, so each product is one launch with f32 accumulation
        qh = qq.to(rows.dtype)
        q2 = torch.cat([qh, (qq - qh.float()).to(rows.dtype)], -1)
        sc = torch.bmm(q2, torch.cat([kk, kk], 1), out_dtype=torch.float32)
        if talk is None:
            w = _ops().ma_chunk_softmax(sc.view(nc * G * nq * rep, nk), nq, G, rep, scale, sink, False, softcap, False, 0, 0, 0, 0, 0)
        else:       # normalised f32 weights in place, then the heads' weights mixed and split into hi + lo halves
            w = _ops().ma_chunk_softmax(sc.view(nc * G * nq * rep, nk), nq, G, rep, scale, sink, False, softcap, True, 0, 0, 0, 0, 0)
            w = _ops().ma_talk_mix(w, talk, nq, G, rep, False)
        o = torch.bmm(w.view(nc * G, nq * rep, 2 * nk), torch.cat([vv, vv], 1), out_dtype=torch.float32)
    o = o.view(nc, G, nq, rep, dv).permute(0, 2, 1, 3, 4).reshape(n, H * dv)
    out[t0:t0 + n] = o.to(out.dtype)


def _window_gemm(q, rows, table_row, G, dv, scale, sink, t0, n, L, size, keep, out, softcap=0.0, talk=None):
    """A portion of ``n`` queries (the step's tokens from ``t0`` on, the last at position L - 1) of one sequence under
    a sliding window, block by block of WINDOW_Q_BLOCK queries: a block sees the kept first tokens and the keys from
    its first query's window start to its last query, as two batched library products per block with the masked
    softmax between them."""
    _, H, d = q.shape
    rep = H // G
    bs = rows.shape[1]
    f32 = rows.dtype == torch.float32
    flat = rows.view(-1, rows.shape[-1])
    p0 = L - n
    for b0 in range(0, n, WINDOW_Q_BLOCK):
        nq = min(WINDOW_Q_BLOCK, n - b0)
        q0 = p0 + b0
        k0 = max(0, q0 - size + 1)
        nkeep = min(keep, k0)
        nr = q0 + nq - k0
        nk = -(-(nkeep + nr) // 8) * 8                               # padded columns: masked (ahead of every query)
        p = torch.cat([torch.arange(nkeep, device=q.device), torch.arange(k0, k0 + nr, device=q.device),
                       torch.full((nk - nkeep - nr,), k0 + nr - 1, device=q.device)])
        ridx = table_row.long()[p // bs] * bs + p % bs
        kv = flat.index_select(0, ridx)
        kk = kv[:, :G * d].reshape(nk, G, d).permute(1, 2, 0)
        vv = kv[:, G * d:].reshape(nk, G, dv).permute(1, 0, 2)
        qq = q[t0 + b0:t0 + b0 + nq].view(nq, G, rep, d).permute(1, 0, 2, 3).reshape(G, nq * rep, d)
        args = (nq, G, rep, scale, sink, f32, softcap)
        win = (size, keep, nkeep, q0, k0)
        if f32:
            sc = torch.bmm(qq, kk)
            w = _ops().ma_chunk_softmax(sc.view(G * nq * rep, nk), *args, True, *win)
            if talk is not None:
                w = _ops().ma_talk_mix(w, talk, nq, G, rep, True)
            o = torch.bmm(w.view(G, nq * rep, nk), vv)
        else:
            qh = qq.to(rows.dtype)
            q2 = torch.cat([qh, (qq - qh.float()).to(rows.dtype)], -1)
            sc = torch.bmm(q2, torch.cat([kk, kk], 1), out_dtype=torch.float32)
            w = _ops().ma_chunk_softmax(sc.view(G * nq * rep, nk), *args, talk is not None, *win)
            if talk is not None:
                w = _ops().ma_talk_mix(w, talk, nq, G, rep, False)
            o = torch.bmm(w.view(G, nq * rep, 2 * nk), torch.cat([vv, vv], 1), out_dtype=torch.float32)
        o = o.view(G, nq, rep, dv).permute(1, 0, 2, 3).reshape(nq, H * dv)
        out[t0 + b0:t0 + b0 + nq] = o.to(out.dtype)


def _masked_attention_gpu(q, rows, G, dv, block_tables, seq_of, pos, scale, mask, size, sink, q_lens, ctx_lens,
                          out_dtype, softcap=0.0, keep_first=0, talk=None):
    T, H, d = q.shape
    f32 = out_dtype == torch.float32
    q = q.contiguous()
    code = MASKS[mask]
    big = mask == "chunk" and GEMM_MIN_CHUNK > 0 and max(q_lens) >= GEMM_MIN_CHUNK and _bmm_f32_ok(rows.dtype) and \
        (talk is None or H <= 256)
    if mask == "window" and WINDOW_GEMM_MIN > 0 and max(q_lens) >= WINDOW_GEMM_MIN and _bmm_f32_ok(rows.dtype) and \
            (talk is None or H <= 256):
        # long portions run block by block as library products, the others (decoded tokens, short portions) together
        # through the one-pass kernel
        out = torch.empty(T, H * dv, dtype=out_dtype, device=q.device)
        rest, rest_ctx, t0 = [], 1, 0
        for b, (n, L) in enumerate(zip(q_lens, ctx_lens)):
            if n >= WINDOW_GEMM_MIN:
                _window_gemm(q, rows, block_tables[b], G, dv, scale, sink, t0, n, L, size, keep_first, out, softcap, talk)
            elif n:
                rest.append(torch.arange(t0, t0 + n, device=q.device))
                rest_ctx = max(rest_ctx, L)
            t0 += n
        if rest:
            idx = torch.cat(rest)
            out[idx] = _ops().ma_masked_attention(q[idx].contiguous(), rows, G, dv, block_tables,
                                                  seq_of[idx].contiguous(), pos[idx].contiguous(), scale, code, size, sink,
                                                  rest_ctx, f32, softcap, keep_first, talk)
        return out
    if not big:
        return _ops().ma_masked_attention(q, rows, G, dv, block_tables, seq_of, pos, scale, code, size, sink,
                                          max(ctx_lens), f32, softcap, keep_first, talk)
    out = torch.empty(T, H * dv, dtype=out_dtype, device=q.device)
    rest, rest_ctx, t0 = [], 1, 0
    for b, (n, L) in enumerate(zip(q_lens, ctx_lens)):
        # the portion [p0, L) falls into: the rest of the chunk it starts in, whole chunks, the start of a last chunk;
        # each is block-diagonal, and those of at least GEMM_MIN_CHUNK queries run as products
        p0, t = L - n, t0
        while p0 < L:
            c0 = p0 - p0 % size                                      # first position of p0's chunk
            if p0 == c0 and L - p0 >= size:
                nc = (L - p0) // size
                nq = nk = size
            else:
                nc, nq = 1, min(L, c0 + size) - p0
                nk = p0 - c0 + nq
            if nq >= GEMM_MIN_CHUNK:
                _pieces_gemm(q, rows, block_tables[b], G, dv, scale, sink, t, c0, nc, nk, nq, out, softcap, talk)
            else:
                rest.append(torch.arange(t, t + nc * nq, device=q.device))
                rest_ctx = max(rest_ctx, L)
            p0 += nc * nq
            t += nc * nq
        t0 += n
    if rest:
        idx = torch.cat(rest)
        out[idx] = _ops().ma_masked_attention(q[idx].contiguous(), rows, G, dv, block_tables, seq_of[idx].contiguous(),
                                              pos[idx].contiguous(), scale, code, size, sink, rest_ctx, f32, softcap,
                                              keep_first, talk)
    return out


_bmm_out_f32: Optional[bool] = None


def _bmm_f32_ok(dtype) -> bool:
    """batched 16-bit products with f32 results (torch.bmm out_dtype)"""
    global _bmm_out_f32
    if dtype == torch.float32:
        return True
    if _bmm_out_f32 is None:
        try:
            a = torch.zeros(1, 16, 16, dtype=dtype, device="cuda")
            torch.bmm(a, a, out_dtype=torch.float32)
            _bmm_out_f32 = True
        except (TypeError, RuntimeError):
            _bmm_out_f32 = False
    return _bmm_out_f32


def sigmoid_gate(o: torch.Tensor, gate_pre: torch.Tensor) -> torch.Tensor:
    """``o * sigmoid(gate_pre)`` element by element (f32 math), o's dtype;
    ``gate_pre`` may be a strided view of a projection's result."""
    if native(o):
        return _ops().ma_sigmoid_gate(o.contiguous(), gate_pre)
    return (o.float() * torch.sigmoid(gate_pre.float())).to(o.dtype)
