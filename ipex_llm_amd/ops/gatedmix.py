"""Ops of the gated recurrent mixers and the two-norm parallel blocks of the
hybrid decoders (models/hybrid.py ``TwoNormParallelLayer``, ``MinGRU``,
``GatedLinearAttention``, ``SideBySide``): a pair of LayerNorms with the token
shift of the mixer's input, a short causal convolution whose last inputs are
per-sequence state, the minGRU recurrence, the gated-linear-attention
recurrence with a decay per key channel, the per-head RMS norm with a SiLU
gate, the mean of two RMS-normed mixer results and the tanh cap of the logits.

Every op takes a *ragged step* like ``ops/seqmix.py``.  GPU tensors run the
HIP kernels of ``csrc/hip/gatedmix.hip``; CPU tensors run the torch forms
below, which are also what the kernels are tested against.

Precision (both paths): norms, the shift, gates, decays with their logarithms
and exponentials, candidates, states and the recurrences' sums are f32
whatever the activation dtype is; the convolution accumulates in f32.
"""
from __future__ import annotations

import os
from typing import List, Optional, Tuple

import torch
import torch.nn.functional as F

from .seqmix import native
from .ssm import conv_silu

__all__ = ["layer_norm_pair_shift", "causal_conv", "mingru_scan", "gla_scan", "head_rms_silu", "rms_pair_mean",
           "softcap_", "GLA_MAX_DIM"]

GLA_MAX_DIM = 1024             # largest key size per head the scan kernel holds (16 waves x 64 state rows)


def _ops():
    return torch.ops.ipex_llm_amd


def _single(q_lens: List[int], T: int) -> bool:
    return len(q_lens) == T and all(n == 1 for n in q_lens)


def layer_norm_pair_shift(x: torch.Tensor, w1: torch.Tensor, w2: Optional[torch.Tensor], mu: Optional[torch.Tensor],
                          eps: float, state: Optional[torch.Tensor], cu: torch.Tensor, seq_of: torch.Tensor,
                          state_slots: torch.Tensor, pos: torch.Tensor, q_lens: List[int],
                          act_dtype: torch.dtype) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Two bias-free LayerNorms of the same f32 rows ``x`` [T, W] (variance =
    mean squared deviation) and the token shift of the first:

        n1 = LN(x) w1,   h1_t = n1_t + (n1_(t-1) - n1_t) mu,   h2 = LN(x) w2

    ``n1_(t-1)`` is the previous token's ``n1`` (zeros at position 0): inside a
    portion the row before, at its start what ``state`` f32 [slots, W] holds for
    the sequence; every portion leaves its last ``n1`` there.  ``mu`` f32 [W] or
    None (no shift, no state); ``w2`` None: one norm.  Returns ``h1`` and ``h2``
    (or None) in ``act_dtype``."""
    if native(x):
        h1, h2 = _ops().gm_layer_norm_pair_shift(x.contiguous(), w1, w2, mu, eps, state, cu, seq_of, state_slots, pos,
                                                 _single(q_lens, x.shape[0]), act_dtype == torch.float32)
        return h1, (h2 if w2 is not None else None)
    d = x - x.mean(-1, keepdim=True)
    xn = d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps)
    n1 = xn * w1.float()
    h2 = (xn * w2.float()).to(act_dtype) if w2 is not None else None
    if mu is None:
        return n1.to(act_dtype), h2
    prev = torch.empty_like(n1)
    slots, first = state_slots.tolist(), pos.tolist()
    t0 = 0
    for b, n in enumerate(q_lens):
        if n == 0:
            continue
        prev[t0] = state[slots[b]] if first[t0] > 0 else 0.0
        prev[t0 + 1:t0 + n] = n1[t0:t0 + n - 1]
        state[slots[b]] = n1[t0 + n - 1]
        t0 += n
    return (n1 + (prev - n1) * mu.float()).to(act_dtype), h2


def causal_conv(u: torch.Tensor, w: torch.Tensor, state: torch.Tensor, cu: torch.Tensor, seq_of: torch.Tensor,
                state_slots: torch.Tensor, pos: torch.Tensor, q_lens: List[int]) -> torch.Tensor:
    """Causal per-channel convolution over time, no bias, no activation: the
    convolution of ``ops/ssm.py`` (same kernel, same state layout) without its
    bias and SiLU.  ``u`` [T, C], ``w`` f32 [C, taps], ``state`` f32
    [slots, taps - 1, C]:

        out_t = sum_j w[:, j] * u_(t - taps + 1 + j)                 f32 [T, C]"""
    return conv_silu(u, w, None, state, cu, seq_of, state_slots, pos, q_lens, act=False)


def mingru_scan(y: torch.Tensor, width: int, state: torch.Tensor, cu: torch.Tensor, state_slots: torch.Tensor,
                pos: torch.Tensor, q_lens: List[int]) -> torch.Tensor:
    """The minGRU recurrence with its output gate, element by element.

    ``y`` [T, 3 width] = ``[z_pre | u | g_pre]`` (a projection's result, biases
    included).  With z = sigmoid(z_pre) and the candidate c = u + 1/2 where
    u >= 0, sigmoid(u) where u < 0:

        S_t = (1 - z_t) S_(t-1) + z_t c_t,        out_t = S_t silu(g_pre_t)

    ``state`` f32 [slots, width] is read at ``state_slots[s]`` (a sequence whose
    first new token is at position 0 starts from zero instead) and written back
    after the last token.  Returns [T, width] in y's dtype."""
    T = y.shape[0]
    if native(y):
        return _ops().gm_mingru_scan(y, width, state, cu, state_slots, pos, max(q_lens))
    yf = y.float()
    z = torch.sigmoid(yf[:, :width])
    u = yf[:, width:2 * width]
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = F.silu(yf[:, 2 * width:])
    out = torch.empty(T, width, dtype=torch.float32, device=y.device)
    slots, first = state_slots.tolist(), pos.tolist()
    t0 = 0
    for s, n in enumerate(q_lens):
        if n == 0:
            continue
        S = torch.zeros(width, device=y.device) if first[t0] == 0 else state[slots[s]].clone()
        for t in range(t0, t0 + n):
            S = (1.0 - z[t]) * S + z[t] * c[t]
            out[t] = S * g[t]
        state[slots[s]] = S
        t0 += n
    return out.to(y.dtype)


def gla_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a_pre: torch.Tensor, tau: float, q_scale: float,
             state: torch.Tensor, cu: torch.Tensor, state_slots: torch.Tensor, pos: torch.Tensor,
             q_lens: List[int]) -> torch.Tensor:
    """Gated linear attention, token by token, per sequence and head.

    ``q`` / ``k`` / ``a_pre`` [T, H, d], ``v`` [T, H, dv] in the activation dtype
    (strided views allowed).  With the decay per key channel
    alpha = sigmoid(a_pre)^(1 / tau) = exp(log_sigmoid(a_pre) / tau):

        S' = diag(alpha) S + k v^T        [d, dv]
        o  = S'^T (q q_scale)             [dv]

    ``state`` f32 [slots, H, d, dv] is read at ``state_slots[s]`` (a sequence
    whose first new token is at position 0 starts from zero instead) and written
    back after the last token.  Returns o f32 [T, H, dv]."""
    T, H, d = q.shape
    dv = v.shape[2]
    if native(q):
        if d > GLA_MAX_DIM:
            raise ValueError(f"gla_scan: key size {d} is above the kernel's {GLA_MAX_DIM}")
        if GLA_PIECE_MIN > 0 and max(q_lens) >= GLA_PIECE_MIN:
            return _gla_scan_pieces(q, k, v, a_pre, tau, q_scale, state, state_slots, pos, q_lens)
        return _ops().gm_gla_scan(q, k, v, a_pre, tau, q_scale, state, cu, state_slots, pos)
    out = torch.empty(T, H, dv, dtype=torch.float32, device=q.device)
    alpha = torch.exp(F.logsigmoid(a_pre.float()) / tau)
    qf, kf, vf = q.float() * q_scale, k.float(), v.float()
    slots, first = state_slots.tolist(), pos.tolist()
    t0 = 0
    for s, n in enumerate(q_lens):
        if n == 0:
            continue
        S = torch.zeros(H, d, dv, device=q.device) if first[t0] == 0 else state[slots[s]].clone()
        for t in range(t0, t0 + n):
            S = alpha[t][:, :, None] * S + kf[t][:, :, None] * vf[t][:, None, :]
            out[t] = torch.einsum("hdp,hd->hp", S, qf[t])
        state[slots[s]] = S
        t0 += n
    return out


# The scan is sequential in time.  A portion of at least GLA_PIECE_MIN tokens is cut into up to GLA_PIECES pieces
# that run side by side, twice: the recurrence is linear in the state, S_end = diag(P) S_start + Z with P the product
# of the piece's decays and Z its result from a zero state, so a first pass gives every piece's Z, a short chain
# over the pieces gives every piece's true start state, and a second pass from those writes the outputs.
GLA_PIECE_MIN = int(os.environ.get("ILLM_GLA_PIECE_MIN", "2048"))
GLA_PIECES = int(os.environ.get("ILLM_GLA_PIECES", "16"))


def _gla_scan_pieces(q, k, v, a_pre, tau, q_scale, state, state_slots, pos, q_lens):
    T, H, d = q.shape
    dev = q.device
    cuts, first, owner = [0], [], []                 # piece borders (token indices); first piece of / pieces per sequence
    t0 = 0
    for s, n in enumerate(q_lens):
        if n == 0:
            continue
        per = max(-(-n // GLA_PIECES), 64) if n >= GLA_PIECE_MIN else n
        first.append(len(cuts) - 1)
        for lo in range(0, n, per):
            cuts.append(t0 + min(n, lo + per))
        owner.append((s, len(cuts) - 1 - first[-1]))
        t0 += n
    NP = len(cuts) - 1
    cu_p = torch.tensor(cuts, dtype=torch.int32, device=dev)
    slots_p = torch.arange(NP, dtype=torch.int32, device=dev)
    first_t = torch.tensor(first, dtype=torch.long, device=dev)
    seqs = torch.tensor([s for s, _ in owner], dtype=torch.long, device=dev)
    real = state_slots.long().index_select(0, seqs)
    later = torch.tensor([cuts[f + j] for f, (_, m) in zip(first, owner) for j in range(1, m)], dtype=torch.long, device=dev)
    # every piece's decay product (sums of log decays in f64)
    P = _ops().gm_gla_piece_decay(a_pre, cu_p, tau)                     # [NP, H, d]
    seqs_p = torch.tensor([[f, m] for f, (_, m) in zip(first, owner)], dtype=torch.int32, device=dev)
    start = state.index_select(0, real)
    Z = torch.empty(NP + 1, *state.shape[1:], dtype=torch.float32, device=dev)
    Z.index_copy_(0, first_t, start)
    pos1 = pos.clone()
    pos1.index_fill_(0, later, 0)                                       # later pieces start from zero in the first pass
    _ops().gm_gla_scan(q, k, v, a_pre, tau, q_scale, Z, cu_p, slots_p, pos1)
    Sin = torch.empty_like(Z)
    Sin.index_copy_(0, first_t, start)
    _ops().gm_gla_chain_(Z, Sin, P, seqs_p)                             # the chain of start states, piece after piece
    out = _ops().gm_gla_scan(q, k, v, a_pre, tau, q_scale, Sin, cu_p, slots_p, pos)
    last = torch.tensor([f + m - 1 for f, (_, m) in zip(first, owner)], dtype=torch.long, device=dev)
    state.index_copy_(0, real, Sin.index_select(0, last))
    return out


def head_rms_silu(o: torch.Tensor, w: torch.Tensor, gate_pre: torch.Tensor, eps: float,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """Every head of ``o`` f32 [T, H, dv] divided by its root mean square, times
    ``w`` ([dv], shared by the heads), times ``silu(gate_pre)`` (``gate_pre``
    [T, H dv], strided view allowed).  Returns [T, H dv] in ``out_dtype``."""
    T, H, dv = o.shape
    if native(o):
        return _ops().gm_head_rms_silu(o.contiguous(), w, gate_pre, eps, out_dtype == torch.float32)
    n = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * w.float()
    return (n.reshape(T, H * dv) * F.silu(gate_pre.float())).to(out_dtype)


def rms_pair_mean(a: torch.Tensor, b: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, eps: float,
                  out_dtype: torch.dtype) -> torch.Tensor:
    """``(rms_norm(a) wa + rms_norm(b) wb) / 2`` row by row (f32 math) for two
    mixers' results [T, W]; returns [T, W] in ``out_dtype``."""
    if native(a):
        return _ops().gm_rms_pair_mean(a.contiguous(), b.contiguous(), wa, wb, eps, out_dtype == torch.float32)
    af, bf = a.float(), b.float()
    ya = af * torch.rsqrt((af * af).mean(-1, keepdim=True) + eps) * wa.float()
    yb = bf * torch.rsqrt((bf * bf).mean(-1, keepdim=True) + eps) * wb.float()
    return (0.5 * (ya + yb)).to(out_dtype)


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """``cap tanh(x / cap)`` in place on f32 values."""
    if native(x):
        _ops().gm_softcap_(x, cap)
        return x
    return x.copy_(cap * torch.tanh(x / cap))
