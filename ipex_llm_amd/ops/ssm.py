"""Ops of the state-space mixer of the hybrid decoders (models/hybrid.py
``SSMMixer``): a short causal convolution with bias and SiLU whose last inputs
are per-sequence state, the selective scan over f32 state slots, and the gated
group norm behind it.

Every op takes a *ragged step* like ``ops/seqmix.py``.  GPU tensors run the
HIP kernels of ``csrc/hip/ssm.hip``; CPU tensors run the torch forms below,
which are also what the kernels are tested against.

Precision (both paths): the step size with its softplus, the decay and its
exponentials, the state, the scan's sums, the gate product and the group norm
are f32 whatever the activation dtype is; the convolution reads activations
and accumulates in f32, and its result stays f32 for the scan.
"""
from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn.functional as F

from .seqmix import native

__all__ = ["conv_silu", "selective_scan", "gated_group_norm", "SCAN_MAX_STATE"]

SCAN_MAX_STATE = 1024          # largest state size N the scan kernel holds (16 waves x 64 values)


def _ops():
    return torch.ops.ipex_llm_amd


def conv_silu(u: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor], state: torch.Tensor, cu: torch.Tensor,
              seq_of: torch.Tensor, state_slots: torch.Tensor, pos: torch.Tensor, q_lens: List[int],
              act: bool = True) -> torch.Tensor:
    """Causal per-channel convolution over time with bias (``b`` None: none), then SiLU (``act`` False: none).

    ``u`` [T, C] (a strided view of a projection's result is allowed), ``w``
    f32 [C, taps] whose last column weighs the current token, ``b`` f32 [C]:

        out_t = silu(b + sum_j w[:, j] * u_(t - taps + 1 + j))       f32 [T, C]

    with zeros before a sequence's start.  ``state`` f32 [slots, taps - 1, C]
    holds, per sequence, the inputs of its last ``taps - 1`` positions (oldest
    first); a portion that does not start at position 0 reads what lies before
    it from there, and every portion leaves its last inputs there."""
    taps = w.shape[1]
    if native(u):
        single = len(q_lens) == u.shape[0] and all(n == 1 for n in q_lens)
        return _ops().ssm_conv_silu(u, w, b, state, cu, seq_of, state_slots, pos, single, act)
    T, C = u.shape
    out = torch.empty(T, C, dtype=torch.float32, device=u.device)
    uf = u.float()
    slots, first = state_slots.tolist(), pos.tolist()
    t0 = 0
    for s, n in enumerate(q_lens):
        if n == 0:
            continue
        p0 = first[t0]
        hist = state[slots[s]].clone()                              # positions p0 - taps + 1 .. p0 - 1
        if p0 < taps - 1:
            hist[:taps - 1 - p0] = 0.0
        ext = torch.cat([hist, uf[t0:t0 + n]], 0)
        acc = b.float()[None].repeat(n, 1) if b is not None else torch.zeros(n, C, device=u.device)
        for j in range(taps):
            acc += w[:, j].float()[None] * ext[j:j + n]
        out[t0:t0 + n] = F.silu(acc) if act else acc
        state[slots[s]] = ext[n:]
        t0 += n
    return out


def selective_scan(x: torch.Tensor, Bm: torch.Tensor, Cm: torch.Tensor, dt_pre: torch.Tensor, dt_bias: torch.Tensor,
                   a_log: torch.Tensor, d_skip: torch.Tensor, state: torch.Tensor, cu: torch.Tensor,
                   state_slots: torch.Tensor, pos: torch.Tensor, q_lens: List[int]) -> torch.Tensor:
    """The state-space recurrence, token by token, per sequence and head.

    ``x`` f32 [T, H, P], ``Bm`` / ``Cm`` f32 [T, G, N] (views of one row-major
    buffer are allowed; head h reads group h // (H / G)), ``dt_pre`` [T, H] in
    the activation dtype (strided view allowed), ``dt_bias`` / ``a_log`` /
    ``d_skip`` f32 [H].  ``state`` f32 [slots, H, N, P] is read at
    ``state_slots[s]`` (a sequence whose first new token is at position 0 starts
    from zero instead) and written back after the last token.  With
    dt = softplus(dt_pre + dt_bias) (no clamp) and a = exp(-exp(a_log) dt):

        S' = a S + dt B x^T          [N, P]
        y  = S'^T C + d_skip x       [P]

    Returns y f32 [T, H, P]."""
    T, H, P = x.shape
    G, N = Bm.shape[1], Bm.shape[2]
    if native(x):
        if N > SCAN_MAX_STATE:
            raise ValueError(f"selective_scan: state size {N} is above the kernel's {SCAN_MAX_STATE}")
        return _ops().ssm_selective_scan(x, Bm, Cm, dt_pre, dt_bias, a_log, d_skip, state, cu, state_slots, pos)
    out = torch.empty(T, H, P, dtype=torch.float32, device=x.device)
    dt = F.softplus(dt_pre.float() + dt_bias.float(), threshold=30.0)
    a = torch.exp(-torch.exp(a_log.float()) * dt)                   # [T, H]
    rep = H // G
    slots, first = state_slots.tolist(), pos.tolist()
    t0 = 0
    for s, n in enumerate(q_lens):
        if n == 0:
            continue
        S = torch.zeros(H, N, P, device=x.device) if first[t0] == 0 else state[slots[s]].clone()
        for t in range(t0, t0 + n):
            Bh = Bm[t].float().repeat_interleave(rep, 0)            # [H, N]
            Ch = Cm[t].float().repeat_interleave(rep, 0)
            S = a[t][:, None, None] * S + (dt[t][:, None] * Bh)[:, :, None] * x[t].float()[:, None, :]
            out[t] = torch.einsum("hnp,hn->hp", S, Ch) + d_skip.float()[:, None] * x[t].float()
        state[slots[s]] = S
        t0 += n
    return out


def gated_group_norm(y: torch.Tensor, z: torch.Tensor, w: torch.Tensor, groups: int, eps: float,
                     out_dtype: torch.dtype) -> torch.Tensor:
    """``y`` f32 [T, C] times ``silu(z)`` (``z`` [T, C] in the activation dtype,
    strided view allowed), then every one of ``groups`` equal parts of a row is
    divided by its own root mean square, then ``* w`` ([C]).  The gate comes
    before the norm.  Returns [T, C] in ``out_dtype``."""
    T, C = y.shape
    if C % groups:
        raise ValueError("gated_group_norm: the row must split into equal groups")
    if native(y):
        return _ops().ssm_gated_group_norm(y.contiguous(), z, w, groups, eps, out_dtype == torch.float32)
    g = (y * F.silu(z.float())).view(T, groups, C // groups)
    g = g * torch.rsqrt((g * g).mean(-1, keepdim=True) + eps)
    return (g.reshape(T, C) * w.float()).to(out_dtype)
