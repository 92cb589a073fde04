"""Decoders of two-norm parallel blocks (Zoguzen layout): the framework --
checkpoint reader, paged rows and state slots, scheduler, ragged engine steps,
kernels -- against the plain float64 forms of tests/dualnorm_oracle.py.

Every test runs on the CPU (torch forms of ops/gatedmix.py, ops/maskattn.py,
...) and, marked ``gpu``, on the HIP kernels.  Models are small random ones
made here.
"""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from . import dualnorm_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVS = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
F64 = torch.float64
TOL = {torch.float32: 2e-4, torch.bfloat16: 0.12}


@pytest.fixture(params=DEVS)
def dev(request):
    if request.param == "cuda":
        if not torch.cuda.is_available():
            pytest.skip("no GPU")
        import ipex_llm_amd.ops as ops
        ops.require_seqmix()
    return torch.device(request.param)


def std_cfg():
    """all three mixers, a layer that borrows keys and values, layers with and without experts; a window and chunks
    shorter than a page and ones that straddle pages"""
    sc = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
    return O.config([O.attn_layer(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, taps=3, mlp=O.moe(5, 2, 12)),
                     O.gru_layer(width=24, mlp=O.moe(3, 1, 16)),
                     O.attn_layer(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, taps=4, kv_from=0),
                     O.pair_layer(heads=4, kv_heads=2, dim=12, vdim=10, window=9, keep=2, taps=2, dims=8, scaling=sc,
                                  rheads=3, rdim=6, rvdim=10, tau=4.0, mlp=O.moe(4, 3, 8)),
                     O.attn_layer(heads=2, kv_heads=1, dim=16, vdim=24, chunk=70, taps=2, scale=0.25, softcap=3.0),
                     O.pair_layer(heads=2, kv_heads=2, dim=8, vdim=16, window=66, keep=5, taps=3, dims=4, rheads=2,
                                  rdim=20, rvdim=70, tau=9.0),
                     O.gru_layer(width=70)], width=40)


def build(cfg, W, dev, dtype=torch.float32):
    from ipex_llm_amd.models import zoguzen as Z
    return Z.build(Z.spec_from_config(cfg, ranks(cfg, W)), W, dtype, dev)


def ranks(cfg, W):
    return {i: W[f"l{i}.mix.right.a1"].shape[0] for i, L in enumerate(cfg["layers"]) if L["type"] == "parallel"}


def engine(cfg, W, dev, dtype=torch.float32, max_batch=4, num_blocks=16, prefill=1 << 30, graph=False):
    from ipex_llm_amd.serving.engine import LLMEngine
    return LLMEngine(build(cfg, W, dev, dtype), max_batch=max_batch, block_size=64, num_blocks=num_blocks,
                     max_model_len=num_blocks * 64, max_prefill_tokens=prefill, use_graph=graph,
                     enable_prefix_caching=False)


def replay(eng, prompts, schedule, keep_open=()):
    """schedule: steps of [(name, count)]; every token's logits are asked for.
    Returns name -> [T, V] (f64, on the CPU) of what was run."""
    at, rid, got = {}, {}, {}
    for step in schedule:
        entries, names = [], []
        for name, n in step:
            lo = at.get(name, 0)
            if name not in rid:
                rid[name] = eng.open_stream()
            entries.append((rid[name], prompts[name][lo:lo + n], list(range(n))))
            names.append((name, n))
            at[name] = lo + n
        lg = eng.feed(entries).double().cpu()
        o = 0
        for name, n in names:
            got.setdefault(name, []).append(lg[o:o + n])
            o += n
        for name, _ in names:
            if at[name] == len(prompts[name]) and name not in keep_open:
                eng.close_stream(rid.pop(name))
    return {k: torch.cat(v) for k, v in got.items()}


def rel_err(got, want):
    """largest row error: rms over the vocabulary of the centred difference, over the logits' spread"""
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / want.std()).max())


def ragged(lens, starts, dev, slot0=1):
    """cu, seq_of, state slots, positions of a step whose sequence s brings lens[s] tokens from position starts[s]"""
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32, device=dev)
    seq_of = torch.cat([torch.full((n,), s, dtype=torch.int32) for s, n in enumerate(lens)]).to(dev)
    pos = torch.cat([torch.arange(a, a + n) for a, n in zip(starts, lens)]).to(dev)
    slots = torch.arange(slot0, slot0 + len(lens), dtype=torch.int32, device=dev)
    return cu, seq_of, slots, pos


def in_portions(f, seqs, cuts, dev):
    """run ``f(rows of the step, lens, cu, seq_of, slots, pos)`` over ``seqs`` (a list of [n_s, ...] inputs) cut into
    the steps ``cuts`` (per step the tokens every sequence brings, 0: it sits the step out); returns per sequence
    the concatenated results"""
    at = [0] * len(seqs)
    outs = [[] for _ in seqs]
    for step in cuts:
        who = [s for s, n in enumerate(step) if n]
        lens = [step[s] for s in who]
        cu, seq_of, _, pos = ragged(lens, [at[s] for s in who], dev)
        slots = torch.tensor([s + 1 for s in who], dtype=torch.int32, device=dev)
        rows = torch.cat([seqs[s][at[s]:at[s] + step[s]] for s in who]).to(dev)
        res = f(rows, lens, cu, seq_of, slots, pos)
        o = 0
        for s, n in zip(who, lens):
            outs[s].append(res[o:o + n].double().cpu())
            o += n
            at[s] += n
    return [torch.cat(o) for o in outs]


CUTS = [[5, 1, 0], [1, 1, 70], [2, 60, 1], [64, 2, 1], [1, 0, 3]]     # three sequences, 73 / 64 / 75 tokens


# ------------------------------------------------------------------ mechanisms alone (ops)
@pytest.mark.parametrize("act", [torch.float32, torch.bfloat16])
def test_norm_pair_and_shift(dev, act):
    """both norms of a row, the first shifted towards the previous token's -- across portions through the slots"""
    from ipex_llm_amd.ops import gatedmix as GM
    g = torch.Generator().manual_seed(0)
    for Wd in (40, 4160):
        seqs = [torch.randn(n, Wd, generator=g) * 2 + 0.7 for n in (73, 64, 75)]
        w1 = (1 + 0.3 * torch.randn(Wd, generator=g)).to(act)
        w2 = (1 + 0.3 * torch.randn(Wd, generator=g)).to(act)
        mu = torch.rand(Wd, generator=g)
        state = torch.randn(5, Wd, generator=g).to(dev)               # slots start dirty
        tol = 2e-5 if act == torch.float32 else 6e-2

        def f(rows, lens, cu, seq_of, slots, pos):
            h1, h2 = GM.layer_norm_pair_shift(rows, w1.to(dev), w2.to(dev), mu.to(dev), 1e-5, state, cu, seq_of, slots,
                                              pos, lens, act)
            assert h1.dtype == act and h2.dtype == act
            return torch.cat([h1, h2], -1)

        got = in_portions(f, seqs, CUTS, dev)
        for x, o in zip(seqs, got):
            n1 = O.layer_norm(x.double(), w1.double(), 1e-5)
            assert (o[:, :Wd] - O.token_shift(n1, mu.double())).abs().max() < tol
            assert (o[:, Wd:] - O.layer_norm(x.double(), w2.double(), 1e-5)).abs().max() < tol
        x = seqs[0][:6].to(dev)                                       # one norm, no shift: no state touched
        cu, seq_of, slots, pos = ragged([6], [0], dev)
        h1, h2 = GM.layer_norm_pair_shift(x, w1.to(dev), None, None, 1e-5, None, cu, seq_of, slots, pos, [6], act)
        assert h2 is None
        assert (h1.double().cpu() - O.layer_norm(seqs[0][:6].double(), w1.double(), 1e-5)).abs().max() < tol


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_convolution_without_bias(dev, taps):
    from ipex_llm_amd.ops import gatedmix as GM
    g = torch.Generator().manual_seed(taps)
    for C, act in ((37, torch.float32), (40, torch.bfloat16)):
        seqs = [torch.randn(n, C + 6, generator=g).to(act) for n in (73, 64, 75)]
        w = torch.randn(C, taps, generator=g)
        state = torch.randn(5, taps - 1, C, generator=g).to(dev)

        def f(rows, lens, cu, seq_of, slots, pos):
            return GM.causal_conv(rows[:, 3:3 + C], w.to(dev), state, cu, seq_of, slots, pos, lens)

        for x, o in zip(seqs, in_portions(f, seqs, CUTS, dev)):
            assert (o - O.causal_conv(x[:, 3:3 + C].double(), w.double())).abs().max() < 1e-4


@pytest.mark.parametrize("width", [5, 64, 200])
def test_mingru_scan_op(dev, width):
    """the recurrence over portions, batches and a long portion that the kernel cuts into pieces"""
    from ipex_llm_amd.ops import gatedmix as GM
    g = torch.Generator().manual_seed(width)
    for act in (torch.float32, torch.bfloat16):
        seqs = [(torch.randn(n, 3 * width, generator=g) * 2).to(act) for n in (73, 64, 75)]
        state = torch.randn(5, width, generator=g).to(dev)
        cuts = CUTS if act == torch.float32 else [[73, 64, 75]]

        def f(rows, lens, cu, seq_of, slots, pos):
            return GM.mingru_scan(rows, width, state, cu, slots, pos, lens)

        for y, o in zip(seqs, in_portions(f, seqs, cuts, dev)):
            y = y.double()
            z, u = O.sigmoid(y[:, :width]), y[:, width:2 * width]
            c = torch.where(u >= 0, u + 0.5, O.sigmoid(u))
            S, want = torch.zeros(width, dtype=F64), []
            for t in range(y.shape[0]):
                S = (1 - z[t]) * S + z[t] * c[t]
                want.append(S * O.silu(y[t, 2 * width:]))
            want = torch.stack(want)
            assert ((o - want).abs() / (1 + want.abs())).max() < (1e-4 if act == torch.float32 else 2e-2)
    long = (torch.randn(700, 3 * width, generator=g) * 2)
    st = torch.zeros(3, width).to(dev)
    cu, _, slots, pos = ragged([700], [0], dev)
    a = GM.mingru_scan(long.to(dev), width, st, cu, slots, pos, [700]).cpu()
    st2 = torch.zeros(3, width)
    b = GM.mingru_scan(long, width, st2, cu.cpu(), slots.cpu(), pos.cpu(), [700])
    assert (a - b).abs().max() < 1e-4 and (st.cpu() - st2).abs().max() < 1e-4


@pytest.mark.parametrize("H,d,dv", [(3, 6, 10), (2, 48, 64), (1, 70, 70), (2, 130, 8)])
def test_gla_scan_op(dev, H, d, dv):
    """decays per key channel; state carried over portions and batches; sizes that are no multiple of a wave's rows"""
    from ipex_llm_amd.ops import gatedmix as GM
    g = torch.Generator().manual_seed(H + d)
    tau, qs = 3.0, d ** -0.5
    for act in (torch.float32, torch.bfloat16):
        Cn = 3 * H * d + H * dv
        seqs = [torch.randn(n, Cn + 4, generator=g).to(act) for n in (73, 64, 75)]
        state = torch.randn(5, H, d, dv, generator=g).to(dev)

        def split(rows):
            T = rows.shape[0]
            q = rows[:, 2:2 + H * d].view(T, H, d)
            k = rows[:, 2 + H * d:2 + 2 * H * d].view(T, H, d)
            a = (rows[:, 2 + 2 * H * d:2 + 3 * H * d] * 2 + 2).contiguous().view(T, H, d)
            v = rows[:, 2 + 3 * H * d:2 + 3 * H * d + H * dv].view(T, H, dv)
            return q, k, v, a

        def f(rows, lens, cu, seq_of, slots, pos):
            q, k, v, a = split(rows)
            return GM.gla_scan(q, k, v, a, tau, qs, state, cu, slots, pos, lens).reshape(rows.shape[0], -1)

        for x, o in zip(seqs, in_portions(f, seqs, CUTS, dev)):
            q, k, v, a = (t.double() for t in split(x))
            alpha = O.sigmoid(a) ** (1 / tau)
            S, want = torch.zeros(H, d, dv, dtype=F64), []
            for t in range(x.shape[0]):
                S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
                want.append((S * (q[t] * qs)[:, :, None]).sum(1).reshape(-1))
            want = torch.stack(want)
            assert (o - want).abs().max() < 2e-4 * max(1.0, float(want.abs().max()))


def test_gla_long_portions_run_in_pieces(dev, monkeypatch):
    """portions long enough to be cut into pieces that run side by side on the GPU (each piece's start state comes
    from the chain of the pieces before it), beside a short one; a fresh sequence and one that continues"""
    from ipex_llm_amd.ops import gatedmix as GM
    monkeypatch.setattr(GM, "GLA_PIECE_MIN", 1024)
    g = torch.Generator().manual_seed(5)
    H, d, dv, tau = 2, 16, 8, 6.0
    lens, starts = [2100, 5, 1300], [0, 3, 70]
    T = sum(lens)
    q, k = torch.randn(T, H, d, generator=g), torch.randn(T, H, d, generator=g)
    v, a = torch.randn(T, H, dv, generator=g), torch.randn(T, H, d, generator=g) * 2 + 3
    S0 = torch.randn(6, H, d, dv, generator=g)
    state = S0.clone().to(dev)
    cu, _, slots, pos = ragged(lens, starts, dev)
    got = GM.gla_scan(q.to(dev), k.to(dev), v.to(dev), a.to(dev), tau, 0.25, state, cu, slots, pos, lens).double().cpu()
    alpha = O.sigmoid(a.double()) ** (1 / tau)
    t0 = 0
    for s, n in enumerate(lens):
        S = torch.zeros(H, d, dv, dtype=F64) if starts[s] == 0 else S0[s + 1].double()
        for t in range(t0, t0 + n):
            S = alpha[t][:, :, None] * S + k[t].double()[:, :, None] * v[t].double()[:, None, :]
            want = (S * (q[t].double() * 0.25)[:, :, None]).sum(1)
            assert (got[t] - want).abs().max() < 2e-4 * max(1.0, float(want.abs().max())), (s, t - t0)
        assert (state[s + 1].double().cpu() - S).abs().max() < 2e-4 * max(1.0, float(S.abs().max()))
        t0 += n


def test_head_norm_pair_mean_and_cap(dev):
    from ipex_llm_amd.ops import gatedmix as GM
    g = torch.Generator().manual_seed(1)
    for act in (torch.float32, torch.bfloat16):
        tol = 2e-5 if act == torch.float32 else 5e-2
        for H, dv in ((3, 10), (2, 70), (1, 130)):
            o = torch.randn(6, H, dv, generator=g)
            w = (1 + 0.2 * torch.randn(dv, generator=g)).to(act)
            gate = torch.randn(6, H * dv + 9, generator=g).to(act)
            got = GM.head_rms_silu(o.to(dev), w.to(dev), gate.to(dev)[:, 4:4 + H * dv], 1e-5, act)
            want = (O.unit_rms(o.double(), 1e-5) * w.double()).reshape(6, -1) * O.silu(gate[:, 4:4 + H * dv].double())
            assert got.dtype == act and (got.double().cpu() - want).abs().max() < tol
        for Wd in (40, 1030):
            a, b = (torch.randn(5, Wd, generator=g) * 3).to(act), torch.randn(5, Wd, generator=g).to(act)
            wa, wb = (1 + 0.2 * torch.randn(Wd, generator=g)).to(act), (1 + 0.2 * torch.randn(Wd, generator=g)).to(act)
            got = GM.rms_pair_mean(a.to(dev), b.to(dev), wa.to(dev), wb.to(dev), 1e-5, act)
            want = 0.5 * (O.unit_rms(a.double(), 1e-5) * wa.double() + O.unit_rms(b.double(), 1e-5) * wb.double())
            assert got.dtype == act and (got.double().cpu() - want).abs().max() < tol
    x = torch.randn(7, 33, generator=g) * 20
    got = GM.softcap_(x.clone().to(dev), 8.0).cpu()
    assert (got.double() - 8.0 * torch.tanh(x.double() / 8.0)).abs().max() < 1e-5


def test_rotary_wavelength_rule(dev):
    """short waves kept, long waves slowed by the factor, a blend between: all three ranges present"""
    from ipex_llm_amd.ops.seqmix import rope_table
    rot = {"dims": 16, "base": 3000.0, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}
    f = O.rotary_freqs(rot)
    plain = O.rotary_freqs({"dims": 16, "base": 3000.0})
    kinds = {("kept" if a == b else ("slowed" if abs(a - b / 4) < 1e-15 else "blend")) for a, b in zip(f.tolist(), plain.tolist())}
    assert kinds == {"kept", "slowed", "blend"}
    tab = rope_table(50, 16, 3000.0, rot["scaling"]).double()
    ang = torch.arange(50, dtype=F64)[:, None] * f[None]
    assert (tab[..., 0] - ang.cos()).abs().max() < 1e-6 and (tab[..., 1] - ang.sin()).abs().max() < 1e-6


def test_router_and_experts(dev):
    """the largest logits win (lowest index among equals), softmax over the winners only, weights on the results"""
    from ipex_llm_amd.ops import blockmix as BM
    g = torch.Generator().manual_seed(2)
    for E, top, ff, Wd, T in ((5, 2, 12, 40, 9), (11, 3, 88, 64, 150), (3, 3, 8, 24, 4), (70, 1, 8, 16, 33)):
        z = torch.randn(T, E, generator=g) * 3
        z[0, :] = 1.5                                                 # all equal: the first `top` indices
        idx, wts = BM.moe_route(z.to(dev), top, "softmax")
        order = torch.sort(z.double(), dim=-1, descending=True, stable=True)
        assert torch.equal(idx.cpu().long(), order.indices[:, :top])
        assert (wts.double().cpu() - torch.softmax(order.values[:, :top], -1)).abs().max() < 1e-6
        for act in (torch.float32, torch.bfloat16):
            Wt = {"router": torch.zeros(E, Wd, dtype=F64)}
            for e in range(E):
                Wt.update({f"e{e}.gate": torch.randn(ff, Wd, generator=g).to(act).double() * Wd ** -0.5,
                           f"e{e}.up": torch.randn(ff, Wd, generator=g).to(act).double() * Wd ** -0.5,
                           f"e{e}.down": torch.randn(Wd, ff, generator=g).to(act).double() * ff ** -0.5})
                for n in ("gate", "up", "down"):
                    Wt[f"e{e}.{n}"] = Wt[f"e{e}.{n}"].to(act).double()
            h = torch.randn(T, Wd, generator=g).to(act)
            w_gu = torch.stack([torch.cat([Wt[f"e{e}.gate"], Wt[f"e{e}.up"]]) for e in range(E)]).to(act).to(dev)
            w_dn = torch.stack([Wt[f"e{e}.down"] for e in range(E)]).to(act).to(dev)
            got = BM.moe_experts(h.to(dev), idx, wts, w_gu, w_dn, float("inf"), 1.0, 0.0, "output").double().cpu()
            want = torch.zeros(T, Wd, dtype=F64)
            for t in range(T):
                for k in range(top):
                    e = int(idx[t, k])
                    y = O.silu(Wt[f"e{e}.gate"] @ h[t].double()) * (Wt[f"e{e}.up"] @ h[t].double())
                    want[t] += float(wts[t, k]) * (Wt[f"e{e}.down"] @ y)
            assert (got - want).abs().max() < (1e-4 if act == torch.float32 else 6e-2)


def plain_attention(q, k, v, scale, positions, mask, size, keep, cap, sink, talk):
    """q [n, H, d] at ``positions`` over keys k [L, G, d], values v [L, G, dv] (f64): capped scores, a window that
    keeps the first tokens or chunks, a sink of a fixed score, the heads' weights mixed after the softmax"""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[-1], dtype=F64)
    for i, p in enumerate(positions):
        if mask == "chunk":
            js = list(range((p // size) * size, p + 1))
        else:
            js = [j for j in range(p + 1) if p - j < size or j < keep]
        w = torch.zeros(H, len(js), dtype=F64)
        for h in range(H):
            s = (k[js, h // (H // G)] @ q[i, h]) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            e = torch.exp(s)
            w[h] = e / (e.sum() + (0.0 if sink is None else math.exp(sink)))
        if talk is not None:
            w = talk @ w
        for h in range(H):
            out[i, h] = w[h] @ v[js, h // (H // G)]
    return out.reshape(n, -1)


def paged_rows(k, v, dev, dtype, bs=64, spare=3, seed=0):
    """[keys | values] rows of one sequence scattered over shuffled pages -> rows [blocks + 1, bs, .], table [1, nb]"""
    L = k.shape[0]
    nb = (L + bs - 1) // bs
    perm = torch.randperm(nb + spare, generator=torch.Generator().manual_seed(seed))[:nb]
    rows = torch.randn(nb + spare + 1, bs, k[0].numel() + v[0].numel(), generator=torch.Generator().manual_seed(seed + 1)).to(dtype)
    flat = torch.cat([k.reshape(L, -1), v.reshape(L, -1)], -1).to(dtype)
    for i in range(nb):
        seg = flat[i * bs:(i + 1) * bs]
        rows[perm[i], :seg.shape[0]] = seg
    return rows.to(dev), perm.to(torch.int32)[None].to(dev)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,dv,mask,size,keep,cap,sink,talk", [
    (4, 2, 12, 10, "chunk", 7, 0, 5.0, 0.0, True), (4, 4, 80, 48, "chunk", 32, 0, 0.0, 0.0, True),
    (8, 1, 16, 24, "window", 5, 3, 0.0, None, False), (3, 3, 20, 70, "window", 130, 20, 2.0, None, True),
    (6, 3, 48, 64, "window", 37, 5, 0.0, None, False), (16, 2, 8, 8, "chunk", 1, 0, 20.0, 0.0, True),
    (2, 2, 33, 130, "window", 1, 1, 0.0, 0.5, False), (6, 2, 128, 128, "chunk", 100, 0, 20.0, 0.0, True)])
def test_attention_op_with_cap_kept_tokens_and_mixing(dev, H, G, d, dv, mask, size, keep, cap, sink, talk, dtype):
    from ipex_llm_amd.ops import maskattn as MA
    g = torch.Generator().manual_seed(H + d)
    L = 200
    k = torch.randn(L, G, d, generator=g).to(dtype)
    v = torch.randn(L, G, dv, generator=g).to(dtype)
    tk = (torch.eye(H) + 0.4 * torch.randn(H, H, generator=g)) if talk else None
    sk = torch.full((H,), sink) if sink is not None else None
    rows, bt = paged_rows(k, v, dev, dtype)
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    for positions in (list(range(120, 200)), [0], [keep], [63], [64], [199]):
        n = len(positions)
        q = torch.randn(n, H, d, generator=g) * 1.5
        got = MA.masked_attention(q.to(dev), rows, G, dv, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                  torch.tensor(positions, device=dev), d ** -0.5, mask, size,
                                  sk.to(dev) if sk is not None else None, [n], [positions[-1] + 1], dtype, softcap=cap,
                                  keep_first=keep, talk=tk.to(dev) if talk else None)
        want = plain_attention(q.double(), k.double(), v.double(), d ** -0.5, positions, mask, size, keep, cap, sink,
                               tk.double() if talk else None)
        assert got.dtype == dtype and (got.double().cpu() - want).abs().max() < tol, positions[:2]


@pytest.mark.parametrize("size,keep", [(70, 3), (64, 17), (33, 1)])
@pytest.mark.parametrize("where", ["window_in", "window_out", "first_in", "first_out"])
def test_one_key_stands_out(dev, size, keep, where):
    """one key's score towers over the others: the output is its value when the key is the last one inside the
    window or the last kept first token, and must not contain it when it is just outside either -- for a query in
    a prompt portion and for a single decoded token"""
    from ipex_llm_amd.ops import maskattn as MA
    g = torch.Generator().manual_seed(size + keep)
    H, G, d, dv, L = 2, 1, 16, 12, 330
    p = 300
    j = {"window_in": p - size + 1, "window_out": p - size, "first_in": keep - 1, "first_out": keep}[where]
    k = torch.randn(L, G, d, generator=g) * 0.1
    v = torch.randn(L, G, dv, generator=g)
    q = torch.randn(1, H, d, generator=g) * 0.1
    k[j, 0] = 30.0 * q[0, 0] / q[0, 0].norm() ** 2
    rows, bt = paged_rows(k, v, dev, torch.float32, seed=5)
    want = plain_attention(q.double(), k.double(), v.double(), 1.0, [p], "window", size, keep, 0.0, None, None)
    for positions in ([p], list(range(p - 40, p + 1))):
        n = len(positions)
        qq = torch.cat([torch.randn(n - 1, H, d, generator=g) * 0.1, q])
        got = MA.masked_attention(qq.to(dev), rows, G, dv, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                  torch.tensor(positions, device=dev), 1.0, "window", size, None, [n], [p + 1],
                                  torch.float32, keep_first=keep)[-1].double().cpu()
        assert (got - want[0]).abs().max() < 1e-4
        hit = (got[:dv] - v[j, 0].double()).abs().max() < 1e-3
        assert hit == where.endswith("_in")


def test_fixed_sink_and_mixing_show(dev):
    """with every score far below 0 the sink of score 0 takes all the weight; a mixing matrix that swaps two heads
    swaps what their weights pick from the values"""
    from ipex_llm_amd.ops import maskattn as MA
    g = torch.Generator().manual_seed(3)
    H, G, d, dv, L = 2, 1, 8, 8, 20
    k, v = torch.randn(L, G, d, generator=g), torch.randn(L, G, dv, generator=g)
    q = torch.randn(1, H, d, generator=g)
    rows, bt = paged_rows(k, v, dev, torch.float32)
    args = (rows, G, dv, bt, torch.zeros(1, dtype=torch.int32, device=dev), torch.tensor([L - 1], device=dev))
    zero = torch.zeros(H, device=dev)
    low = MA.masked_attention((q * 0).to(dev), *args, 1.0, "chunk", 64, zero - 40.0, [1], [L], torch.float32).cpu()
    assert (low - v[:, 0].mean(0).repeat(2)[None]).abs().max() < 1e-5     # no sink to speak of: the plain mean
    got = MA.masked_attention((q * 0).to(dev), *args, 1.0, "chunk", 64, zero, [1], [L], torch.float32).cpu()
    assert (got - low * L / (L + 1)).abs().max() < 1e-5                   # L scores of 0 beside a sink of 0
    swap = torch.tensor([[0.0, 1.0], [1.0, 0.0]])
    a = MA.masked_attention(q.to(dev), *args, 1.0, "chunk", 64, zero, [1], [L], torch.float32).cpu()
    b = MA.masked_attention(q.to(dev), *args, 1.0, "chunk", 64, zero, [1], [L], torch.float32, talk=swap.to(dev)).cpu()
    assert (a[0, :dv] - b[0, dv:]).abs().max() < 1e-5 and (a[0, dv:] - b[0, :dv]).abs().max() < 1e-5
    assert (a[0, :dv] - a[0, dv:]).abs().max() > 1e-2


# ------------------------------------------------------------------ whole models
_want = {}


def oracle(cfg, W, toks, key):
    if key not in _want:
        _want[key] = O.forward(cfg, W, toks)
    return _want[key]


LAYER_CASES = [
    [O.gru_layer(width=24, mlp=O.moe(5, 2, 12))],
    [O.gru_layer(width=1), O.gru_layer(width=130, mlp=O.moe(1, 1, 8))],
    [O.attn_layer(heads=4, kv_heads=2, mlp=O.moe(4, 4, 8))],
    [O.attn_layer(heads=2, kv_heads=2, dim=10, vdim=6, chunk=1, taps=1, softcap=0.0), O.attn_layer(heads=2, kv_heads=2, dim=10, vdim=6, chunk=1, taps=2, kv_from=0)],
    [O.attn_layer(heads=6, kv_heads=1, dim=8, vdim=20, chunk=64, taps=5), O.gru_layer(width=8), O.attn_layer(heads=6, kv_heads=1, dim=8, vdim=20, chunk=64, taps=2, kv_from=0, mlp=O.moe(3, 2, 8))],
    [O.pair_layer(mlp=O.moe(3, 2, 8))],
    [O.pair_layer(heads=2, kv_heads=1, dim=16, vdim=8, window=1, keep=0, taps=1, dims=16, rheads=1, rdim=1, rvdim=1, tau=1.0)],
    [O.pair_layer(heads=3, kv_heads=3, dim=6, vdim=6, window=64, keep=64, taps=4, dims=2, rheads=5, rdim=9, rvdim=3, tau=12.0,
                  scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 32})],
    [O.pair_layer(window=5, keep=9, dims=0)],
]


@pytest.mark.parametrize("case", range(len(LAYER_CASES)))
def test_small_models(dev, case):
    """each mixer alone and in pairs, sizes that are 1 or equal to each other, no token-side input in the odd cases"""
    cfg = O.config(LAYER_CASES[case], width=24 + 2 * case, side=0 if case % 2 else 3, logit_softcap=0.0 if case == 2 else 6.0)
    W = O.random_weights(cfg, case)
    toks = O.random_tokens(cfg, 75, case)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 40)], [("a", 30)]] + [[("a", 1)]] * 5)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


@pytest.mark.parametrize("case", [0, 4, 7])
def test_small_models_bf16(dev, case):
    cfg = O.config(LAYER_CASES[case], width=24 + 2 * case)
    W = O.random_weights(cfg, case)
    toks = O.random_tokens(cfg, 75, case)
    got = replay(engine(cfg, W, dev, torch.bfloat16), {"a": toks}, [[("a", 70)], [("a", 3)]] + [[("a", 1)]] * 2)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.bfloat16]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_sizes(dev, dtype):
    """widths, head sizes, expert sizes, side size and vocabulary that are multiples of nothing"""
    cfg = O.config([O.attn_layer(heads=3, kv_heads=1, dim=9, vdim=7, chunk=5, taps=3, mlp=O.moe(3, 2, 5)),
                    O.gru_layer(width=11, mlp=O.moe(2, 1, 7)),
                    O.attn_layer(heads=3, kv_heads=1, dim=9, vdim=7, chunk=5, taps=2, kv_from=0),
                    O.pair_layer(heads=5, kv_heads=5, dim=9, vdim=3, window=6, keep=1, taps=3, dims=4, rheads=3, rdim=5,
                                 rvdim=3, tau=2.5, mlp=O.moe(5, 5, 3))], vocab=53, width=37, side=5)
    W = O.random_weights(cfg, 31)
    toks = O.random_tokens(cfg, 70, 31)
    got = replay(engine(cfg, W, dev, dtype), {"a": toks}, [[("a", 33)], [("a", 30)]] + [[("a", 1)]] * 7)["a"]
    # 16-bit: rows of 3 to 37 values average little rounding away
    assert rel_err(got, O.forward(cfg, W, toks)) < (TOL[dtype] if dtype == torch.float32 else 0.2)


def test_whole_prompt_and_layers(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 7)
    toks = O.random_tokens(cfg, 141, 7)
    eng = engine(cfg, W, dev)
    eng.model.capture_layers = []
    got = replay(eng, {"a": toks}, [[("a", 141)]])["a"]
    layers = []
    want = O.forward(cfg, W, toks, layers_out=layers)
    assert rel_err(got, want) < TOL[torch.float32]
    assert len(eng.model.capture_layers) == len(layers)
    for a, b in zip(eng.model.capture_layers, layers):
        assert (a.double().cpu() - b).abs().max() < 1e-3 * float(b.abs().max())


def test_first_tokens(dev):
    """sequences of one to four tokens (shorter than the convolutions, inside the kept tokens), each alone and
    decoded one by one"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 8)
    for n in (1, 2, 3, 4):
        toks = O.random_tokens(cfg, n, n)
        want = O.forward(cfg, W, toks)
        assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", n)]])["a"], want) < TOL[torch.float32]
        assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", 1)]] * n)["a"], want) < TOL[torch.float32]


def test_prefill_equals_token_by_token(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 9)
    toks = O.random_tokens(cfg, 80, 9)
    want = oracle(cfg, W, toks, "p9")
    assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", 1)]] * 80)["a"], want) < TOL[torch.float32]
    assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", 80)]])["a"], want) < TOL[torch.float32]


@pytest.mark.parametrize("sizes", [[2] * 40, [63, 2, 64, 1, 3, 65], [5, 59, 1, 1, 62, 2, 70], [130, 2, 2, 66]])
def test_portions(dev, sizes):
    cfg = std_cfg()
    W = O.random_weights(cfg, 10)
    toks = O.random_tokens(cfg, 200, 10)[:sum(sizes)]
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", n)] for n in sizes])["a"]
    assert rel_err(got, oracle(cfg, W, O.random_tokens(cfg, 200, 10), "p10")[:sum(sizes)]) < TOL[torch.float32]


def test_unequal_batch_equals_each_alone(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 11)
    P = {"a": O.random_tokens(cfg, 100, 1), "b": O.random_tokens(cfg, 9, 2), "c": O.random_tokens(cfg, 67, 3),
         "d": O.random_tokens(cfg, 30, 4)}
    schedule = [[("a", 50), ("b", 1)], [("a", 14), ("b", 1), ("c", 64), ("d", 2)], [("a", 1), ("b", 2), ("c", 2), ("d", 27)],
                [("a", 35), ("b", 5), ("c", 1), ("d", 1)]]
    got = replay(engine(cfg, W, dev), P, schedule)
    for name, toks in P.items():
        assert rel_err(got[name], oracle(cfg, W, toks, "b11" + name)) < TOL[torch.float32], name


def test_pages_and_slots_used_again(dev):
    """a pool of three pages and two slots serves five requests one after another and side by side"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 12)
    P = {n: O.random_tokens(cfg, ln, i) for i, (n, ln) in enumerate([("a", 100), ("b", 60), ("c", 120), ("d", 3), ("e", 64)])}
    schedule = [[("a", 100)], [("b", 30)], [("b", 30)], [("c", 64), ("d", 1)], [("c", 56), ("d", 2)], [("e", 2)], [("e", 62)]]
    eng = engine(cfg, W, dev, max_batch=2, num_blocks=3)
    got = replay(eng, P, schedule)
    for name, toks in P.items():
        assert rel_err(got[name], oracle(cfg, W, toks, "s12" + name)) < TOL[torch.float32], name
    assert int(eng.sched.num_free_blocks()) == 3 and int(eng.sched.num_free_slots()) == 2


def test_long_decoding(dev):
    """decoded tokens walk over several windows, chunks and pages"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 13)
    toks = O.random_tokens(cfg, 220, 13)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 60)]] + [[("a", 1)]] * 160)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


def test_bfloat16_serving_precision(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 14)
    toks = O.random_tokens(cfg, 90, 14)
    want = O.forward(cfg, W, toks)
    got = replay(engine(cfg, W, dev, torch.bfloat16), {"a": toks}, [[("a", 73)], [("a", 2)]] + [[("a", 1)]] * 15)["a"]
    assert rel_err(got, want) < TOL[torch.bfloat16]


def test_a_far_token_reaches_through_the_recurrences(dev):
    """changing the first token changes the logits hundreds of tokens later (the recurrent states and the kept
    first tokens carry it); the framework follows the plain form on both prompts"""
    cfg = O.config([O.pair_layer(window=8, keep=2, tau=64.0), O.gru_layer(width=16)], width=24)
    W = O.random_weights(cfg, 16)
    a = O.random_tokens(cfg, 300, 16)
    b = [(a[0] + 1) % cfg["vocab"]] + a[1:]
    wa, wb = O.forward(cfg, W, a)[-1], O.forward(cfg, W, b)[-1]
    assert (wa - wb).abs().max() > 1e-3
    for toks, want in ((a, wa), (b, wb)):
        got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 290)]] + [[("a", 1)]] * 10)["a"][-1]
        assert (got - want).abs().max() < 0.05 * float((wa - wb).abs().max())


@pytest.mark.parametrize("chunk,sizes", [(128, [50, 390, 10]), (300, [140, 310]), (300, [5, 445])])
def test_long_chunks_take_the_product_path(dev, chunk, sizes):
    """pieces of chunks long enough for the batched-product path on the GPU, with capped scores and mixed heads"""
    cfg = O.config([O.attn_layer(heads=4, kv_heads=2, dim=16, vdim=24, chunk=chunk, taps=2, mlp=O.moe(3, 2, 8)),
                    O.attn_layer(heads=4, kv_heads=2, dim=16, vdim=24, chunk=chunk, taps=3, kv_from=0)], width=32)
    W = O.random_weights(cfg, 15)
    toks = O.random_tokens(cfg, 450, 15)
    want = oracle(cfg, W, toks, f"c{chunk}")
    for dtype in (torch.float32, torch.bfloat16):
        got = replay(engine(cfg, W, dev, dtype), {"a": toks}, [[("a", n)] for n in sizes])["a"]
        assert rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("window,keep,sizes", [(100, 3, [50, 390, 10]), (300, 40, [300, 150]), (64, 0, [5, 445]), (700, 9, [450])])
def test_long_windows_take_the_product_path(dev, window, keep, sizes, monkeypatch):
    """portions long enough for the block-by-block product path of a sliding window on the GPU (its threshold and
    block lowered to this test's lengths): blocks whose window starts before, at and after the kept first tokens, a
    portion that continues what an earlier step left"""
    from ipex_llm_amd.ops import maskattn as MA
    monkeypatch.setattr(MA, "WINDOW_GEMM_MIN", 128)
    monkeypatch.setattr(MA, "WINDOW_Q_BLOCK", 160)
    cfg = O.config([O.pair_layer(heads=4, kv_heads=2, dim=16, vdim=24, window=window, keep=keep, taps=2, dims=8,
                                 mlp=O.moe(3, 2, 8)), O.gru_layer(width=8)], width=32)
    W = O.random_weights(cfg, 17)
    toks = O.random_tokens(cfg, 450, 17)
    want = oracle(cfg, W, toks, f"w{window}")
    for dtype in (torch.float32, torch.bfloat16):
        got = replay(engine(cfg, W, dev, dtype), {"a": toks}, [[("a", n)] for n in sizes])["a"]
        # 16-bit: the worst of 450 rows behind two recurrences and up to 340 keys in view
        assert rel_err(got, want) < (TOL[dtype] if dtype == torch.float32 else 0.3)


def test_greedy_generation_scheduler(dev):
    """LLMEngine.generate: C++ scheduler, chunked prompts (7 tokens a step in all), requests of unequal
    length side by side, greedy sampling"""
    from ipex_llm_amd.serving.engine import SamplingParams
    cfg = std_cfg()
    W = O.random_weights(cfg, 19)
    prompts = [O.random_tokens(cfg, n, 20 + n) for n in (23, 3, 70, 11)]
    want = [O.greedy(cfg, W, p, 6) for p in prompts]
    for prefill, batch, graph in ((7, 4, False), (1 << 30, 2, True)):
        eng = engine(cfg, W, dev, max_batch=batch, num_blocks=8, prefill=prefill, graph=graph)
        got = eng.generate(prompts, SamplingParams(max_new_tokens=6))
        assert got == want
        assert int(eng.sched.num_free_blocks()) == 8 and int(eng.sched.num_free_slots()) == batch


@pytest.mark.gpu
def test_decode_graph_replays_equal_eager():
    """pure-decode steps replayed from a captured graph (padded rows on the scratch page and slot), with eager
    prompt steps and synchronisations between the replays"""
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    cfg = std_cfg()
    W = O.random_weights(cfg, 21)
    P = {"a": O.random_tokens(cfg, 90, 1), "b": O.random_tokens(cfg, 40, 2), "c": O.random_tokens(cfg, 75, 3)}
    schedule = [[("a", 60), ("b", 20)]] + [[("a", 1), ("b", 1)]] * 10 + [[("c", 66)]] + \
               [[("a", 1), ("b", 1), ("c", 1)]] * 9 + [[("a", 11)]]
    dev = torch.device("cuda")
    eager = replay(engine(cfg, W, dev, torch.bfloat16), P, schedule, keep_open=P)
    graph = replay(engine(cfg, W, dev, torch.bfloat16, graph=True), P, schedule, keep_open=P)
    for name in P:
        assert torch.equal(eager[name], graph[name]), name


def write_checkpoint(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))


def test_checkpoint_registry_and_generate(tmp_path):
    """a checkpoint folder is recognised by its architecture name and generates through the engine; the rank of
    the decay projection comes from its tensor"""
    from ipex_llm_amd.models.registry import NativeCheckpointLM, native_architecture
    cfg = std_cfg()
    W = O.random_weights(cfg, 22)
    write_checkpoint(str(tmp_path / "m"), cfg, W)
    assert native_architecture(str(tmp_path / "m")) == "Zoguzen"
    lm = NativeCheckpointLM(str(tmp_path / "m"), dtype=torch.float32, device="cpu")
    prompt = O.random_tokens(cfg, 12, 5)
    out = lm.generate([prompt], max_new_tokens=5)
    assert out[0][len(prompt):] == O.greedy(cfg, W, prompt, 5)


def test_reader_refuses_what_it_does_not_know():
    from ipex_llm_amd.models import zoguzen as Z
    with pytest.raises(ValueError):
        Z.spec_from_config(O.config([O.attn_layer(kv_from=0)]))          # borrows from itself
    with pytest.raises(ValueError):
        Z.spec_from_config(O.config([O.gru_layer(), O.attn_layer(kv_from=0)]))   # layer 0 holds no keys
    cfg = O.config([O.attn_layer()])
    cfg["layers"][0]["type"] = "something"
    with pytest.raises(ValueError):
        Z.spec_from_config(cfg)
    with pytest.raises(ValueError):
        Z.spec_from_config(O.config([O.pair_layer()]))                   # the decay projection's rank is not known
    cfg = O.config([O.attn_layer(mlp=O.moe(2, 1, 8))])
    W = O.random_weights(cfg)
    del W["l0.mix.talk"]
    with pytest.raises(KeyError):
        Z.build(Z.spec_from_config(cfg), W, torch.float32, "cpu")


def test_trace_replay_program(tmp_path, dev):
    """bin/trace_run: steps on standard input, logits files out, pages and slots given back at 'end'"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 23)
    write_checkpoint(str(tmp_path / "m"), cfg, W)
    a, b = O.random_tokens(cfg, 70, 1), O.random_tokens(cfg, 20, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[40:69], "want": []}, {"id": "b", "tokens": b[:19], "want": [18]}], "end": []},
             {"step": 2, "entries": [{"id": "b", "tokens": b[19:], "want": [0]}, {"id": "a", "tokens": a[69:], "want": [0]}], "end": ["a", "b"]},
             {"step": 3, "entries": [{"id": "c", "tokens": b, "want": [19]}], "end": ["c"]}]
    env = dict(os.environ, ILLM_TRACE_DEVICE=dev.type)
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path / "m"), "--dtype",
                        "float32", "--out", str(tmp_path / "out"), "--max-tokens", "192"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, env=env,
                       timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    import numpy as np
    V = cfg["vocab"]
    wa, wb = O.forward(cfg, W, a), O.forward(cfg, W, b)
    rd = lambda i: torch.from_numpy(np.fromfile(str(tmp_path / "out" / f"{i}.f32"), dtype="<f4").reshape(-1, V)).double()  # noqa: E731
    assert rel_err(rd(0), wa[[0, 39]]) < TOL[torch.float32]
    assert rel_err(rd(1), wb[[18]]) < TOL[torch.float32]
    assert rel_err(rd(2), torch.stack([wb[19], wa[69]])) < TOL[torch.float32]
    assert rel_err(rd(3), wb[[19]]) < TOL[torch.float32]
