"""Pre-norm hybrid decoders (Vogolix layout): the framework -- checkpoint
reader, paged rows and state slots, scheduler, ragged engine steps, kernels --
against the plain float64 forms of tests/prenorm_oracle.py.

Every test runs on the CPU (torch forms of ops/ssm.py, ops/maskattn.py, ...)
and, marked ``gpu``, on the HIP kernels.  Models are small random ones made
here.
"""
import json
import math
import os
import subprocess
import sys

import pytest
import torch

from . import prenorm_oracle as O

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
    """all three mixers, a layer that borrows keys and values, layers with and without a feed-forward; a window
    and a chunk shorter than a page and ones that straddle pages"""
    return O.config([O.attn_layer(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, dims=8, ff=48),
                     O.ssm_layer(heads=4, vdim=12, state=10, groups=2, taps=3, norm_groups=2, ff=32),
                     O.attn_layer(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, dims=8, kv_from=0),
                     O.latent_layer(heads=3, dim=12, rot_dim=8, vdim=10, kv_rank=20, window=9, ff=40),
                     O.attn_layer(heads=2, kv_heads=1, dim=16, vdim=24, chunk=70, dims=16, scale=0.25, ff=24),
                     O.latent_layer(heads=2, dim=8, rot_dim=4, vdim=16, kv_rank=12, window=66),
                     O.ssm_layer(heads=2, vdim=20, state=70, groups=1, taps=4, norm_groups=1)], width=40)


def build(cfg, W, dev, dtype=torch.float32):
    from ipex_llm_amd.models import vogolix as Z
    return Z.build(Z.spec_from_config(cfg), W, dtype, dev)


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


# ------------------------------------------------------------------ mechanisms alone (ops)
def test_add_norm_and_gates(dev):
    from ipex_llm_amd.ops import blockmix as BM, maskattn as MA, seqmix as SM, ssm as SSM
    g = torch.Generator().manual_seed(0)
    for act in (torch.float32, torch.bfloat16):
        for T, Wd in ((7, 50), (7, 52), (70, 4160)):                        # odd rows, 4-value rows, rows past the registers
            x = torch.randn(T, Wd, generator=g)
            y = torch.randn(T, Wd, generator=g).to(act)
            w = (1 + 0.3 * torch.randn(Wd, generator=g)).to(act)
            xs = x.clone().to(dev)
            h = BM.add_rms_norm_rows_(xs, y.to(dev), w.to(dev), 1e-5, act)
            s = x.double() + y.double()
            assert torch.equal(xs.cpu(), (x + y.float()))
            want = O.unit_rms(s, 1e-5) * w.double()
            assert h.dtype == act and (h.double().cpu() - want).abs().max() < (2e-5 if act == torch.float32 else 5e-2)
            h0 = BM.add_rms_norm_rows_(xs, None, w.to(dev), 1e-5, act)      # nothing to add: a plain norm
            assert (h0.double().cpu() - want).abs().max() < (2e-5 if act == torch.float32 else 5e-2)
        gu = torch.randn(5, 2 * 33, generator=g).to(act)
        for name, f in (("relu", torch.relu), ("silu", O.silu), ("gelu_tanh", None)):
            a = gu[:, :33].double()
            ref = (f(a) if f else 0.5 * a * (1 + torch.tanh(math.sqrt(2 / math.pi) * (a + 0.044715 * a ** 3)))) * gu[:, 33:].double()
            got = SM.glu_act(gu.to(dev), name)
            assert (got.double().cpu() - ref).abs().max() < (1e-5 if act == torch.float32 else 5e-2)
        o = torch.randn(6, 24, generator=g).to(act)
        big = torch.randn(6, 80, generator=g).to(act)
        got = MA.sigmoid_gate(o.clone().to(dev), big.to(dev)[:, 30:54])
        ref = o.double() * torch.sigmoid(big[:, 30:54].double())
        assert (got.double().cpu() - ref).abs().max() < (1e-5 if act == torch.float32 else 3e-2)
        yy = torch.randn(5, 48, generator=g)
        z = torch.randn(5, 100, generator=g).to(act)
        nw = (1 + 0.2 * torch.randn(48, generator=g)).to(act)
        for groups in (1, 3, 48):
            got = SSM.gated_group_norm(yy.to(dev), z.to(dev)[:, 10:58], nw.to(dev), groups, 1e-5, act)
            v = yy.double() * O.silu(z[:, 10:58].double())
            ref = O.unit_rms(v.view(5, groups, -1), 1e-5).reshape(5, 48) * nw.double()
            assert (got.double().cpu() - ref).abs().max() < (1e-5 if act == torch.float32 else 5e-2)


@pytest.mark.parametrize("C,off", [(37, 2), (40, 4)])
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_convolution_state(dev, taps, C, off):
    """portions of every length from the start of a sequence and from its middle, sequences side by side,
    slots that held other sequences before"""
    from ipex_llm_amd.ops import ssm as SSM
    g = torch.Generator().manual_seed(taps)
    n = 23                                                          # (C, off): channels one by one / four at a time
    w = torch.randn(C, taps, generator=g)
    b = torch.randn(C, generator=g)
    seqs = [torch.randn(n, C + 8, generator=g) for _ in range(3)]
    want = [O.silu(O.causal_conv(u[:, off:off + C].double(), w.double(), b.double())) for u in seqs]
    state = torch.randn(5, taps - 1, C, generator=g).to(dev)            # rubbish of earlier owners
    cuts = [[1, 1, 1, 2, 3, 5, 10], [23], [2, 1, 1, 19]]
    at = [0, 0, 0]
    got = [[], [], []]
    for step in range(7):
        act = [s for s in range(3) if step < len(cuts[s])]
        lens = [cuts[s][step] for s in act]
        starts = [at[s] for s in act]
        cu, seq_of, _, pos = ragged(lens, starts, dev)
        slots = torch.tensor([s + 1 for s in act], dtype=torch.int32, device=dev)
        u = torch.cat([seqs[s][at[s]:at[s] + m] for s, m in zip(act, lens)]).to(dev)[:, off:off + C]
        out = SSM.conv_silu(u, w.to(dev), b.to(dev), state, cu, seq_of, slots, pos, lens)
        o = 0
        for s, m in zip(act, lens):
            got[s].append(out[o:o + m].double().cpu())
            o += m
            at[s] += m
    for s in range(3):
        assert (torch.cat(got[s]) - want[s]).abs().max() < 1e-5


@pytest.mark.parametrize("H,G,P,N", [(4, 2, 12, 10), (2, 1, 70, 33), (3, 3, 8, 130), (1, 1, 64, 64)])
def test_selective_scan_op(dev, H, G, P, N):
    from ipex_llm_amd.ops import ssm as SSM
    g = torch.Generator().manual_seed(H * 100 + N)
    n = 41
    x, Bm, Cm = torch.randn(n, H, P, generator=g), torch.randn(n, G, N, generator=g), torch.randn(n, G, N, generator=g)
    dt_pre = torch.randn(n, H + 3, generator=g) * 2
    dt_bias, a_log, d_skip = torch.randn(H, generator=g), torch.randn(H, generator=g) * 0.7 - 0.5, torch.randn(H, generator=g)
    dt = O.softplus(dt_pre[:, 1:1 + H].double() + dt_bias.double())
    want = torch.zeros(n, H, P, dtype=F64)
    for h in range(H):
        S = torch.zeros(N, P, dtype=F64)
        for t in range(n):
            S = math.exp(-math.exp(float(a_log[h])) * float(dt[t, h])) * S + dt[t, h] * torch.outer(Bm[t, h // (H // G)].double(), x[t, h].double())
            want[t, h] = S.t() @ Cm[t, h // (H // G)].double() + d_skip[h].double() * x[t, h].double()
    state = torch.randn(3, H, N, P, generator=g).to(dev)
    got, at = [], 0
    for m in (1, 1, 17, 2, 20):
        cu, _, slots, pos = ragged([m], [at], dev)
        got.append(SSM.selective_scan(x[at:at + m].to(dev), Bm[at:at + m].to(dev), Cm[at:at + m].to(dev),
                                      dt_pre.to(dev)[at:at + m, 1:1 + H], dt_bias.to(dev), a_log.to(dev), d_skip.to(dev),
                                      state, cu, slots, pos, [m]).double().cpu())
        at += m
    got = torch.cat(got)
    assert (got - want).abs().max() < 2e-4 * max(1.0, float(want.abs().max()))


def plain_masked_attention(q, k, v, scale, positions, mask, size, sink):
    """q [n, H, d] at ``positions`` over keys k [L, G, d], values v [L, G, dv] (f64)"""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(n, H, v.shape[-1], dtype=F64)
    for i, p in enumerate(positions):
        lo = 0 if mask == "causal" else (max(0, p - size + 1) if mask == "window" else (p // size) * size)
        for h in range(H):
            g = h // (H // G)
            s = (k[lo:p + 1, g] @ q[i, h]) * scale
            top = float(s.max()) if sink is None else max(float(s.max()), float(sink[h]))
            e = torch.exp(s - top)
            den = e.sum() + (0.0 if sink is None else math.exp(float(sink[h]) - top))
            out[i, h] = (e @ v[lo:p + 1, g]) / den
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
@pytest.mark.parametrize("H,G,d,dv,mask,size,sink", [
    (4, 2, 12, 10, "chunk", 7, True), (4, 4, 80, 48, "chunk", 32, True), (8, 1, 16, 24, "window", 5, False),
    (3, 3, 20, 70, "window", 130, True), (2, 1, 64, 64, "causal", 0, False), (16, 2, 8, 8, "chunk", 1, True),
    (2, 2, 33, 130, "window", 1, False), (6, 2, 128, 128, "chunk", 100, True)])
def test_masked_attention_op(dev, H, G, d, dv, mask, size, sink, dtype):
    """every mask, with and without a sink, one and many query heads per key head, value sizes other than the
    key size: a prompt portion that ends the context, and single tokens at scattered positions"""
    from ipex_llm_amd.ops import maskattn as MA
    g = torch.Generator().manual_seed(H + d)
    L = 200
    k = torch.randn(L, G, d, generator=g).to(dtype)
    v = torch.randn(L, G, dv, generator=g).to(dtype)
    sk = (torch.randn(H, generator=g) + 1.0) if sink else None
    rows, bt = paged_rows(k, v, dev, dtype)
    tol = 1e-4 if dtype == torch.float32 else 3e-2
    for positions in (list(range(120, 200)), [0], [63], [64], [199]):
        n = len(positions)
        q = torch.randn(n, H, d, generator=g) * 1.5
        ctx = positions[-1] + 1
        got = MA.masked_attention(q.to(dev), rows, G, dv, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                  torch.tensor(positions, device=dev), d ** -0.5, mask, size,
                                  sk.to(dev) if sink else None, [n], [ctx], dtype)
        want = plain_masked_attention(q.double(), k.double(), v.double(), d ** -0.5, positions, mask, size, sk)
        assert got.dtype == dtype and (got.double().cpu() - want).abs().max() < tol, positions[:2]


@pytest.mark.parametrize("mask,size", [("window", 70), ("chunk", 70), ("window", 64), ("chunk", 64), ("chunk", 128)])
@pytest.mark.parametrize("edge", [-1, 0, 1])
def test_one_key_stands_out(dev, mask, size, edge):
    """one key's score towers over the others: the output is its value when the key is the last one inside the
    view (or well inside), and must not contain it when it is the first one outside -- for a query in a prompt
    portion and for a single decoded token"""
    from ipex_llm_amd.ops import maskattn as MA
    g = torch.Generator().manual_seed(size + edge)
    H, G, d, dv, L = 2, 1, 16, 12, 330
    p = 300                                                           # the query's position
    first = p - size + 1 if mask == "window" else (p // size) * size
    j = first + edge if edge >= 0 else first - 1                      # inside at the edge, one further in, just outside
    k = torch.randn(L, G, d, generator=g) * 0.1
    v = torch.randn(L, G, dv, generator=g)
    q = torch.randn(1, H, d, generator=g) * 0.1
    k[j, 0] = 30.0 * q[0, 0] / q[0, 0].norm() ** 2                    # score 30 with head 0
    rows, bt = paged_rows(k, v, dev, torch.float32, seed=5)
    want = plain_masked_attention(q.double(), k.double(), v.double(), 1.0, [p], mask, size, None)
    for positions in ([p], list(range(p - 40, p + 1))):
        n = len(positions)
        qq = torch.cat([torch.randn(n - 1, H, d, generator=g) * 0.1, q])
        got = MA.masked_attention(qq.to(dev), rows, G, dv, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                  torch.tensor(positions, device=dev), 1.0, mask, size, None, [n], [p + 1],
                                  torch.float32)[-1].double().cpu()
        assert (got - want[0]).abs().max() < 1e-4
        hit = (got[:dv] - v[j, 0].double()).abs().max() < 1e-3
        assert hit == (edge >= 0)


def test_sink_takes_weight(dev):
    """a sink far above every score leaves almost nothing for the values; one far below changes nothing"""
    from ipex_llm_amd.ops import maskattn as MA
    g = torch.Generator().manual_seed(3)
    H, G, d, dv, L = 2, 2, 8, 8, 20
    k, v, q = torch.randn(L, G, d, generator=g), torch.randn(L, G, dv, generator=g), torch.randn(1, H, d, generator=g)
    rows, bt = paged_rows(k, v, dev, torch.float32)
    args = (rows, G, dv, bt, torch.zeros(1, dtype=torch.int32, device=dev), torch.tensor([L - 1], device=dev), 0.3, "chunk", 64)
    none = MA.masked_attention(q.to(dev), *args, None, [1], [L], torch.float32).cpu()
    for s0, s1 in ((40.0, -40.0), (-40.0, 40.0)):
        sk = torch.tensor([s0, s1])
        got = MA.masked_attention(q.to(dev), *args, sk.to(dev), [1], [L], torch.float32).cpu()
        want = plain_masked_attention(q.double(), k.double(), v.double(), 0.3, [L - 1], "chunk", 64, sk)
        assert (got.double() - want).abs().max() < 1e-5
        hi, lo = (0, 1) if s0 > 0 else (1, 0)
        assert got[0, hi * dv:(hi + 1) * dv].abs().max() < 1e-6
        assert (got[0, lo * dv:(lo + 1) * dv] - none[0, lo * dv:(lo + 1) * dv]).abs().max() < 1e-6


@pytest.mark.parametrize("whole", [True, False])
@pytest.mark.parametrize("layout", ["pairs", "half"])
def test_norm_rotation_and_rows(dev, whole, layout):
    from ipex_llm_amd.ops import maskattn as MA, seqmix as SM
    g = torch.Generator().manual_seed(1)
    T, H, G, d, dv, dims = 9, 4, 2, 12, 10, 8
    y = torch.randn(T, H * d + G * d + G * dv + 3, generator=g)
    q, k = y[:, :H * d].view(T, H, d), y[:, H * d:(H + G) * d].view(T, G, d)
    v = y[:, (H + G) * d:(H + G) * d + G * dv].view(T, G, dv)
    qn = 1 + 0.3 * torch.randn(H * d if whole else d, generator=g)
    kn = 1 + 0.3 * torch.randn(G * d if whole else d, generator=g)
    pos = torch.tensor([0, 1, 2, 70, 71, 5, 200, 3, 64])
    slots = torch.tensor([3, 64, 2, 130, 7, 191, 66, 0, 100])
    rot = {"dims": dims, "base": 700.0}
    table = SM.rope_table(256, dims, 700.0)
    rows = torch.zeros(3, 64, G * (d + dv)).to(dev)
    yd = y.to(dev)
    qf = MA.qkv_norm_rope_store(yd[:, :H * d].view(T, H, d), yd[:, H * d:(H + G) * d].view(T, G, d),
                                yd[:, (H + G) * d:(H + G) * d + G * dv].view(T, G, dv), qn.to(dev), kn.to(dev), whole, 1e-5,
                                table.to(dev), layout, pos.to(dev), slots.to(dev), rows)
    turn = O.turn_pairs if layout == "pairs" else O.turn_split

    def ref(x, w):
        x = x.double()
        if whole:
            x = (O.unit_rms(x.reshape(T, -1), 1e-5) * w.double()).view(x.shape)
        else:
            x = O.unit_rms(x, 1e-5) * w.double()
        return turn(x, rot, pos.tolist())
    assert (qf.double().cpu() - ref(q, qn)).abs().max() < 1e-5
    flat = rows.view(-1, G * (d + dv)).cpu()
    assert (flat[slots, :G * d].double() - ref(k, kn).reshape(T, -1)).abs().max() < 1e-5
    assert torch.equal(flat[slots, G * d:], v.reshape(T, -1))
    # a layer that borrows its keys: queries only, nothing written
    q2 = MA.qkv_norm_rope_store(yd[:, :H * d].view(T, H, d), None, None, qn.to(dev), None, whole, 1e-5, table.to(dev),
                                layout, pos.to(dev), slots.to(dev), None)
    assert torch.equal(q2, qf)


@pytest.mark.parametrize("window", [1, 9, 64, 70])
def test_latent_attention_window(dev, window):
    """the latent-attention op with a window: a key that stands out just inside and just outside of it"""
    from ipex_llm_amd.ops import seqmix as SM
    g = torch.Generator().manual_seed(window)
    H, r, dr, L = 3, 20, 8, 210
    c = torch.randn(L, r, generator=g) * 0.2
    kr = torch.randn(L, dr, generator=g) * 0.2
    rows, bt = paged_rows(c, kr, dev, torch.float32, seed=window)
    for positions in (list(range(150, 210)), [209], [0], [window - 1], [window]):
        n = len(positions)
        ql = torch.randn(n, H, r, generator=g) * 0.2
        qr = torch.randn(n, H, dr, generator=g) * 0.2
        want = torch.zeros(n, H, r, dtype=F64)
        for i, p in enumerate(positions):
            lo = max(0, p - window + 1)
            for h in range(H):
                s = (c[lo:p + 1].double() @ ql[i, h].double() + kr[lo:p + 1].double() @ qr[i, h].double()) * 0.9
                want[i, h] = torch.softmax(s, 0) @ c[lo:p + 1].double()
        got = SM.latent_attention(ql.to(dev), qr.to(dev), rows, bt, torch.zeros(n, dtype=torch.int32, device=dev),
                                  torch.tensor(positions, device=dev), 0.9, None, [n], [positions[-1] + 1], torch.float32,
                                  window=window)
        assert (got.double().cpu() - want).abs().max() < 1e-5, positions[:2]


# ------------------------------------------------------------------ models
LAYER_CASES = [
    ([O.ssm_layer(heads=4, vdim=12, state=10, groups=2, taps=3, norm_groups=2, ff=32)], dict(width=40)),
    # one group, one norm group, one head per group, a state past one wave's rows, two taps
    ([O.ssm_layer(heads=2, vdim=70, state=33, groups=2, taps=2, norm_groups=1)], dict(width=24)),
    ([O.ssm_layer(heads=6, vdim=8, state=130, groups=1, taps=5, norm_groups=6, ff=16)], dict(width=32, logit_scale=1.0)),
    ([O.latent_layer(heads=3, dim=12, rot_dim=8, vdim=10, kv_rank=20, window=9, ff=40)], dict(width=40)),
    ([O.latent_layer(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=8, window=1)], dict(width=16)),
    ([O.latent_layer(heads=5, dim=16, rot_dim=16, vdim=24, kv_rank=70, window=100, scale=0.1)], dict(width=48)),
    ([O.attn_layer(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, dims=8, ff=48)], dict(width=40)),
    # one key head for all, the whole head rotated, a chunk of one position, value size above the key size
    ([O.attn_layer(heads=3, kv_heads=1, dim=8, vdim=20, chunk=1, dims=8)], dict(width=24)),
    ([O.attn_layer(heads=2, kv_heads=2, dim=32, vdim=8, chunk=64, dims=2, ff=24),
      O.attn_layer(heads=2, kv_heads=2, dim=32, vdim=8, chunk=64, dims=2, kv_from=0)], dict(width=32)),
    ([O.attn_layer(heads=8, kv_heads=2, dim=16, vdim=16, chunk=100, dims=16),
      O.ssm_layer(heads=2, vdim=8, state=4, groups=1, taps=4),
      O.attn_layer(heads=8, kv_heads=2, dim=16, vdim=16, chunk=100, dims=16, kv_from=0, ff=40)], dict(width=40)),
]


@pytest.mark.parametrize("case", range(len(LAYER_CASES)))
def test_small_models(dev, case):
    layers, kw = LAYER_CASES[case]
    cfg = O.config(layers, **kw)
    W = O.random_weights(cfg, case)
    toks = O.random_tokens(cfg, 150, case)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 150)]])["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", 61)], [("a", 5)], [("a", 2)]] + [[("a", 1)]] * 82)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


@pytest.mark.parametrize("case", [1, 5, 9])
def test_small_models_bf16(dev, case):
    layers, kw = LAYER_CASES[case]
    cfg = O.config(layers, **kw)
    W = O.random_weights(cfg, case)
    toks = O.random_tokens(cfg, 80, case)
    got = replay(engine(cfg, W, dev, torch.bfloat16), {"a": toks}, [[("a", 70)], [("a", 3)]] + [[("a", 1)]] * 7)["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.bfloat16]


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
    """sequences of one to four tokens (shorter than the convolutions), each alone and decoded one by one"""
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
    want = O.forward(cfg, W, toks)
    assert rel_err(replay(engine(cfg, W, dev), {"a": toks}, [[("a", 1)]] * 80)["a"], want) < TOL[torch.float32]


@pytest.mark.parametrize("sizes", [[2] * 40, [63, 2, 64, 1, 3, 65], [5, 59, 1, 1, 62, 2, 70], [130, 2, 2, 66]])
def test_portions(dev, sizes):
    cfg = std_cfg()
    W = O.random_weights(cfg, 10)
    toks = O.random_tokens(cfg, sum(sizes), 10)
    got = replay(engine(cfg, W, dev), {"a": toks}, [[("a", n)] for n in sizes])["a"]
    assert rel_err(got, O.forward(cfg, W, toks)) < TOL[torch.float32]


def test_unequal_batch_equals_each_alone(dev):
    cfg = std_cfg()
    W = O.random_weights(cfg, 11)
    P = {"a": O.random_tokens(cfg, 100, 1), "b": O.random_tokens(cfg, 9, 2), "c": O.random_tokens(cfg, 67, 3),
         "d": O.random_tokens(cfg, 30, 4)}
    schedule = [[("a", 50), ("b", 1)], [("a", 14), ("b", 1), ("c", 64), ("d", 2)], [("a", 1), ("b", 2), ("c", 2), ("d", 27)],
                [("a", 35), ("b", 5), ("c", 1), ("d", 1)]]
    got = replay(engine(cfg, W, dev), P, schedule)
    for name, toks in P.items():
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[torch.float32], name


def test_pages_and_slots_used_again(dev):
    """a pool of three pages and two slots serves five requests one after another and side by side"""
    cfg = std_cfg()
    W = O.random_weights(cfg, 12)
    P = {n: O.random_tokens(cfg, ln, i) for i, (n, ln) in enumerate([("a", 100), ("b", 60), ("c", 120), ("d", 3), ("e", 64)])}
    schedule = [[("a", 100)], [("b", 30)], [("b", 30)], [("c", 64), ("d", 1)], [("c", 56), ("d", 2)], [("e", 2)], [("e", 62)]]
    eng = engine(cfg, W, dev, max_batch=2, num_blocks=3)
    got = replay(eng, P, schedule)
    for name, toks in P.items():
        assert rel_err(got[name], O.forward(cfg, W, toks)) < TOL[torch.float32], name
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


@pytest.mark.parametrize("chunk,sizes", [(128, [50, 390, 10]), (300, [140, 310]), (300, [5, 445])])
def test_long_chunks_take_the_product_path(dev, chunk, sizes):
    """pieces of chunks long enough for the batched-product path on the GPU: whole chunks inside a portion that
    starts and ends mid-chunk, the start of a chunk, and the rest of a chunk whose first keys an earlier step left"""
    cfg = O.config([O.attn_layer(heads=4, kv_heads=2, dim=16, vdim=24, chunk=chunk, dims=8, ff=32),
                    O.attn_layer(heads=4, kv_heads=2, dim=16, vdim=24, chunk=chunk, dims=8, kv_from=0)], width=32)
    W = O.random_weights(cfg, 15)
    toks = O.random_tokens(cfg, 450, 15)
    want = O.forward(cfg, W, toks)
    for dtype in (torch.float32, torch.bfloat16):
        got = replay(engine(cfg, W, dev, dtype), {"a": toks}, [[("a", n)] for n in sizes])["a"]
        assert rel_err(got, want) < TOL[dtype]


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
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))


def test_checkpoint_registry_and_generate(tmp_path):
    """a checkpoint folder is recognised by its architecture name and generates through the engine"""
    from ipex_llm_amd.models.registry import NativeCheckpointLM, native_architecture
    cfg = std_cfg()
    W = O.random_weights(cfg, 22)
    write_checkpoint(str(tmp_path / "m"), cfg, W)
    assert native_architecture(str(tmp_path / "m")) == "Vogolix"
    lm = NativeCheckpointLM(str(tmp_path / "m"), dtype=torch.float32, device="cpu")
    prompt = O.random_tokens(cfg, 12, 5)
    out = lm.generate([prompt], max_new_tokens=5)
    assert out[0][len(prompt):] == O.greedy(cfg, W, prompt, 5)


def test_reader_refuses_what_it_does_not_know():
    from ipex_llm_amd.models import vogolix as Z
    cfg = O.config([O.attn_layer(kv_from=0)])
    with pytest.raises(ValueError):
        Z.spec_from_config(cfg)                                      # borrows from itself
    cfg = O.config([O.ssm_layer(), O.attn_layer(kv_from=0)])
    with pytest.raises(ValueError):
        Z.spec_from_config(cfg)                                      # layer 0 holds no keys
    cfg = O.config([O.attn_layer()])
    cfg["layers"][0]["type"] = "something"
    with pytest.raises(ValueError):
        Z.spec_from_config(cfg)
    cfg = O.config([O.attn_layer(ff=8)])
    W = O.random_weights(cfg)
    del W["l0.mix.sink"]
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
