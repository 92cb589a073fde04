"""Plain float64 forms of the mechanisms of the pre-norm hybrid decoders
(Vogolix layout): a state-space mixer, windowed latent attention and chunked
grouped attention with a sink, one function per mechanism, written from
their equations.  Slow and simple on purpose; shares no code with the package.

A model is (cfg, W): ``cfg`` in the checkpoint's config.json layout, ``W`` a
dict name -> tensor (as stored: bf16 values, [out, in]).
"""
import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ small pieces
def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z / (1 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def angles(rot, positions):
    """[T, dims / 2]: position * base^(-2 i / dims)"""
    n = rot["dims"]
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / n) for i in range(n // 2)], dtype=F64)
    return torch.tensor(positions, dtype=F64)[:, None] * f[None]


def turn_split(x, rot, positions):
    """x [T, heads, n]: value i of the first rot.dims is paired with value i + dims / 2"""
    n = rot["dims"]
    a = angles(rot, positions)[:, None]
    u, v = x[..., :n // 2], x[..., n // 2:n]
    return torch.cat([u * a.cos() - v * a.sin(), v * a.cos() + u * a.sin(), x[..., n:]], -1)


def turn_pairs(x, rot, positions):
    """x [T, heads, n]: value 2 i of the first rot.dims is paired with value 2 i + 1"""
    n = rot["dims"]
    a = angles(rot, positions)[:, None]
    out = x.clone()
    u, v = x[..., 0:n:2], x[..., 1:n:2]
    out[..., 0:n:2] = u * a.cos() - v * a.sin()
    out[..., 1:n:2] = v * a.cos() + u * a.sin()
    return out


# ------------------------------------------------------------------ state-space mixer
def causal_conv(u, w, b):
    """u [T, C], w [C, taps] (last column: the current token), zeros before the start"""
    T, taps = u.shape[0], w.shape[1]
    out = torch.zeros_like(u)
    for t in range(T):
        acc = b.clone()
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                acc = acc + w[:, j] * u[s]
        out[t] = acc
    return out


def ssm_mixer(W, p, m, h, eps):
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    T = h.shape[0]
    y = h @ W[p + "in"].to(F64).t()
    z, xbc, dt = y[:, :inner], y[:, inner:2 * inner + 2 * G * N], y[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"].to(F64), W[p + "conv.b"].to(F64)))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + W[p + "dt_bias"].to(F64))
    rate = torch.exp(W[p + "A_log"].to(F64))
    D = W[p + "D"].to(F64)
    out = torch.zeros(T, H, P, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = math.exp(-float(rate[hd]) * float(dt[t, hd])) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            out[t, hd] = S.t() @ C[t, g] + D[hd] * x[t, hd]
    o = out.reshape(T, inner) * silu(z)
    k = m["norm_groups"]
    o = unit_rms(o.reshape(T, k, inner // k), eps).reshape(T, inner) * W[p + "norm"].to(F64)
    return o @ W[p + "o"].to(F64).t()


# ------------------------------------------------------------------ latent attention in a window
def latent_attention(W, p, m, h, eps):
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    pos = list(range(T))
    q = (h @ W[p + "q"].to(F64).t()).reshape(T, H, d + dr)
    qa, qb = q[..., :d], turn_split(q[..., d:], m["rot"], pos)
    ckr = h @ W[p + "dkv"].to(F64).t()
    c = unit_rms(ckr[:, :r], eps) * W[p + "dkv.norm"].to(F64)
    kb = turn_split(ckr[:, None, r:], m["rot"], pos)[:, 0]
    ka = (c @ W[p + "uk"].to(F64).t()).reshape(T, H, d)
    v = (c @ W[p + "uv"].to(F64).t()).reshape(T, H, dv)
    win = m["mask"]["size"]
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        lo = max(0, t - win + 1)
        for hd in range(H):
            s = (ka[lo:t + 1, hd] @ qa[t, hd] + kb[lo:t + 1] @ qb[t, hd]) * m["scale"]
            out[t, hd] = torch.softmax(s, 0) @ v[lo:t + 1, hd]
    o = out.reshape(T, H * dv) * torch.sigmoid(h @ W[p + "g"].to(F64).t())
    return o @ W[p + "o"].to(F64).t()


# ------------------------------------------------------------------ chunked attention with a sink
def attention_keys(W, p, m, h, eps):
    """the keys (normed, turned) and values of a layer that projects its own: [T, G, d], [T, G, dv]"""
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    k = h @ W[p + "k"].to(F64).t() + W[p + "k.b"].to(F64)
    k = unit_rms(k, eps) * W[p + "k.norm"].to(F64)
    k = turn_pairs(k.reshape(T, G, d), m["rot"], list(range(T)))
    v = (h @ W[p + "v"].to(F64).t() + W[p + "v.b"].to(F64)).reshape(T, G, dv)
    return k, v


def attention(W, p, m, h, eps, kv):
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    k, v = kv
    q = h @ W[p + "q"].to(F64).t() + W[p + "q.b"].to(F64)
    q = unit_rms(q, eps) * W[p + "q.norm"].to(F64)
    q = turn_pairs(q.reshape(T, H, d), m["rot"], list(range(T)))
    size = m["mask"]["size"]
    sink = W[p + "sink"].to(F64)
    out = torch.zeros(T, H, dv, dtype=F64)
    for t in range(T):
        lo = (t // size) * size
        for hd in range(H):
            g = hd // (H // G)
            s = (k[lo:t + 1, g] @ q[t, hd]) * m["scale"]
            top = max(float(s.max()), float(sink[hd]))
            e = torch.exp(s - top)
            out[t, hd] = (e @ v[lo:t + 1, g]) / (e.sum() + math.exp(float(sink[hd]) - top))
    return out.reshape(T, H * dv) @ W[p + "o"].to(F64).t()


# ------------------------------------------------------------------ feed-forward, model
def feed_forward(W, p, h):
    g = torch.relu(h @ W[p + "gate"].to(F64).t())
    return (g * (h @ W[p + "up"].to(F64).t())) @ W[p + "down"].to(F64).t()


def forward(cfg, W, tokens, layers_out=None):
    """logits [T, vocab] of one sequence from position 0 (float64)"""
    eps = cfg["norm"]["eps"]
    x = W["embed"].to(F64)[torch.tensor(tokens)]
    kept = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        h = unit_rms(x, eps) * W[f"l{i}.norm1"].to(F64)
        if L["type"] == "mamba2":
            y = ssm_mixer(W, p, m, h, eps)
        elif L["type"] == "latent_attention":
            y = latent_attention(W, p, m, h, eps)
        else:
            if m.get("kv_from") is None:
                kept[i] = attention_keys(W, p, m, h, eps)
            y = attention(W, p, m, h, eps, kept[m["kv_from"] if m.get("kv_from") is not None else i])
        x = x + y
        if L["mlp"] is not None:
            x = x + feed_forward(W, f"l{i}.mlp.", unit_rms(x, eps) * W[f"l{i}.norm2"].to(F64))
        if layers_out is not None:
            layers_out.append(x.clone())
    x = unit_rms(x, eps) * W["final.norm"].to(F64)
    return (x @ W["head"].to(F64).t()) * cfg.get("logit_scale", 1.0)


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


# ------------------------------------------------------------------ configurations
def ssm_layer(heads=4, vdim=12, state=10, groups=2, taps=3, norm_groups=2, ff=0):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": taps,
                                        "norm_groups": norm_groups}, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def latent_layer(heads=3, dim=12, rot_dim=8, vdim=10, kv_rank=20, window=9, scale=0.2, base=5000.0, ff=0):
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale,
                      "mask": {"size": window}, "rot": {"dims": rot_dim, "base": base}},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def attn_layer(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, dims=8, scale=0.3, base=3000.0, kv_from=None, ff=0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": chunk},
         "rot": {"dims": dims, "base": base}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, vocab=89, width=40, eps=1e-5, logit_scale=0.7):
    return {"architecture": "Vogolix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "logit_scale": logit_scale,
            "layers": layers}


def random_weights(cfg, seed=0):
    """name -> bf16 tensor of every tensor of ``cfg``"""
    g = torch.Generator().manual_seed(seed)
    Wd, V = cfg["width"], cfg["vocab"]

    def mat(o, i, s=None):
        return torch.randn(o, i, generator=g) * (s if s is not None else i ** -0.5)

    def vec(n, mean=0.0, s=1.0):
        return mean + s * torch.randn(n, generator=g)

    W = {"embed": torch.randn(V, Wd, generator=g), "head": mat(V, Wd), "final.norm": vec(Wd, 1.0, 0.2)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        W[f"l{i}.norm1"] = vec(Wd, 1.0, 0.2)
        if L["type"] == "mamba2":
            H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            ch = H * P + 2 * G * N
            W[p + "in"] = mat(2 * H * P + 2 * G * N + H, Wd)
            W[p + "conv"], W[p + "conv.b"] = mat(ch, m["conv"], 0.5), vec(ch, 0.0, 0.2)
            W[p + "dt_bias"], W[p + "A_log"], W[p + "D"] = vec(H, -1.0, 0.5), vec(H, -0.5, 0.7), vec(H, 1.0, 0.3)
            W[p + "norm"], W[p + "o"] = vec(H * P, 1.0, 0.2), mat(Wd, H * P)
        elif L["type"] == "latent_attention":
            H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            W[p + "q"], W[p + "dkv"] = mat(H * (d + dr), Wd, 2 * Wd ** -0.5), mat(r + dr, Wd, 2 * Wd ** -0.5)
            W[p + "dkv.norm"] = vec(r, 1.0, 0.2)
            W[p + "uk"], W[p + "uv"] = mat(H * d, r), mat(H * dv, r)
            W[p + "g"], W[p + "o"] = mat(H * dv, Wd), mat(Wd, H * dv)
        else:
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[p + "q"], W[p + "q.b"], W[p + "q.norm"] = mat(H * d, Wd), vec(H * d, 0.0, 0.3), vec(H * d, 1.5, 0.3)
            if m.get("kv_from") is None:
                W[p + "k"], W[p + "k.b"], W[p + "k.norm"] = mat(G * d, Wd), vec(G * d, 0.0, 0.3), vec(G * d, 1.5, 0.3)
                W[p + "v"], W[p + "v.b"] = mat(G * dv, Wd), vec(G * dv, 0.0, 0.3)
            W[p + "sink"], W[p + "o"] = vec(H, 0.5, 1.0), mat(Wd, H * dv)
        if L["mlp"] is not None:
            q, ff = f"l{i}.mlp.", L["mlp"]["ff"]
            W[f"l{i}.norm2"] = vec(Wd, 1.0, 0.2)
            W[q + "gate"], W[q + "up"], W[q + "down"] = mat(ff, Wd), mat(ff, Wd), mat(Wd, ff)
    return {k: v.to(torch.bfloat16) for k, v in W.items()}


def random_tokens(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()
