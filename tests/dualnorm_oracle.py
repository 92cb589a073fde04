"""Plain float64 forms of a decoder of two-norm parallel blocks (Zoguzen
layout), written from the equations alone: whole sequences, explicit loops
over time, no cache, no batching.  Shares no code with the framework.

A model is ``(cfg, W)``: the configuration dictionary a checkpoint's
``config.json`` holds and ``name -> float64 tensor``.

Block:  x <- x + mixer(shift(LN1(x))) + ff(LN2(x)),  then the token-side
input.  shift(h)_t = h_t + (h_(t-1) - h_t) * mu  (h_(-1) = 0).
"""
import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------ small pieces
def layer_norm(x, w, eps):
    d = x - x.mean(-1, keepdim=True)
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def token_shift(h, mu):
    out = torch.empty_like(h)
    prev = torch.zeros_like(h[0])
    for t in range(h.shape[0]):
        out[t] = h[t] + (prev - h[t]) * mu
        prev = h[t]
    return out


def causal_conv(u, w):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start"""
    T, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def rotary_freqs(rot):
    """frequencies of the pairs, with the wavelength-dependent scaling: short waves kept, long waves divided by
    the factor, a linear blend between"""
    dims = int(rot["dims"])
    f = [float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if sc:
        factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
        out = []
        for fi in f:
            wl = 2.0 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = out
    return torch.tensor(f, dtype=F64)


def turn_pairs(x, rot, positions):
    """x [T, heads, d]: value 2i is paired with 2i + 1 on the first rot.dims values"""
    dims = int(rot["dims"])
    a = positions.to(F64)[:, None] * rotary_freqs(rot)[None]          # [T, dims / 2]
    c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ------------------------------------------------------------------ mixers
def mingru(W, p, m, h):
    z = sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    u = h @ W[p + "x"].T + W[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, sigmoid(u))
    g = silu(h @ W[p + "g"].T)
    S = torch.zeros(int(m["width"]), dtype=F64)
    out = torch.empty_like(z)
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        out[t] = S * g[t]
    return out @ W[p + "o"].T


def visible(i, j, mask, chunked):
    if j > i:
        return False
    size = int(mask["size"])
    if chunked:
        return i // size == j // size
    return i - j < size or j < int(mask.get("keep_first", 0))


def window_attention(W, p, m, h):
    """grouped heads, short convolutions, rotation, a window that keeps the first tokens, sigmoid gate"""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = causal_conv(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, H, d)
    k = causal_conv(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, d)
    v = causal_conv(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, G, dv)
    if m.get("rot"):
        q, k = turn_pairs(q, m["rot"], pos), turn_pairs(k, m["rot"], pos)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, m["mask"], False)]
            s = (k[js, g] @ q[i, hd]) * float(m["scale"])
            out[i, hd] = torch.softmax(s, 0) @ v[js, g]
    o = out.reshape(T, H * dv) * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def linear_attention(W, p, m, h, eps):
    """per head S <- diag(alpha) S + k v^T, o = S^T q with a decay per key channel"""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / float(m["tau"]))).view(T, H, d)
    S = torch.zeros(H, d, dv, dtype=F64)
    o = torch.empty(T, H, dv, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = (S * q[t][:, :, None]).sum(1)
    o = unit_rms(o, eps) * W[p + "norm"]
    return (o.reshape(T, H * dv) * silu(h @ W[p + "g"].T)) @ W[p + "o"].T


def side_by_side(W, p, m, h, eps):
    a = window_attention(W, p + "left.", m["left"], h)
    b = linear_attention(W, p + "right.", m["right"], h, eps)
    return 0.5 * (unit_rms(a, eps) * W[p + "left.out"] + unit_rms(b, eps) * W[p + "right.out"])


def attention_keys(W, p, m, h, eps):
    T = h.shape[0]
    G, d, dv = int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    k = causal_conv(h @ W[p + "k"].T + W[p + "k.b"], W[p + "k.conv"]).view(T, G, d)
    v = causal_conv(h @ W[p + "v"].T + W[p + "v.b"], W[p + "v.conv"]).view(T, G, dv)
    return unit_rms(k, eps) * W[p + "k.norm"], v


def chunk_attention(W, p, m, h, eps, kv):
    """chunks counted from position 0, capped scores, a sink of score 0, the heads' weights mixed afterwards"""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = causal_conv(h @ W[p + "q"].T + W[p + "q.b"], W[p + "q.conv"]).view(T, H, d)
    q = unit_rms(q, eps) * W[p + "q.norm"]
    k, v = kv
    cap = float(m.get("softcap") or 0.0)
    wts = torch.zeros(H, T, T, dtype=F64)
    for hd in range(H):
        g = hd // (H // G)
        for i in range(T):
            js = [j for j in range(i + 1) if visible(i, j, m["mask"], True)]
            s = (k[js, g] @ q[i, hd]) * float(m["scale"])
            if cap:
                s = cap * torch.tanh(s / cap)
            e = torch.exp(s)
            wts[hd, i, js] = e / (1.0 + e.sum())
    mixed = torch.einsum("hg,gij->hij", W[p + "talk"], wts)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        out[:, hd] = mixed[hd] @ v[:, hd // (H // G)]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def experts(W, p, m, h):
    E, top = int(m["router"]["experts"]), int(m["router"]["top"])
    z = h @ W[p + "router"].T
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(z[t, order], 0)
        for wk, e in zip(w, order):
            q = f"{p}e{e}."
            y = silu(W[q + "gate"] @ h[t]) * (W[q + "up"] @ h[t])
            out[t] += wk * (W[q + "down"] @ y)
    return out


# ------------------------------------------------------------------ model
def forward(cfg, W, tokens, layers_out=None):
    """logits f64 [T, vocab] of one sequence run whole"""
    eps = float(cfg["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = W["embed"][ids].clone()
    side = int((cfg.get("token_side") or {}).get("dim", 0))
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = token_shift(layer_norm(x, W[p + "norm1"], eps), W[p + "shift"])
        if L["type"] == "mingru":
            y = mingru(W, p + "mix.", m, h)
        elif L["type"] == "parallel":
            y = side_by_side(W, p + "mix.", m, h, eps)
        elif L["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = attention_keys(W, p + "mix.", m, h, eps)
            y = chunk_attention(W, p + "mix.", m, h, eps, kvs[i if src is None else int(src)])
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            y = y + experts(W, p + "mlp.", L["mlp"], layer_norm(x, W[p + "norm2"], eps))
        x = x + y
        if side:
            e = W["side.embed"][ids, i * side:(i + 1) * side]
            g = gelu_tanh(x @ W[p + "side.gate"].T) * e
            x = x + unit_rms(g @ W[p + "side.proj"].T, eps) * W[p + "side.norm"]
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = layer_norm(x, W["final.norm"], eps) @ W["embed"].T
    cap = float(cfg.get("logit_softcap") or 0.0)
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(cfg, W, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, W, toks)[-1].argmax()))
    return toks[len(prompt):]


# ------------------------------------------------------------------ configurations and weights
def moe(experts=5, top=2, ff=12):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def attn_layer(heads=4, kv_heads=2, dim=12, vdim=10, chunk=7, taps=3, scale=0.3, softcap=5.0, kv_from=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps, "mask": {"size": chunk},
         "scale": scale, "softcap": softcap}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp}


def gru_layer(width=24, mlp=None):
    return {"type": "mingru", "mixer": {"width": width}, "mlp": mlp}


def pair_layer(heads=4, kv_heads=2, dim=12, vdim=10, window=9, keep=2, taps=2, dims=8, base=3000.0, scaling=None,
               scale=0.3, rheads=3, rdim=6, rvdim=10, tau=4.0, mlp=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps,
            "mask": {"size": window, "keep_first": keep},
            "rot": {"dims": dims, "base": base, "scaling": scaling}, "scale": scale}
    if scaling is None:
        del left["rot"]["scaling"]
    right = {"heads": rheads, "dim": rdim, "vdim": rvdim, "tau": tau}
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def config(layers, vocab=89, width=40, eps=1e-5, side=6, logit_softcap=8.0):
    cfg = {"architecture": "Zoguzen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
           "logit_softcap": logit_softcap}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def tensor_shapes(cfg):
    Wd, V = int(cfg["width"]), int(cfg["vocab"])
    side = int((cfg.get("token_side") or {}).get("dim", 0))
    out = {"embed": (V, Wd)}
    if side:
        out["side.embed"] = (V, side * len(cfg["layers"]))
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = (Wd,)
        out[p + "shift"] = (Wd,)
        if L["type"] == "mingru":
            n = m["width"]
            out.update({p + "mix.z": (n, Wd), p + "mix.z.b": (n,), p + "mix.x": (n, Wd), p + "mix.x.b": (n,),
                        p + "mix.g": (n, Wd), p + "mix.o": (Wd, n)})
        elif L["type"] == "attention":
            H, G, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            out.update({p + "mix.q": (H * d, Wd), p + "mix.q.b": (H * d,), p + "mix.q.norm": (d,),
                        p + "mix.q.conv": (H * d, taps), p + "mix.talk": (H, H), p + "mix.o": (Wd, H * dv)})
            if m.get("kv_from") is None:
                out.update({p + "mix.k": (G * d, Wd), p + "mix.k.b": (G * d,), p + "mix.k.norm": (d,),
                            p + "mix.k.conv": (G * d, taps), p + "mix.v": (G * dv, Wd), p + "mix.v.b": (G * dv,),
                            p + "mix.v.conv": (G * dv, taps)})
        else:
            a, b = m["left"], m["right"]
            H, G, d, dv, taps = a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["conv"]
            q = p + "mix.left."
            out.update({q + "q": (H * d, Wd), q + "k": (G * d, Wd), q + "v": (G * dv, Wd), q + "q.conv": (H * d, taps),
                        q + "k.conv": (G * d, taps), q + "v.conv": (G * dv, taps), q + "g": (H * dv, Wd),
                        q + "o": (Wd, H * dv), q + "out": (Wd,)})
            H, d, dv = b["heads"], b["dim"], b["vdim"]
            q = p + "mix.right."
            rank = b.get("rank", 4)
            out.update({q + "q": (H * d, Wd), q + "k": (H * d, Wd), q + "v": (H * dv, Wd), q + "g": (H * dv, Wd),
                        q + "o": (Wd, H * dv), q + "norm": (dv,), q + "a1": (rank, Wd), q + "a2": (H * d, rank),
                        q + "a2.b": (H * d,), q + "out": (Wd,)})
        if L.get("mlp") is not None:
            out[p + "norm2"] = (Wd,)
            ff, E = L["mlp"]["expert"]["ff"], L["mlp"]["router"]["experts"]
            for e in range(E):
                out.update({f"{p}mlp.e{e}.gate": (ff, Wd), f"{p}mlp.e{e}.up": (ff, Wd), f"{p}mlp.e{e}.down": (Wd, ff)})
            out[p + "mlp.router"] = (E, Wd)
        if side:
            out.update({p + "side.gate": (side, Wd), p + "side.proj": (Wd, side), p + "side.norm": (Wd,)})
    out["final.norm"] = (Wd,)
    return out


def random_weights(cfg, seed=0):
    """bf16-representable float64 weights"""
    g = torch.Generator().manual_seed(seed)
    W = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(("norm1", "norm2", "final.norm", ".norm", ".out")):
            w = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif name.endswith("shift"):
            w = torch.rand(shape, generator=g)
        elif name.endswith("talk"):
            w = torch.eye(shape[0]) + 0.3 * torch.randn(shape, generator=g)
        elif name.endswith(".conv"):
            w = 0.6 * torch.randn(shape, generator=g)
        elif name.endswith("a2.b"):
            w = 2.0 + torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            w = 0.3 * torch.randn(shape, generator=g)
        elif name.endswith("router"):
            w = torch.randn(shape, generator=g)
        elif name in ("embed", "side.embed"):
            w = torch.randn(shape, generator=g)
        else:
            w = torch.randn(shape, generator=g) * 1.5 * shape[1] ** -0.5
        W[name] = w.to(torch.bfloat16).to(F64)
    return W


def random_tokens(cfg, n, seed=0):
    g = torch.Generator().manual_seed(1000 + seed)
    return torch.randint(0, int(cfg["vocab"]), (n,), generator=g).tolist()
