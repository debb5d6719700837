"""Plain, slow implementation of the Nidozen hybrid decoder, written from its equations.

One function per mechanism, float64 throughout, whole sequences at once, no cache and no
batching. The tests compare the engine against it; nothing here is imported by the package.

Weights come as a dict name -> tensor with the checkpoint's names: ``embed``, ``head``,
``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
The configuration is the parsed ``config.json`` (a dict).
"""
import math

import torch

F = torch.float64


def scalar_rms_norm(y, g, eps):
    """y / sqrt(mean(y^2) + eps) * g with one gain for all coordinates."""
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * g


def weighted_rms_norm(y, w, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w


def relu2_mlp(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def mingru(h, W, p):
    """h [T, d]. Gates read the current token only; the state starts at zero."""
    z = torch.sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    u = h @ W[p + "x"].T + W[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = h @ W[p + "g"].T
    S = torch.zeros(z.shape[1], dtype=F)
    out = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        out.append(S * (g[t] * torch.sigmoid(g[t])))
    return torch.stack(out) @ W[p + "o"].T


def rotate_partial(x, base, dims):
    """x [T, heads, dim]: the first ``dims`` coordinates of every head turn by position * f_i,
    coordinate i paired with i + dims/2; the rest pass."""
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F)
    a = torch.arange(T, dtype=F)[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def attention_kv(h, W, p, m, eps):
    """Keys (normed over the whole projection, rotated) and values (unit RMS per head)."""
    T = h.shape[0]
    G, D, Dv = m["kv_heads"], m["dim"], m["vdim"]
    k = weighted_rms_norm(h @ W[p + "k"].T + W[p + "k.b"], W[p + "k.norm"], eps).view(T, G, D)
    k = rotate_partial(k, m["rot"]["base"], m["rot"]["dims"])
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, Dv)
    v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)
    return k, v


def chunked_attention(h, W, p, m, eps, kv):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = weighted_rms_norm(h @ W[p + "q"].T + W[p + "q.b"], W[p + "q.norm"], eps).view(T, H, D)
    q = rotate_partial(q, m["rot"]["base"], m["rot"]["dims"])
    k, v = kv
    C = m["mask"]["size"]
    out = torch.zeros(T, H, Dv, dtype=F)
    for i in range(T):
        lo = (i // C) * C
        for hh in range(H):
            g = hh // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hh]) * m["scale"]
            w = torch.softmax(s, 0)
            out[i, hh] = w @ v[lo:i + 1, g]
    return out.reshape(T, H * Dv) @ W[p + "o"].T + W[p + "o.b"]


def gla(h, W, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    z = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / m["tau"])).view(T, H, D)
    g = h @ W[p + "g"].T
    S = torch.zeros(H, D, Dv, dtype=F)
    out = []
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o = torch.einsum("hdv,hd->hv", S, q[t])
        out.append(weighted_rms_norm(o, W[p + "norm"], eps).reshape(H * Dv))
    o = torch.stack(out) * (g * torch.sigmoid(g))
    return o @ W[p + "o"].T


def forward(cfg, W, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    W = {k: v.to(F) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    kvs, streams = {}, []
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        if L["type"] == "mingru":
            y = mingru(x, W, p)
        elif L["type"] == "gla":
            y = gla(x, W, p, m, eps)
        elif L["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kvs[i] = attention_kv(x, W, p, m, eps)
                src = i
            y = chunked_attention(x, W, p, m, eps, kvs[src])
        else:
            raise ValueError(L["type"])
        x = x + scalar_rms_norm(y, W[f"l{i}.norm1"], eps)
        if L.get("mlp") is not None:
            y = relu2_mlp(x, W[f"l{i}.mlp.up"], W[f"l{i}.mlp.down"])
            x = x + scalar_rms_norm(y, W[f"l{i}.norm2"], eps)
        streams.append(x)
    logits = scalar_rms_norm(x, W["final.norm"], eps) @ W["head"].T
    return (logits, torch.stack(streams)) if return_layers else logits


def random_weights(cfg, seed=0, dtype=torch.bfloat16, scale=None):
    """Random tensors with the checkpoint's names and shapes (rounded to ``dtype``)."""
    gen = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def mat(n, k, s=None):
        return (torch.randn(n, k, generator=gen) * (s or (scale or 1.0) / math.sqrt(k))).to(dtype)

    def vec(n, s=0.1, mean=0.0):
        return (mean + torch.randn(n, generator=gen) * s).to(dtype)

    W = {"embed": mat(cfg["vocab"], d, 1.0), "head": mat(cfg["vocab"], d), "final.norm": vec((), 0.1, 1.0)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        W[f"l{i}.norm1"] = vec((), 0.1, 1.0)
        if L["type"] == "mingru":
            w = m["width"]
            for n in ("z", "x", "g"):
                W[p + n] = mat(w, d)
            W[p + "z.b"], W[p + "x.b"] = vec(w), vec(w)
            W[p + "o"] = mat(d, w)
        elif L["type"] == "gla":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            r = m.get("rank", 16)
            W[p + "q"], W[p + "k"] = mat(H * D, d), mat(H * D, d)
            W[p + "v"], W[p + "g"] = mat(H * Dv, d), mat(H * Dv, d)
            W[p + "a1"], W[p + "a2"], W[p + "a2.b"] = mat(r, d), mat(H * D, r), vec(H * D, 1.0, 2.0)
            W[p + "norm"] = vec(Dv, 0.1, 1.0)
            W[p + "o"] = mat(d, H * Dv)
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            W[p + "q"], W[p + "q.b"], W[p + "q.norm"] = mat(H * D, d), vec(H * D), vec(H * D, 0.1, 1.0)
            if m.get("kv_from") is None:
                W[p + "k"], W[p + "k.b"], W[p + "k.norm"] = mat(G * D, d), vec(G * D), vec(G * D, 0.1, 1.0)
                W[p + "v"], W[p + "v.b"] = mat(G * Dv, d), vec(G * Dv)
            W[p + "o"], W[p + "o.b"] = mat(d, H * Dv), vec(d)
        if L.get("mlp") is not None:
            W[f"l{i}.norm2"] = vec((), 0.1, 1.0)
            W[f"l{i}.mlp.up"], W[f"l{i}.mlp.down"] = mat(L["mlp"]["ff"], d), mat(d, L["mlp"]["ff"])
    return W
