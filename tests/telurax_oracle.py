"""Plain, slow implementation of the Telurax hybrid decoder, written from its equations.

One function per mechanism, float64 throughout, whole sequences at once, no cache and no
batching. The tests compare the engine against it; nothing here is imported by the package and
nothing of the package is imported here.

Weights come as a dict name -> tensor with the checkpoint's names: ``embed``, ``head``,
``final.norm``, and per layer i ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``.
The configuration is the parsed ``config.json`` (a dict).
"""
import math

import torch

F = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """The layer norm of the design: the stored weight is the distance from one."""
    return unit_rms(x, eps) * (1.0 + w)


def position_vectors(T, d):
    out = torch.zeros(T, d, dtype=F)
    for p in range(T):
        for i in range(d // 2):
            a = p * 10000.0 ** (-2.0 * i / d)
            out[p, 2 * i], out[p, 2 * i + 1] = math.sin(a), math.cos(a)
    return out


def latent_attention(h, W, p, m, eps):
    """Every head's keys and values are linear maps of ONE normed low-rank row per token; full causal
    softmax; a scalar gate per head."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, D)
    c = unit_rms(h @ W[p + "dkv"].T, eps) * W[p + "dkv.norm"]
    k = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, Dv)
    gate = torch.sigmoid(h @ W[p + "g"].T)                      # [T, H]
    out = torch.zeros(T, H, Dv, dtype=F)
    for i in range(T):
        for hh in range(H):
            s = (k[:i + 1, hh] @ q[i, hh]) * m["scale"]
            out[i, hh] = (torch.softmax(s, 0) @ v[:i + 1, hh]) * gate[i, hh]
    return out.reshape(T, H * Dv) @ W[p + "o"].T


def soft_cap(x, cap):
    return cap * torch.tanh(x / cap) if cap else x


def mlstm(h, W, p, m, eps):
    """Matrix memory with exponential input gate, stabilised by a running maximum that starts at 0."""
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m.get("gate_cap", 0.0)
    q = (h @ W[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    li = soft_cap(h @ W[p + "i"].T + W[p + "i.b"], cap)
    lf = torch.nn.functional.logsigmoid(soft_cap(h @ W[p + "f"].T + W[p + "f.b"], cap))
    S = torch.zeros(H, D, Dv, dtype=F)
    n = torch.zeros(H, D, dtype=F)
    mx = torch.zeros(H, dtype=F)
    rows = []
    for t in range(T):
        new = torch.maximum(lf[t] + mx, li[t])
        keep, take = torch.exp(lf[t] + mx - new), torch.exp(li[t] - new)
        S = keep[:, None, None] * S + take[:, None, None] * (k[t][:, :, None] * v[t][:, None, :])
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        rows.append(unit_rms(num / den[:, None], eps).reshape(H * Dv))
    o = torch.stack(rows) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def gated_relu_mlp(h, W, p):
    return (torch.relu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def relu2_expert(h, W, p):
    return torch.relu(h @ W[p + "up"].T) ** 2 @ W[p + "down"].T


def route(h, W, p, r, use_groups=True, use_correction=True):
    """(chosen outputs [T, top], their weights [T, top]) of the router."""
    n = r["experts"] + r.get("identity", 0)
    s = torch.softmax(h @ W[p + "router"].T, -1)
    choice = s + W[p + "correction"] if use_correction else s.clone()
    g = r.get("groups") or {"count": 1, "keep": 1}
    if use_groups and g["keep"] < g["count"]:
        size = n // g["count"]
        for t in range(h.shape[0]):
            best = sorted(range(g["count"]), key=lambda j: -float(choice[t, j * size:(j + 1) * size].max()))[:g["keep"]]
            for j in range(g["count"]):
                if j not in best:
                    choice[t, j * size:(j + 1) * size] = -math.inf
    ids = torch.topk(choice, r["top"], -1).indices
    return ids, s.gather(1, ids) * r.get("scale", 1.0)


def routed_mlp(h, W, p, mlp):
    r = mlp["router"]
    ids, wts = route(h, W, p, r)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), wts[t]):
            out[t] += w * (relu2_expert(h[t:t + 1], W, p + f"e{e}.")[0] if e < r["experts"] else h[t])
    if mlp.get("shared"):
        out = out + relu2_expert(h, W, p + "shared.")
    return out


def forward(cfg, W, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the residual stream after every layer)."""
    W = {k: v.to(F) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg.get("embedding", {}).get("scale", 1.0)
    x = x + position_vectors(T, cfg["width"])
    streams = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = offset_norm(x, W[p + "norm1"], eps)
        mix = {"latent_attention": latent_attention, "mlstm": mlstm}[L["type"]]
        x = x + mix(h, W, p + "mix.", L["mixer"], eps)
        mlp = L.get("mlp")
        if mlp is not None:
            h = offset_norm(x, W[p + "norm2"], eps)
            x = x + (gated_relu_mlp(h, W, p + "mlp.") if mlp["kind"] == "dense" else routed_mlp(h, W, p + "mlp.", mlp))
        streams.append(x)
    logits = offset_norm(x, W["final.norm"], eps) @ W["head"].T * cfg.get("logit_scale", 1.0)
    return (logits, torch.stack(streams)) if return_layers else logits


def random_weights(cfg, seed=0, dtype=torch.bfloat16, router_gain=4.0):
    """Random tensors with the checkpoint's names and shapes (rounded to ``dtype``). The router's
    rows are ``router_gain`` times larger than the others so that its choices are clear-cut."""
    gen = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def mat(n, k, s=None):
        return (torch.randn(n, k, generator=gen) * (s or 1.0 / math.sqrt(k))).to(dtype)

    def vec(n, s=0.1, mean=0.0):
        return (mean + torch.randn(n, generator=gen) * s).to(dtype)

    W = {"embed": mat(cfg["vocab"], d, 1.0), "head": mat(cfg["vocab"], d), "final.norm": vec(d)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", L["mixer"]
        W[f"l{i}.norm1"] = vec(d)
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        if L["type"] == "latent_attention":
            R = m["kv_rank"]
            W[p + "q"], W[p + "dkv"], W[p + "dkv.norm"] = mat(H * D, d), mat(R, d), vec(R, 0.1, 1.0)
            W[p + "uk"], W[p + "uv"] = mat(H * D, R), mat(H * Dv, R)
            W[p + "g"], W[p + "o"] = mat(H, d), mat(d, H * Dv)
        else:
            W[p + "q"], W[p + "k"] = mat(H * D, d), mat(H * D, d)
            W[p + "v"], W[p + "g"] = mat(H * Dv, d), mat(H * Dv, d)
            W[p + "o"], W[p + "norm"] = mat(d, H * Dv), vec(H * Dv, 0.1, 1.0)
            W[p + "i"], W[p + "i.b"] = mat(H, d), vec(H, 0.5)
            W[p + "f"], W[p + "f.b"] = mat(H, d), vec(H, 1.0, 2.0)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        f = f"l{i}.mlp."
        W[f"l{i}.norm2"] = vec(d)
        if mlp["kind"] == "dense":
            W[f + "gate"], W[f + "up"], W[f + "down"] = mat(mlp["ff"], d), mat(mlp["ff"], d), mat(d, mlp["ff"])
            continue
        r = mlp["router"]
        n = r["experts"] + r.get("identity", 0)
        for e in range(r["experts"]):
            W[f + f"e{e}.up"], W[f + f"e{e}.down"] = mat(mlp["expert"]["ff"], d), mat(d, mlp["expert"]["ff"])
        W[f + "router"] = mat(n, d, router_gain / math.sqrt(d))
        W[f + "correction"] = vec(n, 0.05)
        if mlp.get("shared"):
            W[f + "shared.up"], W[f + "shared.down"] = mat(mlp["shared"]["ff"], d), mat(d, mlp["shared"]["ff"])
    return W
