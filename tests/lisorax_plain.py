"""Plain, slow Lisorax forward for the tests: one function per mechanism, whole sequences only, no cache, no state
carried between calls, float64 by default. It shares nothing with the package: the engine's chunked, paged and batched
results are compared with what these functions give for the whole token list at once.

``cfg`` is the model's config.json as a dict, ``W`` maps tensor names to torch tensors.
"""
from __future__ import annotations

import math

import torch


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_conv(u, w, b=None):
    """u [T, C], w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j) with zeros before the first row; the last
    column of w multiplies the row itself."""
    T, taps = u.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], 0)
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    return y if b is None else y + b


def attention_kv(h, W, p):
    """Keys and values of an attention layer that owns them: projections, then the short convolution."""
    k = causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])
    v = causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])
    return k, v


def query_temperature(T, m):
    qt = m.get("q_temp")
    if not qt:
        return torch.ones(T, dtype=torch.float64)
    pos = torch.arange(T, dtype=torch.float64)
    return 1.0 + float(qt["coef"]) * torch.log(torch.floor((pos + 1.0) / float(qt["every"])) + 1.0)


def sigmoid_attention(h, W, p, m, kv=None):
    """Causal attention without softmax: every visible key weighs sigmoid(capped score - distance bias + head bias),
    weights are not normalised. ``kv``: the (keys, values) of the layer this one borrows, its own when None."""
    T = h.shape[0]
    H, G, D, Dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])
    k, v = kv if kv is not None else attention_kv(h, W, p)
    q = (q * query_temperature(T, m).to(q.dtype)[:, None]).view(T, H, D)
    k, v = k.view(T, G, D), v.view(T, G, Dv)
    i = torch.arange(T)
    dist = (i[:, None] - i[None, :]).clamp(min=0).to(q.dtype)
    visible = i[None, :] <= i[:, None]
    cap = float(m.get("softcap") or 0.0)
    outs = []
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * float(m["scale"])
        if cap:
            s = cap * torch.tanh(s / cap)
        s = s - W[p + "r1"][hd] * torch.log1p(W[p + "r2"][hd] * dist)
        w = torch.sigmoid(s + W[p + "pb"][hd]) * visible
        outs.append(w @ v[:, g])
    return torch.cat(outs, -1) @ W[p + "o"].T


def rglru(h, W, p, m):
    """Two branches: gelu(W_y h + b) and a convolved W_x h + b that drives a gated diagonal linear recurrence."""
    T = h.shape[0]
    Wd, nb = int(m["width"]), int(m["blocks"])
    y = gelu_tanh(h @ W[p + "y"].T + W[p + "y.b"])
    u = causal_conv(h @ W[p + "x"].T + W[p + "x.b"], W[p + "conv"], W[p + "conv.b"])
    ub = u.view(T, nb, Wd // nb)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", W[p + "ra"], ub) + W[p + "ra.b"]).reshape(T, Wd)
    ig = torch.sigmoid(torch.einsum("boi,tbi->tbo", W[p + "ri"], ub) + W[p + "ri.b"]).reshape(T, Wd)
    log_a = -8.0 * r * torch.nn.functional.softplus(W[p + "lam"])
    a = torch.exp(log_a)
    inp = torch.sqrt(1.0 - a * a) * ig * u
    S = torch.zeros(Wd, dtype=h.dtype)
    out = []
    for t in range(T):
        S = a[t] * S + inp[t]
        out.append(S * y[t])
    return torch.stack(out) @ W[p + "o"].T


def mlstm(h, W, p, m, eps):
    """Matrix memory per head with exponential input gate, sigmoid forget gate and a running maximum that starts at 0."""
    T = h.shape[0]
    H, D, Dv, cap = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"])
    q = (h @ W[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    n = torch.zeros(H, D, dtype=h.dtype)
    mx = torch.zeros(H, dtype=h.dtype)
    rows = []
    for t in range(T):
        m_new = torch.maximum(fg[t] + mx, ig[t])
        decay = torch.exp(fg[t] + mx - m_new)
        gain = torch.exp(ig[t] - m_new)
        S = decay[:, None, None] * S + gain[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = decay[:, None] * n + gain[:, None] * k[t]
        mx = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        rows.append(rms_unit(num / den[:, None], eps).reshape(H * Dv))
    o = torch.stack(rows) * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def moe(h, W, p, mlp):
    """Each row uses the ``top`` experts with the largest router logits, weighted by a softmax over those logits only."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ W[p + "router"].T + W[p + "router.b"]
    val, idx = torch.topk(z, top, dim=-1)
    wt = torch.softmax(val, -1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            assert 0 <= e < E
            g = h[t] @ W[f"{p}e{e}.gate"].T
            a = g * torch.sigmoid(g) * (h[t] @ W[f"{p}e{e}.up"].T)
            out[t] += wt[t, j] * (a @ W[f"{p}e{e}.down"].T)
    return out


def forward(cfg: dict, W: dict, tokens: list[int], dtype=torch.float64, layers_out: list | None = None):
    """Logits [T, vocab] of one whole sequence."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)] * float(cfg["embedding"]["scale"])
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = rms_unit(x, eps) * W[p + "norm1"]
        hm = h + causal_conv(h, W[p + "canon1"]) if cfg.get("canon") else h
        if L["type"] == "attention":
            if m.get("kv_from") is None:
                kvs[i] = attention_kv(hm, W, p + "mix.")
                y = sigmoid_attention(hm, W, p + "mix.", m, kvs[i])
            else:
                y = sigmoid_attention(hm, W, p + "mix.", m, kvs[int(m["kv_from"])])
        elif L["type"] == "rglru":
            y = rglru(hm, W, p + "mix.", m)
        elif L["type"] == "mlstm":
            y = mlstm(hm, W, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            y = y + moe(h, W, p + "mlp.", L["mlp"])
        x = x + y
        if layers_out is not None:
            layers_out.append(x.clone())
    return (rms_unit(x, eps) * W["final.norm"]) @ W["embed"].T
