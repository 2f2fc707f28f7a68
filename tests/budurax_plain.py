"""Plain, slow Budurax forward for the tests: one function per mechanism, whole sequences only, no cache, no state
carried between calls, float64 by default. It shares nothing with the package: the engine's chunked, paged and batched
results are compared with what these functions give for the whole token list at once.

``cfg`` is the model's config.json as a dict, ``W`` maps tensor names to torch tensors.
"""
from __future__ import annotations

import math

import torch


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    m = x.mean(-1, keepdim=True)
    d = x - m
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


def token_shift(h, mu):
    """h [T, d]: every row moves towards the row before it (zeros before the first) by the per-channel factor mu."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def rotary_tables(n_pos, rot):
    """cos / sin [n_pos, dims / 2] of the rotate-half rotary embedding with optional YaRN frequency blending."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def corr(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(corr(float(sc["fast"]))), 0)
        hi = min(math.ceil(corr(float(sc["slow"]))), dims - 1)
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(n_pos, dtype=torch.float64)[:, None] * torch.tensor(f, dtype=torch.float64)[None]
    return torch.cos(ang) * mag, torch.sin(ang) * mag


def rotate(x, cos, sin, dims):
    """x [T, ..., D]: the first ``dims`` entries are rotated pairwise (i with i + dims / 2), the rest pass."""
    half = dims // 2
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = cos.view(shape).to(x.dtype), sin.view(shape).to(x.dtype)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def latent_kv(h, W, p, m, eps):
    """The cached pair of a latent-attention layer: normed latent c [T, kv_rank] and rotated shared key [T, rot_dim]."""
    r, rd = int(m["kv_rank"]), int(m["rot_dim"])
    dkv = h @ W[p + "dkv"].T
    c = rms_unit(dkv[:, :r], eps) * W[p + "dkv.norm"]
    cos, sin = rotary_tables(h.shape[0], m["rot"])
    return c, rotate(dkv[:, r:r + rd], cos, sin, int(m["rot"]["dims"]))


def latent_attention(h, W, p, m, eps, kv=None):
    """``kv`` = (c, k_rot) of the layer this one borrows from (its own when None)."""
    T = h.shape[0]
    H, D, rd, vd = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
    c, kr = kv if kv is not None else latent_kv(h, W, p, m, eps)
    q = (h @ W[p + "q"].T).view(T, H, D + rd)
    cos, sin = rotary_tables(T, m["rot"])
    qu, qr = q[..., :D], rotate(q[..., D:], cos, sin, int(m["rot"]["dims"]))
    ku = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, vd)
    s = (torch.einsum("thd,shd->hts", qu, ku) + torch.einsum("thd,sd->hts", qr, kr)) * float(m["scale"])
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    s = s.masked_fill(~mask[None], float("-inf"))
    o = torch.einsum("hts,shd->thd", torch.softmax(s, -1), v).reshape(T, H * vd)
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T, (c, kr)


def causal_conv(u, w, b):
    """u [T, C], w [C, taps] (last column = current token), zeros before the start."""
    T, taps = u.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u], 0)
    out = b.expand(T, -1).clone()
    for k in range(taps):
        out = out + pad[k:k + T] * w[:, k]
    return out


def mamba2(h, W, p, m, eps):
    T = h.shape[0]
    Hh, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = Hh * P
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].view(T, Hh, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.nn.functional.softplus(dt + W[p + "dt_bias"], threshold=1e9)
    A = -torch.exp(W[p + "A_log"])
    S = torch.zeros(Hh, N, P, dtype=h.dtype)
    y = torch.zeros(T, Hh, P, dtype=h.dtype)
    grp = torch.arange(Hh) // (Hh // G)
    for t in range(T):
        Bt, Ct = B[t][grp], C[t][grp]                      # [heads, N]
        S = torch.exp(A * dt[t])[:, None, None] * S + dt[t][:, None, None] * Bt[:, :, None] * x[t][:, None, :]
        y[t] = torch.einsum("hnp,hn->hp", S, Ct) + W[p + "D"][:, None] * x[t]
    y = y.reshape(T, inner) * silu(z)
    ng = int(m["norm_groups"])
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def dense_ff(h, W, p):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def token_side(x, tokens, W, i, dim, eps):
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e
    y = g @ W[f"l{i}.side.proj"].T
    return x + rms_unit(y, eps) * W[f"l{i}.side.norm"]


def forward(cfg, W, tokens, dtype=torch.float64, return_layers=False):
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    eps = float(cfg["norm"]["eps"])

    def norm(x, name):
        return layer_norm(x, W[name], W[name + ".b"], eps)

    x = W["embed"][tokens]
    outs, kvs, layers = [x], {}, []
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = norm(x, p + "norm1")
        if p + "shift" in W:
            h = token_shift(h, W[p + "shift"])
        if L["type"] == "latent_attention":
            src = m.get("kv_from")
            y, kvs[i] = latent_attention(h, W, p + "mix.", m, eps, kvs[src] if src is not None else None)
        elif L["type"] == "mamba2":
            y = mamba2(h, W, p + "mix.", m, eps)
        else:
            raise ValueError(L["type"])
        x = x + norm(y, p + "norm1b")
        if L.get("mlp") is not None:
            x = x + norm(dense_ff(norm(x, p + "norm2"), W, p + "mlp."), p + "norm2b")
        if cfg.get("token_side") and "side.embed" in W:
            x = token_side(x, tokens, W, i, int(cfg["token_side"]["dim"]), eps)
        outs.append(x)
        if p + "dwa" in W:
            a = W[p + "dwa"]
            x = sum(a[j] * outs[j] for j in range(i + 2))
        layers.append(x)
    logits = norm(x, "final.norm") @ W["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits
