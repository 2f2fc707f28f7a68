"""fp32 PyTorch references of the hybrid-model ops in ``ops/hybrid.py`` (CPU tensors: unit tests, CPU-only runs).

Same signatures and in-place effects as the HIP kernels of ``csrc/hybrid.hip``. Every op works on a step's flat token
rows; ``seg`` int32 [R, 4] = (first row, rows, first position, state slot) names the step's segments (one per
sequence in the step) and ``tok_seg`` int32 [T] the segment of each row. A segment whose first position is 0 starts
from zero state whatever its slot holds.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def _ln(x, w, b, eps):
    x = x.float()
    m = x.mean(-1, keepdim=True)
    d = x - m
    return d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w.float() + b.float()


def ln_shift(x, w, b, eps, out, mu=None, tok_seg=None, seg=None, state=None, last=None):
    h = _ln(x, w, b, eps)
    if mu is None:
        out.copy_(h)
        return
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    for s, (q0, n, p0, slot) in enumerate(seg.tolist()):
        prev[q0] = state[slot] if p0 > 0 else 0.0
        last[s] = h[q0 + n - 1]
    out.copy_(h + (prev - h) * mu.float())


def scatter_rows(dst, seg, src):
    dst[seg[:, 3].long()] = src[:seg.shape[0]].to(dst.dtype)


def add_ln(x, y, w, b, eps, out2=None, w2=None, b2=None):
    x += _ln(y, w, b, eps)
    if out2 is not None:
        out2.copy_(_ln(x, w2, b2, eps) if w2 is not None else x)


def gelu_mul(gu, out):
    Fh = out.shape[-1]
    g = gu.float()
    out.copy_(gelu_tanh(g[:, :Fh]) * g[:, Fh:])


def side_gate(sg, tokens, side_embed, col0, out):
    dim = out.shape[-1]
    e = side_embed[tokens.long(), col0:col0 + dim].float()
    out.copy_(gelu_tanh(sg.float()) * e)


def side_dwa(x, y, side_w, eps, stack, layer, dwa):
    if y is not None:
        yf = y.float()
        x += yf * torch.rsqrt((yf * yf).mean(-1, keepdim=True) + eps) * side_w.float()
    if stack is not None:
        stack[layer + 1].copy_(x)
        if dwa is not None:
            x.copy_((dwa.float()[:, None, None] * stack[:layer + 2]).sum(0))


def latent_prep(qgd, H, dim, rd, R, dkv_off, dkv_w, eps, positions, cos_sin, rot_dims, cache, slot_mapping, q_rot):
    """qgd [T, ...]: the fused projection's row: q heads ([dim | rd] each) first, the latent pair at ``dkv_off``
    (< 0: the layer borrows its cache). Writes [normed latent | rotated shared key] into ``cache`` rows and the
    rotated query parts into ``q_rot`` [T, H, rd]."""
    T = qgd.shape[0]
    half = rot_dims // 2
    cs = cos_sin[positions.long()]
    c, s = cs[:, :half], cs[:, half:]

    def rot(v):  # [T, ..., rd]
        shp = [T] + [1] * (v.dim() - 2) + [half]
        cc, ss = c.view(shp), s.view(shp)
        u, w = v[..., :half], v[..., half:rot_dims]
        return torch.cat([u * cc - w * ss, w * cc + u * ss, v[..., rot_dims:]], -1)

    q = qgd[:, :H * (dim + rd)].float().view(T, H, dim + rd)
    q_rot.copy_(rot(q[..., dim:]))
    if dkv_off >= 0:
        dkv = qgd[:, dkv_off:dkv_off + R + rd].float()
        lat = dkv[:, :R]
        lat = lat * torch.rsqrt((lat * lat).mean(-1, keepdim=True) + eps) * dkv_w.float()
        row = torch.cat([lat, rot(dkv[:, R:])], -1).to(cache.dtype)
        ok = slot_mapping >= 0
        cache.view(-1, R + rd)[slot_mapping[ok].long()] = row[ok]


def latent_attn(q_lat, q_rot, cache, block_tables, tok_seg, seg, positions, scale, out):
    """q_lat [H, T, R], q_rot [T, H, rd], cache [pages, page, R + rd]; out [H, T, R] = softmax-weighted latents."""
    H, T, R = q_lat.shape
    page = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1]).float()
    for t in range(T):
        r = int(tok_seg[t])
        n = int(positions[t]) + 1
        pages = block_tables[r, :(n + page - 1) // page].long()
        idx = (pages[:, None] * page + torch.arange(page)[None]).reshape(-1)[:n]
        kv = flat[idx]
        s = (q_lat[:, t].float() @ kv[:, :R].T + q_rot[t].float() @ kv[:, R:].T) * scale
        out[:, t] = (torch.softmax(s, -1) @ kv[:, :R]).to(out.dtype)


def sigmoid_mul(a, g, out):
    """a [H, T, v] (head-major), g [T, H * v] -> out [T, H * v]."""
    H, T, v = a.shape
    out.copy_(a.float().permute(1, 0, 2).reshape(T, H * v) * torch.sigmoid(g.float()))


def conv_silu(proj, c0, w, b, tok_seg, seg, state, out):
    C, taps = w.shape
    u = proj[:, c0:c0 + C].float()
    for q0, n, p0, slot in seg.tolist():
        hist = state[slot].float() if p0 > 0 else torch.zeros(taps - 1, C)
        full = torch.cat([hist, u[q0:q0 + n]], 0)
        acc = b.float().expand(n, C).clone()
        for k in range(taps):
            acc = acc + full[k:k + n] * w[:, k].float()
        out[q0:q0 + n] = F.silu(acc).to(out.dtype)
        state[slot] = full[n:].to(state.dtype)


def ssm_scan(xbc, proj, dt_off, dt_bias, A_log, D, heads, P, N, G, tok_seg, seg, state, y):
    """xbc [T, heads * P + 2 G N] (after conv + silu), raw dt at proj[:, dt_off + h]; state f32 [slots, heads, N, P]."""
    inner = heads * P
    grp = torch.arange(heads) // (heads // G)
    A = -torch.exp(A_log.float())
    for q0, n, p0, slot in seg.tolist():
        S = state[slot].clone() if p0 > 0 else torch.zeros(heads, N, P)
        for t in range(q0, q0 + n):
            x = xbc[t, :inner].float().view(heads, P)
            B = xbc[t, inner:inner + G * N].float().view(G, N)[grp]
            C = xbc[t, inner + G * N:].float().view(G, N)[grp]
            dt = F.softplus(proj[t, dt_off:dt_off + heads].float() + dt_bias.float(), threshold=1e9)
            S = torch.exp(A * dt)[:, None, None] * S + (dt[:, None] * B)[:, :, None] * x[:, None, :]
            y[t] = (torch.einsum("hnp,hn->hp", S, C) + D.float()[:, None] * x).reshape(-1)
        state[slot] = S


def gated_norm(y, proj, w, groups, eps, out):
    T, inner = y.shape
    v = y.float() * F.silu(proj[:, :inner].float())
    v = v.view(T, groups, inner // groups)
    v = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps)
    out.copy_(v.reshape(T, inner) * w.float())
