"""Ops of the hybrid decoder family (layer norm, token shift, latent attention, Mamba-2, depth average): GPU tensors
run the HIP kernels of ``csrc/hybrid.hip``, CPU tensors the fp32 references of ``hybrid_reference.py``.

Activations are bf16 or fp32 (the model's dtype, the kernels are built for both); the residual stream, recurrent
state, norms, softmax and every gate of a recurrence are fp32 in both. A step's rows are described by ``seg`` int32
[R, 4] = (first row, rows, first position, state slot) and ``tok_seg`` int32 [T] (see hybrid_reference.py).
"""
from __future__ import annotations

import torch

from . import hybrid_reference as ref
from ._ext import ext

SCAN_MAX_TAPS = 8


def _gpu(t: torch.Tensor) -> bool:
    return t.is_cuda


def ln_shift(x, w, b, eps, out, mu=None, tok_seg=None, seg=None, state=None, last=None) -> None:
    """out = layer_norm(x) (x fp32 [T, d]); with ``mu`` each row is then moved towards the previous row's normed
    value (the slot's ``state`` row for a segment's first row) by mu, and every segment's last normed row lands in
    ``last`` [R, d] (``scatter_rows`` stores it once all rows have read the old state)."""
    if _gpu(x):
        ext().hy_ln_shift(x, w, b, float(eps), out, mu, tok_seg, seg, state, last)
    else:
        ref.ln_shift(x, w, b, eps, out, mu, tok_seg, seg, state, last)


def scatter_rows(dst, seg, src) -> None:
    """dst[seg[r].slot] = src[r]."""
    if _gpu(dst):
        ext().hy_scatter_rows(dst, seg, src)
    else:
        ref.scatter_rows(dst, seg, src)


def add_ln(x, y, w, b, eps, out2=None, w2=None, b2=None) -> None:
    """x += layer_norm(y; w, b) in place (x fp32); with ``out2`` also out2 = layer_norm(x; w2, b2), or the new x in
    out2's dtype when no second norm is given."""
    if _gpu(x):
        ext().hy_add_ln(x, y, w, b, float(eps), out2, w2, b2)
    else:
        ref.add_ln(x, y, w, b, eps, out2, w2, b2)


def gelu_mul(gu, out) -> None:
    """out = gelu_tanh(gu[:, :F]) * gu[:, F:]."""
    if _gpu(gu):
        ext().hy_gelu_mul(gu, out)
    else:
        ref.gelu_mul(gu, out)


def side_gate(sg, tokens, side_embed, col0: int, out) -> None:
    """out = gelu_tanh(sg) * side_embed[token, col0 : col0 + dim]."""
    if _gpu(sg):
        ext().hy_side_gate(sg, tokens, side_embed, int(col0), out)
    else:
        ref.side_gate(sg, tokens, side_embed, col0, out)


def side_dwa(x, y, side_w, eps, stack, layer: int, dwa) -> None:
    """x += y / rms(y) * side_w (when y is given); stack[layer + 1] = x; with ``dwa`` x = sum_j dwa[j] stack[j]."""
    if _gpu(x):
        ext().hy_side_dwa(x, y, side_w, float(eps), stack, int(layer), dwa)
    else:
        ref.side_dwa(x, y, side_w, eps, stack, layer, dwa)


def latent_prep(qgd, H, dim, rd, R, dkv_off, dkv_w, eps, positions, cos_sin, rot_dims, cache, slot_mapping,
                q_rot, cache_t=None) -> None:
    """RMS norm of the latent and rotary on the shared key part of the fused projection row -> the row's cache slot
    ([latent | rotated key]; with ``cache_t`` [pages, kv_rank, page] also the latent page-wise transposed, the value
    operand of the matrix-core attention kernel); rotary on every head's query part -> ``q_rot``."""
    if _gpu(qgd):
        ext().hy_latent_prep(qgd, int(H), int(dim), int(rd), int(R), int(dkv_off), dkv_w, float(eps), positions,
                             cos_sin, int(rot_dims), cache, slot_mapping, q_rot, cache_t)
    else:
        ref.latent_prep(qgd, H, dim, rd, R, dkv_off, dkv_w, eps, positions, cos_sin, rot_dims, cache, slot_mapping,
                        q_rot)
        if cache_t is not None and dkv_off >= 0:
            ok = slot_mapping >= 0
            page = cache.shape[1]
            sl = slot_mapping[ok].long()
            cache_t[sl // page, :, sl % page] = cache.view(-1, R + rd)[sl][:, :R]


MFMA_ROWS = 32  # (token, head) rows of one tile of the matrix-core attention kernel


def latent_mfma_ok(cache: torch.Tensor, R: int, rd: int) -> bool:
    """bf16 GPU caches of sizes the matrix-core kernel takes (16-token pages, kv_rank % 32 == 0, rot_dim % 16 == 0)."""
    return cache.is_cuda and cache.dtype == torch.bfloat16 and bool(ext().hy_latent_mfma_ok(cache.shape[1], R, rd))


def tile_tokens(heads: int) -> int:
    """Tokens per attention tile: as many whole tokens (all their heads) as fit 32 rows, at least one."""
    return max(1, MFMA_ROWS // heads)


ATTN_SPLIT_WGS = 256   # workgroups a matrix-core attention launch should reach before its key ranges are left whole
ATTN_SPLIT_MAX = 16


def attn_splits(n_tiles: int, heads: int, max_keys: int) -> int:
    """Key-range splits of a matrix-core attention launch: few tiles (a decode step's one tile per sequence) against
    long contexts are dealt over more workgroups, each at least two 128-key blocks long; a merge pass combines them."""
    wgs = n_tiles * -(-heads // MFMA_ROWS)
    blocks = -(-max_keys // 128)
    if wgs >= ATTN_SPLIT_WGS // 2 or blocks < 4:
        return 1
    return max(1, min(ATTN_SPLIT_MAX, ATTN_SPLIT_WGS // wgs, blocks // 2))


def latent_attn(q_lat, q_rot, cache, block_tables, tok_seg, seg, positions, scale, out, cache_t=None,
                tiles=None, max_keys: int = 0) -> None:
    """Causal softmax attention of every row's heads over its sequence's cached [latent | rotated key] rows:
    out[h, t] = sum_j softmax_j((q_lat[h, t] . c_j + q_rot[t, h] . k_j) scale) c_j over the keys j <= position[t].
    With the transposed latent copy ``cache_t`` and ``tiles`` (int32 [n, 4] = (first row, tokens, segment, 0), at
    most ``tile_tokens(H)`` tokens of one segment each) bf16 runs on the matrix cores; else one wave per (row, 4
    heads) on the vector units (fp32, odd sizes). ``max_keys`` (the step's longest context) lets a launch of few
    tiles split its key ranges over more workgroups (``attn_splits``)."""
    if _gpu(q_lat):
        if cache_t is not None and tiles is not None and q_lat.dtype == torch.bfloat16:
            H, T, R = q_lat.shape
            ns = attn_splits(tiles.shape[0], H, max_keys) if max_keys else 1
            po = pml = None
            if ns > 1:
                po = torch.empty(ns, H, T, R, dtype=torch.float32, device=q_lat.device)
                pml = torch.empty(ns, H, T, 2, dtype=torch.float32, device=q_lat.device)
            ext().hy_latent_attn_mfma(q_lat, q_rot, cache, cache_t, block_tables, tiles, tile_tokens(H), positions,
                                      float(scale), out, ns, po, pml)
        else:
            ext().hy_latent_attn(q_lat, q_rot, cache, block_tables, tok_seg, positions, float(scale), out)
    else:
        ref.latent_attn(q_lat, q_rot, cache, block_tables, tok_seg, seg, positions, scale, out)


def sigmoid_mul(a, g, out) -> None:
    if _gpu(a):
        ext().hy_sigmoid_mul(a, g, out)
    else:
        ref.sigmoid_mul(a, g, out)


def conv_silu(proj, c0: int, w, b, tok_seg, seg, state, out) -> None:
    """Causal per-channel convolution + silu over columns [c0, c0 + C) of ``proj``; ``state`` [slots, taps - 1, C]
    holds each sequence's last raw inputs and is advanced."""
    if w.shape[1] > SCAN_MAX_TAPS:
        raise ValueError(f"short convolution of {w.shape[1]} taps (at most {SCAN_MAX_TAPS})")
    if _gpu(proj):
        ext().hy_conv_silu(proj, int(c0), w, b, tok_seg, seg, state, out)
    else:
        ref.conv_silu(proj, c0, w, b, tok_seg, seg, state, out)


def ssm_scan(xbc, proj, dt_off: int, dt_bias, A_log, D, heads, P, N, G, tok_seg, seg, state, y) -> None:
    """Mamba-2 recurrence per (segment, head): S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x, with
    dt = softplus(raw dt + bias); fp32 state [slots, heads, N, P] read (unless the segment starts at 0) and left."""
    if _gpu(xbc):
        ext().hy_ssm_scan(xbc, proj, int(dt_off), dt_bias, A_log, D, int(heads), int(P), int(N), int(G), seg, state,
                          y)
    else:
        ref.ssm_scan(xbc, proj, dt_off, dt_bias, A_log, D, heads, P, N, G, tok_seg, seg, state, y)


SCAN_CHUNK = 256        # tokens per chunk of the chunk-parallel scan
SCAN_CHUNK_MIN = 512    # a step is scanned in chunks when its longest segment has at least this many rows ...
SCAN_CHUNK_WORK = 2048  # ... and it has fewer (segment, head) pairs than this (else the plain scan fills the GPU)


def scan_chunks(seg_host, heads: int):
    """Chunk tables of a step for the chunk-parallel scan, or None when the plain scan is the better fit:
    (vseg_fresh, vseg_cont, cs, max chunks) as numpy int32 - every segment cut into chunks of SCAN_CHUNK rows, chunk c
    of the step using scratch slot c; vseg_fresh starts every chunk from zero, vseg_cont from its scratch slot."""
    import numpy as np

    if seg_host is None or len(seg_host) == 0:
        return None
    n_max = int(seg_host[:, 1].max())
    if n_max < SCAN_CHUNK_MIN or len(seg_host) * heads >= SCAN_CHUNK_WORK or n_max > 256 * SCAN_CHUNK:
        return None
    vs, cs = [], []
    for q0, n, p0, slot in seg_host.tolist():
        first = len(vs)
        for a in range(0, n, SCAN_CHUNK):
            vs.append((q0 + a, min(SCAN_CHUNK, n - a), 0, len(vs)))
        cs.append((first, len(vs) - first, p0, slot))
    fresh = np.asarray(vs, dtype=np.int32)
    cont = fresh.copy()
    cont[:, 2] = 1
    return fresh, cont, np.asarray(cs, dtype=np.int32), max(c[1] for c in cs)


def ssm_scan_chunked(xbc, proj, dt_off: int, dt_bias, A_log, D, heads, P, N, G, plan, state, y) -> None:
    """The recurrence of ``ssm_scan`` in three launches that expose more parallelism for long segments: every chunk
    scanned from a zero state, the chunks' entry states rebuilt in order (and the sequence's state advanced), every
    chunk scanned again from its entry state. ``plan``: device tensors (vseg_fresh, vseg_cont, cs) + max chunks from
    ``scan_chunks``. Twice the arithmetic of the plain scan over (chunks) times the workgroups; the result differs
    from the token-by-token order only by fp32 rounding (the entry states are re-associated)."""
    fresh, cont, cs, max_chunks = plan
    tmp = torch.empty(fresh.shape[0], heads, N, P, dtype=torch.float32, device=xbc.device)
    e = ext()
    e.hy_ssm_scan(xbc, proj, int(dt_off), dt_bias, A_log, D, int(heads), int(P), int(N), int(G), fresh, tmp, y)
    e.hy_ssm_combine(proj, int(dt_off), dt_bias, A_log, int(heads), fresh, cs, int(max_chunks), tmp, state)
    e.hy_ssm_scan(xbc, proj, int(dt_off), dt_bias, A_log, D, int(heads), int(P), int(N), int(G), cont, tmp, y)


def gated_norm(y, proj, w, groups: int, eps, out) -> None:
    """out = group_rms_norm(y * silu(proj[:, :inner])) * w, the norm over ``groups`` equal parts of a row."""
    if _gpu(y):
        ext().hy_gated_norm(y, proj, w, int(groups), float(eps), out)
    else:
        ref.gated_norm(y, proj, w, groups, eps, out)
