"""Budurax in the serving engine against the plain whole-sequence implementation of tests/budurax_plain.py.

Small configurations of odd sizes (nothing a multiple of 64, a rotary part wider than its rotated dimensions, one
state-space group, a layer without feed-forward, a model without shift / depth average / token input) with random
weights made here. Each test runs on the CPU reference ops and, marked ``gpu``, on the HIP kernels.
"""
import copy
import math

import pytest
import torch

import budurax_plain as plain
from kafka_llm_service_amd.engine.engine import EngineConfig, LLMEngine
from kafka_llm_service_amd.engine.sequence import SamplingParams
from kafka_llm_service_amd.models import budurax as bx
from kafka_llm_service_amd.ops import hybrid as hops

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def _attn(heads=3, dim=24, rot_dim=16, dims=8, vdim=20, rank=40, scaling=True, kv_from=None, scale=None):
    rot = {"base": 10000.0, "dims": dims}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "rot": rot,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _mamba(heads=4, vdim=12, state=20, groups=2, norm_groups=4, conv=3):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}


def cfg_a(scale=None):
    ff = {"kind": "dense", "ff": 72}
    return {"architecture": "Budurax", "vocab": 211, "width": 88, "norm": {"eps": 1e-5}, "token_side": {"dim": 6},
            "layers": [{"type": "mamba2", "mixer": _mamba(), "mlp": ff},
                       {"type": "latent_attention", "mixer": _attn(scale=scale), "mlp": ff},
                       {"type": "latent_attention", "mixer": _attn(kv_from=1, scale=scale), "mlp": None},
                       {"type": "mamba2", "mixer": _mamba(heads=2, vdim=40, state=9, groups=1, norm_groups=1, conv=5),
                        "mlp": ff}]}


def cfg_b():
    """Ones and equal values: one head, one group, two taps, rot.dims = rot_dim, no scaling, no extras."""
    ff = {"kind": "dense", "ff": 40}
    return {"architecture": "Budurax", "vocab": 97, "width": 48, "norm": {"eps": 1e-6},
            "layers": [{"type": "latent_attention", "mixer": _attn(1, 16, 8, 8, 16, 16, scaling=False), "mlp": ff},
                       {"type": "mamba2", "mixer": _mamba(1, 16, 16, 1, 1, 2), "mlp": ff}]}


class Bench:
    """A config, its random weights and engines over them."""

    def __init__(self, cfg: dict, seed=0, extras=True, sharpen=1.0):
        self.cfg = cfg
        self.mc = bx.BuduraxConfig.from_dict(cfg, name="test")
        self.W = bx.random_tensors(self.mc, seed, shift=extras, dwa=extras)
        if sharpen != 1.0:  # peaky softmax: single keys carry the result
            for k in self.W:
                if k.endswith("mix.q"):
                    self.W[k] = (self.W[k].float() * sharpen).to(torch.bfloat16)
        self._oracle = {}

    def engine(self, device, dtype="float32", blocks=64, seqs=4, **kw):
        model = bx.BuduraxLM(self.mc, device, dtype=getattr(torch, dtype), max_positions=1024).load_tensors(self.W)
        return LLMEngine(EngineConfig(model="test", device=device, num_kv_blocks=blocks, max_num_seqs=seqs,
                                      max_model_len=1024, dtype=dtype, **kw), model_cfg=self.mc, model=model)

    def oracle(self, tokens):
        key = tuple(tokens)
        if key not in self._oracle:
            self._oracle[key] = plain.forward(self.cfg, self.W, list(tokens)).float()
        return self._oracle[key]


def toks(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def rel_err(got, want):
    """Per row: rms of the mean-free difference over the rms of the mean-free expectation."""
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()).max().item()


TOL = {"float32": 2e-4, "bfloat16": 0.08}


def feed_all(eng, rid, tokens, cuts):
    """Feed ``tokens`` in portions of the given sizes (the last size repeats), all positions wanted."""
    rows, at, i = [], 0, 0
    while at < len(tokens):
        n = min(cuts[min(i, len(cuts) - 1)], len(tokens) - at)
        last = at + n == len(tokens)
        rows.append(eng.feed([(rid, tokens[at:at + n], list(range(n)))], [rid] if last else []))
        at += n
        i += 1
    return torch.cat(rows)


@pytest.fixture(scope="module")
def bench_a():
    return Bench(cfg_a())


@pytest.fixture(scope="module")
def bench_sharp():
    return Bench(cfg_a(scale=1.2), seed=3, sharpen=3.0)


# ---- mechanisms alone ----------------------------------------------------------------------------------------------
def _seg(device, runs):
    """runs: (rows, first position, slot) -> seg, tok_seg"""
    seg, ts, r = [], [], 0
    for j, (n, p0, slot) in enumerate(runs):
        seg.append((r, n, p0, slot))
        ts += [j] * n
        r += n
    return (torch.tensor(seg, dtype=torch.int32, device=device), torch.tensor(ts, dtype=torch.int32, device=device))


@pytest.mark.parametrize("device", DEVICES)
def test_rotary_table(device):
    for rot in (_attn()["rot"], _attn(scaling=False)["rot"], {"base": 250.0, "dims": 6,
                                                               "scaling": {"factor": 16.0, "original": 32, "fast": 4.0,
                                                                           "slow": 0.5}}):
        t = bx.rotary_table(300, rot, device).cpu().double()
        cos, sin = plain.rotary_tables(300, rot)
        half = rot["dims"] // 2
        assert torch.allclose(t[:, :half], cos, atol=3e-5) and torch.allclose(t[:, half:], sin, atol=3e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d", [70, 2500, 4200])   # (the kernels keep rows of up to 1024 / 4096 values in registers)
def test_norm_and_shift(device, d):
    torch.manual_seed(0)
    T = 9
    x = torch.randn(T, d) * 3 + 1
    w, b, mu = torch.randn(d), torch.randn(d), torch.rand(d)
    want = plain.token_shift(plain.layer_norm(x.double(), w.double(), b.double(), 1e-5), mu.double())
    # the same rows as two runs of one sequence (5 + 4 rows) and, between them in the batch, another sequence's run
    other = torch.randn(3, d)
    state = torch.full((3, d), float("nan"), device=device)
    out1 = torch.empty(5, d, device=device)
    last = torch.empty(2, d, device=device)
    seg, ts = _seg(device, [(5, 0, 2)])
    hops.ln_shift(x[:5].to(device), w.to(device), b.to(device), 1e-5, out1, mu.to(device), ts, seg, state, last)
    hops.scatter_rows(state, seg, last)
    xb = torch.cat([other, x[5:]]).to(device)
    seg, ts = _seg(device, [(3, 0, 0), (4, 5, 2)])
    out2 = torch.empty(7, d, device=device)
    hops.ln_shift(xb, w.to(device), b.to(device), 1e-5, out2, mu.to(device), ts, seg, state, last)
    got = torch.cat([out1, out2[3:]]).cpu().double()
    assert torch.allclose(got, want, atol=2e-5)
    want_o = plain.token_shift(plain.layer_norm(other.double(), w.double(), b.double(), 1e-5), mu.double())
    assert torch.allclose(out2[:3].cpu().double(), want_o, atol=2e-5)
    # plain norm (no shift), bf16 output
    o = torch.empty(T, d, dtype=torch.bfloat16, device=device)
    hops.ln_shift(x.to(device), w.bfloat16().to(device), b.bfloat16().to(device), 1e-5, o)
    ref = plain.layer_norm(x.double(), w.bfloat16().double(), b.bfloat16().double(), 1e-5)
    assert torch.allclose(o.cpu().double(), ref, atol=0.05, rtol=0.01)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d", [52, 2500, 4200])
def test_add_norm_gelu_side_depth(device, d):
    torch.manual_seed(1)
    T, F, sd, V = 6, 30, 5, 40
    x, y = torch.randn(T, d), torch.randn(T, d) * 2
    w, b, w2, b2 = (torch.randn(d) for _ in range(4))
    xd = x.clone().to(device)
    h2 = torch.empty(T, d, device=device)
    hops.add_ln(xd, y.to(device), w.to(device), b.to(device), 1e-6, h2, w2.to(device), b2.to(device))
    x1 = x.double() + plain.layer_norm(y.double(), w.double(), b.double(), 1e-6)
    assert torch.allclose(xd.cpu().double(), x1, atol=1e-5)
    assert torch.allclose(h2.cpu().double(), plain.layer_norm(x1, w2.double(), b2.double(), 1e-6), atol=2e-5)
    xc = x.clone().to(device)
    hops.add_ln(xc, y.to(device), w.to(device), b.to(device), 1e-6, h2)
    assert torch.allclose(h2.cpu(), xc.cpu()) and torch.allclose(xc.cpu().double(), x1, atol=1e-5)
    gu = torch.randn(T, 2 * F) * 2
    a = torch.empty(T, F, device=device)
    hops.gelu_mul(gu.to(device), a)
    assert torch.allclose(a.cpu().double(), plain.gelu_tanh(gu[:, :F].double()) * gu[:, F:].double(), atol=1e-5)
    # token input + depth average over a stack of three earlier results
    tokens = torch.randint(0, V, (T,))
    emb, sgate = torch.randn(V, 3 * sd), torch.randn(T, sd)
    g = torch.empty(T, sd, device=device)
    hops.side_gate(sgate.to(device), tokens.to(device), emb.to(device), sd, g)
    want_g = plain.gelu_tanh(sgate.double()) * emb[tokens][:, sd:2 * sd].double()
    assert torch.allclose(g.cpu().double(), want_g, atol=1e-5)
    stack = torch.randn(5, T, d)
    sw, dwa = torch.randn(d), torch.rand(4)
    sd_dev = stack.clone().to(device)
    xs = x.clone().to(device)
    hops.side_dwa(xs, y.to(device), sw.to(device), 1e-6, sd_dev, 2, dwa.to(device))
    x2 = x.double() + plain.rms_unit(y.double(), 1e-6) * sw.double()
    want = sum(dwa[j].double() * stack[j].double() for j in range(3)) + dwa[3].double() * x2
    assert torch.allclose(sd_dev[3].cpu().double(), x2, atol=1e-5)
    assert torch.allclose(xs.cpu().double(), want, atol=1e-5)


def _paged(device, rows, page=16, n_pages=12, order=(7, 2, 9, 4, 0, 11)):
    """rows [n, w] scattered into a page pool through a shuffled page list."""
    cache = torch.full((n_pages, page, rows.shape[1]), float("nan"), device=device)
    need = -(-rows.shape[0] // page)
    bt = torch.tensor([list(order[:need]) + [0] * (8 - need)], dtype=torch.int32, device=device)
    flat = cache.view(-1, rows.shape[1])
    for j in range(rows.shape[0]):
        flat[order[j // page] * page + j % page] = rows[j].to(device)
    flat[torch.isnan(flat)] = 1e4  # rows beyond the sequence: finite garbage that must never be attended
    return cache, bt


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("R,rd,H", [(40, 16, 3), (72, 8, 5), (200, 24, 2), (448, 64, 9)])
def test_latent_attention_single_keys(device, R, rd, H):
    """One key is made to dominate each row's softmax: the output must be that key's latent, wherever the key lies
    (the first keys, both sides of every page border, the row's own position) - and a key one past the row's position
    must never be seen."""
    torch.manual_seed(2)
    n = 70
    kv = torch.randn(n, R + rd)
    kv = kv / kv.norm(dim=-1, keepdim=True)
    cache, bt = _paged(device, kv)
    targets = [0, 1, 15, 16, 17, 31, 32, 47, 48, 63, 64, 69]
    pos = [69, 69, 15, 16, 17, 31, 32, 47, 48, 63, 64, 69]   # the target is the row's own position from 15 on
    T = len(targets)
    q = torch.stack([kv[j] for j in targets]) * 60.0         # score 60 for the target, < 60 elsewhere
    q_lat = q[:, :R][None].repeat(H, 1, 1).contiguous()
    q_rot = q[:, R:][:, None].repeat(1, H, 1).contiguous()
    out = torch.empty(H, T, R, device=device)
    seg, ts = _seg(device, [(T, 0, 0)])
    positions = torch.tensor(pos, device=device)
    hops.latent_attn(q_lat.to(device), q_rot.to(device), cache, bt, ts, seg, positions, 1.0, out)
    for i, j in enumerate(targets):
        assert torch.allclose(out[:, i].cpu(), kv[j, :R].expand(H, R), atol=2e-3), (i, j)
    # the same queries one position short of their target: the target is outside and must not win
    short = torch.tensor([max(p - 1, 0) if t == p else p for t, p in zip(targets, pos)], device=device)
    hops.latent_attn(q_lat.to(device), q_rot.to(device), cache, bt, ts, seg, short, 1.0, out)
    for i, (j, p) in enumerate(zip(targets, pos)):
        if j == p and p > 0:
            assert (out[:, i].cpu() - kv[j, :R]).abs().max() > 0.05, (i, j)
    # against the plain softmax over all visible keys, diffuse scores, per head different queries
    q_lat, q_rot = torch.randn(H, T, R), torch.randn(T, H, rd)
    hops.latent_attn(q_lat.to(device), q_rot.to(device), cache, bt, ts, seg, positions, 0.3, out)
    for i, p in enumerate(pos):
        s = (q_lat[:, i].double() @ kv[:p + 1, :R].double().T + q_rot[i].double() @ kv[:p + 1, R:].double().T) * 0.3
        want = torch.softmax(s, -1) @ kv[:p + 1, :R].double()
        assert torch.allclose(out[:, i].cpu().double(), want, atol=1e-5), i


@pytest.mark.gpu
@pytest.mark.parametrize("R,rd,H", [(64, 16, 3), (128, 32, 6), (256, 16, 32), (512, 64, 40), (96, 16, 1), (32, 48, 9)])
def test_latent_attention_matrix_cores(R, rd, H):
    """The bf16 matrix-core kernel: a 40-token portion of a 150-token sequence beside another sequence's single
    token. Every row's query singles out one key - the first keys, both sides of page and 128-key block borders, the
    row's own position and the one before - and must return that key's latent; then diffuse queries against the plain
    softmax."""
    device = "cuda:0"
    torch.manual_seed(5)
    nA, nB, page = 150, 37, 16
    kvA = torch.nn.functional.normalize(torch.randn(nA, R + rd), dim=-1).bfloat16()
    kvB = torch.nn.functional.normalize(torch.randn(nB, R + rd), dim=-1).bfloat16()
    cache = torch.zeros(24, page, R + rd, dtype=torch.bfloat16, device=device)
    orderA, orderB = [7, 2, 9, 4, 0, 11, 20, 13, 5, 16], [3, 21, 8]
    bt = torch.zeros(2, 16, dtype=torch.int32, device=device)
    bt[0, :len(orderA)] = torch.tensor(orderA)
    bt[1, :len(orderB)] = torch.tensor(orderB)
    flat = cache.view(-1, R + rd)
    for kv, order in ((kvA, orderA), (kvB, orderB)):
        for j in range(kv.shape[0]):
            flat[order[j // page] * page + j % page] = kv[j].to(device)
    cache_t = cache[:, :, :R].transpose(1, 2).contiguous()
    posA = list(range(110, 150))
    pos = posA + [nB - 1]
    T = len(pos)
    cands = [0, 1, 15, 16, 17, 31, 32, 111, 112, 127, 128, 129]
    targets = [[c for c in cands + [p - 1, p] if c <= p][(i * 5) % len([c for c in cands + [p - 1, p] if c <= p])]
               for i, p in enumerate(posA)] + [nB - 1]
    kvs = [kvA] * len(posA) + [kvB]
    tt = hops.tile_tokens(H)
    tiles = [(a, min(tt, 40 - a), 0, 0) for a in range(0, 40, tt)] + [(40, 1, 1, 0)]
    tiles = torch.tensor(tiles, dtype=torch.int32, device=device)
    seg, ts = _seg(device, [(40, 110, 0), (1, nB - 1, 1)])
    positions = torch.tensor(pos, device=device)
    q = torch.stack([kvs[i][j].float() for i, j in enumerate(targets)]) * 80.0
    q_lat = q[:, :R][None].repeat(H, 1, 1).bfloat16().contiguous().to(device)
    q_rot = q[:, R:][:, None].repeat(1, H, 1).bfloat16().contiguous().to(device)
    out = torch.empty(H, T, R, dtype=torch.bfloat16, device=device)
    hops.latent_attn(q_lat, q_rot, cache, bt, ts, seg, positions, 1.0, out, cache_t, tiles)
    for i, j in enumerate(targets):
        assert torch.allclose(out[:, i].float().cpu(), kvs[i][j, :R].float().expand(H, R), atol=6e-3), (i, pos[i], j)
    q_lat = torch.randn(H, T, R).bfloat16()
    q_rot = torch.randn(T, H, rd).bfloat16()
    hops.latent_attn(q_lat.to(device), q_rot.to(device), cache, bt, ts, seg, positions, 0.4, out, cache_t, tiles)
    ref = torch.empty(H, T, R, dtype=torch.bfloat16, device=device)
    hops.latent_attn(q_lat.to(device), q_rot.to(device), cache, bt, ts, seg, positions, 0.4, ref)  # vector kernel
    for i, p in enumerate(pos):
        kv = kvs[i][:p + 1].double()
        s = (q_lat[:, i].double() @ kv[:, :R].T + q_rot[i].double() @ kv[:, R:].T) * 0.4
        want = torch.softmax(s, -1) @ kv[:, :R]
        assert torch.allclose(out[:, i].double().cpu(), want, atol=3e-3), (i, p)
        assert torch.allclose(ref[:, i].double().cpu(), want, atol=3e-3), (i, p)


@pytest.mark.gpu
@pytest.mark.parametrize("R,rd,H", [(64, 16, 3), (512, 64, 40)])
def test_latent_attention_split_key_ranges(R, rd, H):
    """A decode step of three sequences (1100, 300 and 5 cached keys): the launch deals each tile's key blocks over
    several workgroups and merges them; sequences shorter than a split's range leave it empty."""
    device = "cuda:0"
    torch.manual_seed(7)
    lens, page = [1100, 300, 5], 16
    cache = torch.zeros(100, page, R + rd, dtype=torch.bfloat16, device=device)
    perm = torch.randperm(100).tolist()
    bt = torch.zeros(3, 80, dtype=torch.int32, device=device)
    kvs, at = [], 0
    for r, n in enumerate(lens):
        kv = torch.nn.functional.normalize(torch.randn(n, R + rd), dim=-1).bfloat16()
        kvs.append(kv)
        need = -(-n // page)
        pages = perm[at:at + need]
        at += need
        bt[r, :need] = torch.tensor(pages)
        flat = cache.view(-1, R + rd)
        for j in range(n):
            flat[pages[j // page] * page + j % page] = kv[j].to(device)
    cache_t = cache[:, :, :R].transpose(1, 2).contiguous()
    seg, ts = _seg(device, [(1, n - 1, r) for r, n in enumerate(lens)])
    positions = torch.tensor([n - 1 for n in lens], device=device)
    tiles = torch.tensor([(r, 1, r, 0) for r in range(3)], dtype=torch.int32, device=device)
    assert hops.attn_splits(3, H, max(lens)) > 1
    q_lat, q_rot = torch.randn(H, 3, R).bfloat16(), torch.randn(3, H, rd).bfloat16()
    out = torch.empty(H, 3, R, dtype=torch.bfloat16, device=device)
    hops.latent_attn(q_lat.to(device), q_rot.to(device), cache, bt, ts, seg, positions, 0.5, out, cache_t, tiles,
                     max_keys=max(lens))
    for i, n in enumerate(lens):
        kv = kvs[i].double()
        sc = (q_lat[:, i].double() @ kv[:, :R].T + q_rot[i].double() @ kv[:, R:].T) * 0.5
        want = torch.softmax(sc, -1) @ kv[:, :R]
        assert torch.allclose(out[:, i].double().cpu(), want, atol=3e-3), i
    # single dominant keys in the first, a middle and the last split
    for j in (0, 640, 1099):
        q = kvs[0][j].float() * 80.0
        ql = q[:R][None, None].repeat(H, 3, 1).bfloat16().contiguous().to(device)
        qr = q[R:][None, None].repeat(3, H, 1).bfloat16().contiguous().to(device)
        hops.latent_attn(ql, qr, cache, bt, ts, seg, positions, 1.0, out, cache_t, tiles, max_keys=max(lens))
        assert torch.allclose(out[:, 0].float().cpu(), kvs[0][j, :R].float().expand(H, R), atol=6e-3), j


def cfg_m():
    """Sizes the matrix-core attention kernel takes (latent 64, rotary part 16), two attention layers sharing a cache."""
    ff = {"kind": "dense", "ff": 96}
    return {"architecture": "Budurax", "vocab": 173, "width": 80, "norm": {"eps": 1e-5}, "token_side": {"dim": 4},
            "layers": [{"type": "latent_attention", "mixer": _attn(5, 16, 16, 16, 24, 64), "mlp": ff},
                       {"type": "mamba2", "mixer": _mamba(2, 16, 8, 1, 2, 4), "mlp": ff},
                       {"type": "latent_attention", "mixer": _attn(5, 16, 16, 16, 24, 64, kv_from=0), "mlp": ff}]}


@pytest.mark.gpu
def test_matrix_core_attention_in_the_engine():
    """bf16 on the GPU with an eligible latent size: whole prompt, portions, single tokens and a mixed batch through
    the matrix-core kernel against the plain model, and against the same engine in fp32 (vector kernel)."""
    b = Bench(cfg_m(), seed=11, sharpen=2.0)
    t, u = toks(300, 173, 1), toks(41, 173, 2)
    eng = b.engine("cuda:0", "bfloat16", blocks=40)
    assert any(p is not None for p in eng.model.pages_t)
    assert rel_err(feed_all(eng, "w", t, [300]), b.oracle(t)) < TOL["bfloat16"]
    assert rel_err(feed_all(eng, "c", t, [130, 2, 61, 1, 1, 1, 40, 1]), b.oracle(t)) < TOL["bfloat16"]
    got_t, got_u = [], []
    got_t.append(eng.feed([("t", t[:200], list(range(200)))]))
    out = eng.feed([("u", u[:40], list(range(40))), ("t", t[200:201], [0])])
    got_u.append(out[:40])
    got_t.append(out[40:])
    out = eng.feed([("t", t[201:], list(range(99))), ("u", u[40:], [0])], ["t", "u"])
    got_t.append(out[:99])
    got_u.append(out[99:])
    assert rel_err(torch.cat(got_t), b.oracle(t)) < TOL["bfloat16"]
    assert rel_err(torch.cat(got_u), b.oracle(u)) < TOL["bfloat16"]
    assert eng.kvm.num_free() == 40


@pytest.mark.gpu
def test_chunk_parallel_scan():
    """Long segments scanned in chunks (zero-state scan, ordered rebuild of the entry states, second scan) against the
    token-by-token reference: a fresh 700-row segment, a 3-row one and a 600-row one that continue stored states."""
    from kafka_llm_service_amd.ops import hybrid_reference as href

    device = "cuda:0"
    torch.manual_seed(6)
    Hh, P, N, G = 6, 24, 40, 2
    inner, C = Hh * P, Hh * P + 2 * G * N
    runs = [(700, 0, 1), (3, 5, 0), (600, 40, 2)]
    T = sum(r[0] for r in runs)
    xbc, proj = torch.randn(T, C) / 2, torch.randn(T, inner + C + Hh)
    dt_bias, A_log, D = torch.randn(Hh) / 2 - 2.0, torch.rand(Hh), torch.randn(Hh)
    state0 = torch.randn(3, Hh, N, P)
    seg, ts = _seg("cpu", runs)
    want_state, want_y = state0.clone(), torch.empty(T, inner)
    href.ssm_scan(xbc, proj, inner + C, dt_bias, A_log, D, Hh, P, N, G, ts, seg, want_state, want_y)
    plan = hops.scan_chunks(seg.numpy(), Hh)
    assert plan is not None and plan[3] == 3 and plan[0].shape[0] == 3 + 1 + 3
    dplan = tuple(torch.from_numpy(a).to(device) for a in plan[:3]) + (plan[3],)
    state, y = state0.clone().to(device), torch.empty(T, inner, device=device)
    hops.ssm_scan_chunked(xbc.to(device), proj.to(device), inner + C, dt_bias.to(device), A_log.to(device),
                          D.to(device), Hh, P, N, G, dplan, state, y)
    assert torch.allclose(y.cpu(), want_y, atol=2e-4, rtol=2e-4)
    assert torch.allclose(state.cpu(), want_state, atol=2e-4, rtol=2e-4)
    assert hops.scan_chunks(_seg("cpu", [(100, 0, 0)])[0].numpy(), Hh) is None      # short: plain scan
    assert hops.scan_chunks(_seg("cpu", [(600, 0, 0)])[0].numpy(), 4096) is None    # enough workgroups already


@pytest.mark.gpu
def test_long_prompt_in_the_engine():
    """A 900-token prompt in one step, and in portions of 600 + 300 (chunk-parallel scan in both), beside a short
    request, against the plain model (fp32)."""
    b = Bench(cfg_a(), seed=13)
    t, u = toks(900, 211, 4), toks(30, 211, 5)
    eng = b.engine("cuda:0", "float32", blocks=80)
    assert rel_err(feed_all(eng, "w", t, [900]), b.oracle(t)) < TOL["float32"]
    got = [eng.feed([("t", t[:600], list(range(600))), ("u", u[:29], list(range(29)))])]
    got.append(eng.feed([("u", u[29:], [0]), ("t", t[600:], list(range(300)))], ["t", "u"]))
    got_t = torch.cat([got[0][:600], got[1][1:]])
    got_u = torch.cat([got[0][600:], got[1][:1]])
    assert rel_err(got_t, b.oracle(t)) < TOL["float32"]
    assert rel_err(got_u, b.oracle(u)) < TOL["float32"]


@pytest.mark.gpu
def test_streamed_projections():
    """Decode-sized steps run the projections on the weight-streaming GEMM when their shapes fit it (width 256 here):
    single tokens and a 100-token portion (streamed) against the plain model, and the same steps with streaming off."""
    ff = {"kind": "dense", "ff": 512}
    cfg = {"architecture": "Budurax", "vocab": 320, "width": 256, "norm": {"eps": 1e-5}, "token_side": {"dim": 8},
           "layers": [{"type": "latent_attention", "mixer": _attn(4, 32, 32, 32, 64, 64), "mlp": ff},
                      {"type": "mamba2", "mixer": _mamba(8, 32, 16, 2, 2, 4), "mlp": ff}]}
    b = Bench(cfg, seed=12)
    t = toks(140, 320, 3)
    outs = []
    for mode in ("stream", "blas"):
        eng = b.engine("cuda:0", "bfloat16", decode_gemm=mode)
        assert eng.model.stream == (mode == "stream")
        outs.append(feed_all(eng, "r", t, [100, 1]))
        assert rel_err(outs[-1], b.oracle(t)) < TOL["bfloat16"]
    assert rel_err(outs[0], outs[1].float().cpu()) < TOL["bfloat16"]


@pytest.mark.parametrize("device", DEVICES)
def test_conv_and_scan_portions(device):
    """Convolution tail and state-space state carried over portions of 1, 2, 3 and 7 rows, with another sequence's run
    in the same launch, against the plain whole-sequence functions; the slot starts out holding NaN."""
    torch.manual_seed(3)
    Hh, P, N, G, taps, T = 4, 12, 20, 2, 4, 23
    inner, C = Hh * P, Hh * P + 2 * G * N
    proj = torch.randn(T, inner + C + Hh)
    w, b = torch.randn(C, taps) / 2, torch.randn(C) / 4
    dt_bias, A_log, D = torch.randn(Hh) / 2, torch.rand(Hh), torch.randn(Hh)
    xbc_want = plain.silu(plain.causal_conv(proj[:, inner:inner + C].double(), w.double(), b.double()))
    # the recurrence, written out once more for this test
    S = torch.zeros(Hh, N, P, dtype=torch.float64)
    y_want = torch.zeros(T, inner, dtype=torch.float64)
    grp = torch.arange(Hh) // (Hh // G)
    for t in range(T):
        x = xbc_want[t, :inner].view(Hh, P)
        B, Cc = xbc_want[t, inner:inner + G * N].view(G, N)[grp], xbc_want[t, inner + G * N:].view(G, N)[grp]
        dt = torch.log1p(torch.exp(proj[t, inner + C:].double() + dt_bias.double()))
        S = torch.exp(-torch.exp(A_log.double()) * dt)[:, None, None] * S + dt[:, None, None] * B[:, :, None] * x[:, None]
        y_want[t] = (torch.einsum("hnp,hn->hp", S, Cc) + D.double()[:, None] * x).reshape(-1)
    conv_state = torch.full((3, taps - 1, C), float("nan"), device=device)
    ssm_state = torch.full((3, Hh, N, P), float("nan"), device=device)
    other = torch.randn(2, inner + C + Hh)
    got_x, got_y, at = [], [], 0
    for n in (1, 2, 3, 7, 1, 9):
        rows = torch.cat([other, proj[at:at + n]]).to(device)
        seg, ts = _seg(device, [(2, 0, 0), (n, at, 2)])
        xbc = torch.empty(2 + n, C, device=device)
        hops.conv_silu(rows, inner, w.to(device), b.to(device), ts, seg, conv_state, xbc)
        y = torch.empty(2 + n, inner, device=device)
        hops.ssm_scan(xbc, rows, inner + C, dt_bias.to(device), A_log.to(device), D.to(device), Hh, P, N, G, ts, seg,
                      ssm_state, y)
        got_x.append(xbc[2:].cpu())
        got_y.append(y[2:].cpu())
        at += n
    assert at == T
    assert torch.allclose(torch.cat(got_x).double(), xbc_want, atol=1e-5)
    assert torch.allclose(torch.cat(got_y).double(), y_want, atol=1e-4, rtol=1e-4)
    assert torch.allclose(ssm_state[2].cpu().double(), S, atol=1e-4, rtol=1e-4)
    # gate + grouped norm
    yv, z, nw = torch.randn(5, inner), torch.randn(5, inner + 3), torch.randn(inner)
    out = torch.empty(5, inner, device=device)
    hops.gated_norm(yv.to(device), z.to(device), nw.to(device), 4, 1e-5, out)
    v = (yv.double() * plain.silu(z[:, :inner].double())).view(5, 4, inner // 4)
    want = plain.rms_unit(v, 1e-5).reshape(5, inner) * nw.double()
    assert torch.allclose(out.cpu().double(), want, atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("P,N", [(64, 128), (32, 32), (40, 9), (128, 64)])
def test_scan_state_sizes(device, P, N):
    torch.manual_seed(4)
    Hh, G, T = 2, 1, 11
    inner, C = Hh * P, Hh * P + 2 * G * N
    xbc, proj = torch.randn(T, C) / 2, torch.randn(T, Hh)
    dt_bias, A_log, D = torch.zeros(Hh), torch.rand(Hh), torch.ones(Hh)
    state = torch.zeros(1, Hh, N, P, device=device)
    y = torch.empty(T, inner, device=device)
    seg, ts = _seg(device, [(T, 0, 0)])
    hops.ssm_scan(xbc.to(device), proj.to(device), 0, dt_bias.to(device), A_log.to(device), D.to(device), Hh, P, N, G,
                  ts, seg, state, y)
    S = torch.zeros(Hh, N, P, dtype=torch.float64)
    for t in range(T):
        x = xbc[t, :inner].double().view(Hh, P)
        B, Cc = xbc[t, inner:inner + N].double(), xbc[t, inner + N:].double()
        dt = torch.log1p(torch.exp(proj[t].double()))
        S = torch.exp(-torch.exp(A_log.double()) * dt)[:, None, None] * S + dt[:, None, None] * B[None, :, None] * x[:, None]
        want = (torch.einsum("hnp,n->hp", S, Cc) + x).reshape(-1)
        assert torch.allclose(y[t].cpu().double(), want, atol=1e-4, rtol=1e-4), t
    # a step of single tokens (the decode kernel): the same sequence goes on, beside another one's first token in a
    # slot that holds NaN
    state = torch.cat([state, torch.full_like(state, float("nan"))])
    xb2, pr2 = torch.randn(2, C) / 2, torch.randn(2, Hh)
    seg, ts = _seg(device, [(1, T, 0), (1, 0, 1)])
    y2 = torch.empty(2, inner, device=device)
    hops.ssm_scan(xb2.to(device), pr2.to(device), 0, dt_bias.to(device), A_log.to(device), D.to(device), Hh, P, N, G,
                  ts, seg, state, y2)
    for r, S0 in ((0, S), (1, torch.zeros_like(S))):
        x = xb2[r, :inner].double().view(Hh, P)
        B, Cc = xb2[r, inner:inner + N].double(), xb2[r, inner + N:].double()
        dt = torch.log1p(torch.exp(pr2[r].double()))
        S1 = torch.exp(-torch.exp(A_log.double()) * dt)[:, None, None] * S0 + dt[:, None, None] * B[None, :, None] * x[:, None]
        want = (torch.einsum("hnp,n->hp", S1, Cc) + x).reshape(-1)
        assert torch.allclose(y2[r].cpu().double(), want, atol=1e-4, rtol=1e-4), r
        assert torch.allclose(state[r].cpu().double(), S1, atol=1e-4, rtol=1e-4), r


# ---- the model in the engine ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_and_layers(bench_a, device, dtype):
    t = toks(45, 211, 1)
    eng = bench_a.engine(device, dtype)
    lay = []
    got = eng.feed([("a", t, list(range(len(t))))], ["a"], layers_out=lay)
    assert rel_err(got, bench_a.oracle(t)) < TOL[dtype]
    if dtype == "float32":
        _, want_l = plain.forward(bench_a.cfg, bench_a.W, t, return_layers=True)
        for i, x in enumerate(lay):
            assert torch.allclose(x.cpu().double(), want_l[i], atol=2e-3, rtol=1e-4), f"layer {i}"


@pytest.mark.parametrize("device", DEVICES)
def test_other_sizes_and_no_extras(device):
    for b in (Bench(cfg_b(), seed=5, extras=False), Bench(cfg_b(), seed=6)):
        t = toks(37, 97, 2)
        eng = b.engine(device)
        assert rel_err(feed_all(eng, "w", t, [len(t)]), b.oracle(t)) < TOL["float32"]
        assert rel_err(feed_all(eng, "c", t, [2, 3, 16, 1, 1, 5]), b.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_models_of_one_layer_kind(device):
    """Only Mamba-2 layers (the page pool stays unused), only attention layers (no recurrent matrices), one tap."""
    ff = {"kind": "dense", "ff": 56}
    only_m = {"architecture": "Budurax", "vocab": 131, "width": 40, "norm": {"eps": 1e-6},
              "layers": [{"type": "mamba2", "mixer": _mamba(2, 10, 6, 2, 1, 1), "mlp": ff},
                         {"type": "mamba2", "mixer": _mamba(4, 5, 3, 1, 2, 8), "mlp": None}]}
    only_a = {"architecture": "Budurax", "vocab": 131, "width": 40, "norm": {"eps": 1e-6}, "token_side": {"dim": 3},
              "layers": [{"type": "latent_attention", "mixer": _attn(2, 8, 4, 4, 6, 12), "mlp": None},
                         {"type": "latent_attention", "mixer": _attn(7, 4, 4, 4, 3, 12, kv_from=0), "mlp": ff}]}
    for cfg in (only_m, only_a):
        b = Bench(cfg, seed=21)
        t = toks(50, 131, 8)
        eng = b.engine(device)
        assert rel_err(feed_all(eng, "w", t, [50]), b.oracle(t)) < TOL["float32"]
        assert rel_err(feed_all(eng, "c", t, [7, 2, 20, 1]), b.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2], [16], [17, 15, 1, 2], [31, 1, 1, 1, 33], [64, 2]])
def test_portions_and_decoding(bench_sharp, device, cuts):
    """Prompt portions of several sizes (down to two tokens, [1] = everything decoded token by token: 100 steps) give
    the whole prompt's logits at every position; the softmax is peaky, so a key lost at a page or portion border
    shows."""
    t = toks(100, 211, 7)
    eng = bench_sharp.engine(device)
    assert rel_err(feed_all(eng, "r", t, cuts), bench_sharp.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_and_reuse(bench_sharp, device, dtype):
    """Four unequal requests interleaved in shared steps (portions beside single tokens, a request sitting out a
    step), then more requests through the same two slots and a pool of few pages: every request's logits equal the
    request alone."""
    b = bench_sharp
    reqs = {k: toks(n, 211, 10 + i) for i, (k, n) in enumerate([("a", 70), ("b", 1), ("c", 33), ("d", 18),
                                                                ("e", 50), ("f", 40)])}
    eng = b.engine(device, dtype, blocks=10, seqs=2)   # 160 cached tokens, two slots
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}

    def step(parts):
        entries, end = [], []
        for k, n in parts:
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        out = eng.feed(entries, end)
        r = 0
        for k, n in parts:
            got[k].append(out[r:r + n])
            r += n

    step([("a", 17), ("b", 1)])          # b ends: its slot and page go back
    step([("a", 2), ("c", 30)])          # c takes b's slot; a crosses a page border inside a portion
    step([("c", 1), ("a", 13)])
    step([("a", 1)])                     # c sits out
    step([("c", 1), ("a", 36)])
    step([("a", 1), ("c", 1)])           # both end here: a at 70, c at 33
    assert at["a"] == 70 and at["c"] == 33
    step([("d", 18), ("e", 2)])          # reused slots and pages, fresh state
    step([("e", 47)])
    step([("e", 1), ("f", 40)])
    assert eng.kvm.num_free() == 10 and eng.slots.num_free() == 2
    for k, t in reqs.items():
        assert rel_err(torch.cat(got[k]), b.oracle(t)) < TOL[dtype], k
    st = eng.slots.stats()
    assert st["acquired_total"] == 6


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_and_dirty_state(bench_a, device):
    """A short prompt, then 150 single-token steps (the rotary positions pass the YaRN original context, the scan state
    and convolution tail are carried 150 times); the state tensors start out as NaN: a sequence's first portion must
    not read its slot."""
    t = toks(160, 211, 20)
    eng = bench_a.engine(device)
    for group in (eng.v_cache.shift, eng.v_cache.conv, eng.v_cache.ssm):
        for s in group:
            if s is not None:
                s.fill_(float("nan"))
    got = feed_all(eng, "r", t, [10, 1])
    assert torch.isfinite(got).all()
    assert rel_err(got, bench_a.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(bench_a, device):
    """engine.generate: the engine's scheduler, chunked prefill (8-token chunks), slot-limited admission (3 prompts,
    2 slots), sampling kernel; every generated token is the plain model's argmax up to a rounding-sized gap."""
    eng = bench_a.engine(device, seqs=2, max_prefill_chunk=8, max_num_batched_tokens=24)
    prompts = [toks(n, 211, 30 + n) for n in (21, 9, 34)]
    outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=7, ignore_eos=True))
    assert all(len(o) == 7 for o in outs)
    for p, o in zip(prompts, outs):
        lg = bench_a.oracle(p + o)
        for i, tok in enumerate(o):
            row = lg[len(p) - 1 + i]
            assert (row.max() - row[tok]).item() < 1e-3 * row.abs().max().item(), i
    assert eng.slots.num_free() == 2 and eng.kvm.num_free() == eng.num_blocks


def test_config_registry_and_checkpoint(tmp_path):
    from kafka_llm_service_amd.models.config import get_config

    b = Bench(cfg_b(), seed=8)
    bx.save_checkpoint(b.mc, b.W, tmp_path / "m")
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "budurax" and mc.num_layers == 2 and mc.vocab_size == 97
    eng = LLMEngine(EngineConfig(model=str(tmp_path / "m"), weights=str(tmp_path / "m"), device="cpu",
                                 num_kv_blocks=8, max_num_seqs=2, max_model_len=128, dtype="float32"))
    t = toks(20, 97, 9)
    assert rel_err(feed_all(eng, "x", t, [20]), b.oracle(t)) < TOL["float32"]
    bad = copy.deepcopy(b.W)
    bad["l0.mix.q"] = bad["l0.mix.q"][:-1]
    with pytest.raises(ValueError):
        bx.BuduraxLM(b.mc, "cpu").load_tensors(bad)
    assert get_config("budurax-tiny").arch == "budurax"
    assert math.isclose(get_config("budurax-tiny").norm_eps, 1e-6)


def test_trace_runner_command_line(tmp_path):
    """bin/trace_run as a program (reference ops on the CPU): a checkpoint folder, three steps on standard input - a
    new request, two requests in one step, a step in which nothing is wanted - then the logits files, the "done"
    lines and the exit code."""
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    b = Bench(cfg_b(), seed=14)
    bx.save_checkpoint(b.mc, b.W, tmp_path / "m")
    t, u = toks(21, 97, 1), toks(6, 97, 2)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": t[:9], "want": [0, 8]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": u, "want": [5]}, {"id": "a", "tokens": t[9:20], "want": []}],
              "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": t[20:], "want": [0]}], "end": ["a"]}]
    out = subprocess.run([sys.executable, str(root / "bin/trace_run"), "--model", str(tmp_path / "m"), "--dtype",
                          "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64", "--device", "cpu"],
                         input="".join(json.dumps(x) + "\n" for x in steps), capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert [ln for ln in out.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    got = {n: torch.from_numpy(np.fromfile(tmp_path / "o" / f"{n}.f32", dtype="<f4").reshape(-1, 97)) for n in range(3)}
    assert rel_err(got[0], b.oracle(t)[[0, 8]]) < TOL["float32"]
    assert rel_err(got[1], b.oracle(u)[[5]]) < TOL["float32"]
    assert rel_err(got[2], b.oracle(t)[[20]]) < TOL["float32"]
