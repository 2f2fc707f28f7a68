"""Lisorax in the serving engine against the plain whole-sequence implementation of tests/lisorax_plain.py.

Small configurations of odd sizes (nothing a multiple of 64, head sizes that differ between keys and values and
between layers, a layer without feed-forward, a borrowed key/value cache) with random weights made here. Each test
runs on the CPU reference ops and, marked ``gpu``, on the HIP kernels.
"""
import copy
import math

import pytest
import torch

import lisorax_plain as plain
from kafka_llm_service_amd.engine.engine import EngineConfig, LLMEngine
from kafka_llm_service_amd.engine.sequence import SamplingParams
from kafka_llm_service_amd.models import lisorax as lx
from kafka_llm_service_amd.ops import hybrid as hops

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def _attn(heads=6, kv_heads=2, dim=24, vdim=20, conv=3, kv_from=None, scale=None, every=16, coef=0.4, softcap=20.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
         "scale": scale if scale is not None else dim ** -0.5}
    if softcap:
        m["softcap"] = softcap
    if coef:
        m["q_temp"] = {"coef": coef, "every": every}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(experts=5, top=2, ff=28):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def cfg_a(scale=None):
    return {"architecture": "Lisorax", "vocab": 211, "width": 88, "norm": {"eps": 2e-5}, "embedding": {"scale": 2.5},
            "canon": {"taps": 4},
            "layers": [{"type": "rglru", "mixer": {"width": 60, "blocks": 3, "conv": 3}, "mlp": _moe()},
                       {"type": "attention", "mixer": _attn(scale=scale), "mlp": _moe(7, 3, 20)},
                       {"type": "mlstm", "mixer": {"heads": 3, "dim": 12, "vdim": 20, "gate_cap": 12.0}, "mlp": None},
                       {"type": "attention", "mixer": _attn(heads=4, conv=2, kv_from=1, scale=scale, every=5),
                        "mlp": _moe(3, 1, 36)}]}


def cfg_b():
    """Ones and equal values: one head, as many key/value heads as query heads, one block, one expert of one, one tap,
    two input taps, no temperature, no cap, key and value sizes equal."""
    return {"architecture": "Lisorax", "vocab": 97, "width": 48, "norm": {"eps": 1e-6}, "embedding": {"scale": 1.0},
            "canon": {"taps": 2},
            "layers": [{"type": "attention", "mixer": _attn(1, 1, 16, 16, 1, coef=0.0, softcap=0.0), "mlp": _moe(1, 1, 40)},
                       {"type": "rglru", "mixer": {"width": 48, "blocks": 1, "conv": 1}, "mlp": _moe(2, 2, 8)},
                       {"type": "mlstm", "mixer": {"heads": 1, "dim": 16, "vdim": 16, "gate_cap": 4.0}, "mlp": _moe(4, 1, 8)},
                       {"type": "attention", "mixer": _attn(3, 3, 8, 40, 5, every=1), "mlp": None}]}


class Bench:
    """A config, its random weights and engines over them."""

    def __init__(self, cfg: dict, seed=0, sharpen=1.0, static_routes=False):
        self.cfg = cfg
        self.mc = lx.LisoraxConfig.from_dict(cfg, name="test")
        self.W = lx.random_tensors(self.mc, seed)
        for k in self.W:
            if sharpen != 1.0 and (k.endswith("mix.q") or k.endswith("mix.pb")):
                # scores far from zero: single keys carry the result
                self.W[k] = (self.W[k].float() * sharpen).to(torch.bfloat16)
            if static_routes and k.endswith("router.b"):
                # router biases far apart: the choice of experts rarely follows the input, and never hangs on a bf16
                # rounding (the fp32 benches keep input-driven routes)
                self.W[k] = (torch.arange(self.W[k].numel()).float() * 48.0).roll(seed + len(k)).to(torch.bfloat16)
        self._oracle = {}

    def engine(self, device, dtype="float32", blocks=64, seqs=4, **kw):
        model = lx.LisoraxLM(self.mc, device, dtype=getattr(torch, dtype), max_positions=1024).load_tensors(self.W)
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


def mean_err(got, want):
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want.double() - want.double().mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt()).mean().item()


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
    return Bench(cfg_a(), static_routes=True)


@pytest.fixture(scope="module")
def bench_sharp():
    return Bench(cfg_a(scale=0.9), seed=3, sharpen=2.0)


def _seg(device, runs):
    """runs: (rows, first position, slot) -> seg, tok_seg"""
    seg, ts, r = [], [], 0
    for j, (n, p0, slot) in enumerate(runs):
        seg.append((r, n, p0, slot))
        ts += [j] * n
        r += n
    return (torch.tensor(seg, dtype=torch.int32, device=device), torch.tensor(ts, dtype=torch.int32, device=device))


def _portions(total, cuts):
    at, i = 0, 0
    while at < total:
        n = min(cuts[i % len(cuts)], total - at)
        yield at, n
        at += n
        i += 1


CUTS = [[1000], [1], [2], [3, 1, 7, 2], [9, 16]]


# ---- mechanisms alone ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d,taps", [(70, 3), (2500, 2), (333, 5), (70, 11)])
def test_norm_and_input_convolution(device, d, taps):
    """RMS norm of the fp32 stream, then h + conv(h) with the tail of normed rows carried through a slot, for two
    sequences side by side cut into unequal portions; the slots start out as NaN."""
    g = torch.Generator().manual_seed(d)
    n = [23, 11]
    xs = [torch.randn(k, d, generator=g) * 3 for k in n]
    w, cw = 1 + 0.1 * torch.randn(d, generator=g), torch.randn(d, taps, generator=g) / taps
    want = []
    for x in xs:
        h = plain.rms_unit(x.double(), 1e-5) * w.double()
        want.append(h + plain.causal_conv(h, cw.double()))
    for cuts in CUTS:
        state = torch.full((5, taps - 1, d), float("nan"), device=device)
        got = [[], []]
        pa, pb = list(_portions(n[0], cuts)), list(_portions(n[1], cuts[::-1]))
        for i in range(max(len(pa), len(pb))):
            runs, rows = [], []
            for s, (parts, slot) in enumerate(((pa, 3), (pb, 1))):
                if i < len(parts):
                    at, k = parts[i]
                    runs.append((k, at, slot))
                    rows.append((s, xs[s][at:at + k]))
            seg, ts = _seg(device, runs)
            x = torch.cat([r for _, r in rows]).to(device)
            h, hm = torch.empty_like(x), torch.empty_like(x)
            hops.rms_norm(x, w.to(device), 1e-5, h)
            hops.short_conv(h, 0, cw.to(device), None, ts, seg, state, hm, residual=True)
            at = 0
            for s, r in rows:
                got[s].append(hm[at:at + r.shape[0]].cpu())
                at += r.shape[0]
        for s in range(2):
            assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=1e-4, rtol=1e-4), (cuts, s)


def _paged(device, n_pages, G, D, Dv, dtype=torch.float32):
    return (torch.zeros(n_pages, 16, G * D, dtype=dtype, device=device),
            torch.zeros(n_pages, G * Dv, 16, dtype=dtype, device=device))


def _attention_case(device, H, G, D, Dv, T, every, marks, dtype=torch.float32, seed=0, softcap=25.0, tiles=False):
    """Sigmoid attention of one sequence of T tokens through scattered pages, in two portions, against the plain
    function. ``marks``: (query position, key position) pairs - that query and that key are scaled so that this one
    score stands far out while every other weight is tiny (head bias -12), so a lost or extra key shows."""
    g = torch.Generator().manual_seed(seed)
    W = {"q": torch.eye(H * D), "k": torch.eye(G * D), "v": torch.eye(G * Dv), "o": torch.eye(H * Dv),
         "q.conv": torch.ones(H * D, 1), "k.conv": torch.ones(G * D, 1), "v.conv": torch.ones(G * Dv, 1),
         "r1": 2 * torch.rand(H, generator=g), "r2": 0.1 + 0.4 * torch.rand(H, generator=g),
         "pb": torch.full((H,), -12.0)}
    q = torch.randn(T, H * D, generator=g)
    k = 0.2 * torch.randn(T, G * D, generator=g)
    v = torch.randn(T, G * Dv, generator=g)
    for qi, ki in marks:  # align query qi with key ki in every head and make the pair loud
        kk = k[ki].view(G, D)
        q[qi] = (kk / kk.norm(dim=-1, keepdim=True)).repeat_interleave(H // G, 0).reshape(-1) * 6.0
        k[ki] = k[ki] * 12.0
    if dtype == torch.bfloat16:
        q, k, v = (t.bfloat16().float() for t in (q, k, v))
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": 1.0, "softcap": softcap,
         "q_temp": {"coef": 0.4, "every": every}}
    # the plain function projects its input: with identity projections the input is the concatenated q | k | v
    Wd = {n: t.double() for n, t in W.items()}
    want = _plain_attention(q.double(), k.double(), v.double(), Wd, m)
    n_pages = -(-T // 16)
    perm = torch.randperm(n_pages + 3, generator=g)[:n_pages].to(torch.int32)
    kc, vt = _paged(device, n_pages + 3, G, D, Dv, dtype)
    bt = perm.view(1, -1).to(device)
    pos = torch.arange(T, dtype=torch.int64, device=device)
    slots = (perm.long()[torch.arange(T) // 16] * 16 + torch.arange(T) % 16).to(device)
    qkv = torch.cat([q, k, v], 1).to(device=device, dtype=dtype)
    out = torch.zeros(T, H * Dv, dtype=dtype, device=device)
    cut = max(1, T - 5)
    for a, b in ((0, cut), (cut, T)):  # keys of the second portion's rows lie in an earlier step's pages
        n = b - a
        seg, ts = _seg(device, [(n, a, 0)])
        hops.kv_store(qkv[a:b], H * D, H * D + G * D, kc, vt, slots[a:b])
        tl = None
        if tiles:
            tt = hops.sig_tile_tokens(H, G)
            tl = torch.tensor([(x, min(tt, n - x), 0, 0) for x in range(0, n, tt)], dtype=torch.int32, device=device)
        hops.sigmoid_attn(qkv[a:b], 0, kc, vt, bt, ts, pos[a:b], H, G, 1.0, softcap, 0.4, float(every),
                          W["r1"].to(device), W["r2"].to(device), W["pb"].to(device), out[a:b], tl, b)
    return out.float().cpu(), want.float()


def _plain_attention(q, k, v, W, m):
    """plain.sigmoid_attention over given q / k / v: identity projections, one-tap convolutions."""
    T = q.shape[0]
    Wq = dict(W)
    Wq["q"] = torch.cat([torch.eye(q.shape[1], dtype=q.dtype), torch.zeros(q.shape[1], k.shape[1] + v.shape[1],
                                                                           dtype=q.dtype)], 1)
    h = torch.cat([q, k, v], 1)
    return plain.sigmoid_attention(h, Wq, "", m, kv=(k, v))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv", [(6, 2, 24, 20), (4, 4, 7, 70), (3, 1, 100, 9)])
def test_sigmoid_attention_single_keys(device, H, G, D, Dv):
    """Loud keys far away (the first position from the last rows), on both sides of page borders, at the row's own
    position, and one position ahead of the row, which it must not see; the temperature period (7) makes the query
    scale change several times inside the prompt."""
    T = 150
    marks = [(149, 0), (148, 1), (120, 15), (121, 16), (122, 17), (100, 100), (63, 64), (31, 32), (47, 47),
             (140, 127), (139, 128), (146, 143), (16, 15), (17, 17)]
    got, want = _attention_case(device, H, G, D, Dv, T, 7, marks, seed=H)
    assert want.abs().max() > 1.0  # the marked keys do carry weight
    # (rows 63 and 31 are aligned with the loud keys at 64 and 32: seeing one would add about its whole value row)
    assert torch.allclose(got, want, atol=2e-4, rtol=2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv", [(8, 2, 32, 48), (4, 4, 16, 20), (32, 1, 64, 96), (6, 3, 96, 96), (8, 2, 128, 256),
                                      (5, 5, 256, 8), (9, 3, 32, 32), (10, 2, 48, 40), (14, 2, 16, 136)])
def test_sigmoid_attention_matrix_cores(H, G, D, Dv):
    """The bf16 matrix-core kernel on the same loud keys (tiles of several tokens, 128-key blocks, the first and the
    last key of a block, a tile whose rows see different numbers of keys), against the plain function on the
    bf16-rounded inputs; the weights go through bf16 once, the sums are fp32."""
    T = 300
    marks = [(299, 0), (298, 1), (270, 15), (271, 16), (272, 17), (200, 200), (63, 64), (31, 32), (47, 47),
             (260, 127), (259, 128), (258, 129), (290, 255), (289, 256), (296, 293), (16, 15), (17, 17), (130, 127)]
    assert hops.sigmoid_attn_mfma_ok(torch.empty(1, 8 * (H * D + G * D + G * Dv) // 8 * 8, dtype=torch.bfloat16,
                                                 device="cuda:0"),
                                     *_paged("cuda:0", 1, G, D, Dv, torch.bfloat16), H, G)
    got, want = _attention_case("cuda:0", H, G, D, Dv, T, 7, marks, dtype=torch.bfloat16, seed=H, tiles=True)
    assert want.abs().max() > 1.0
    assert torch.allclose(got, want, atol=0.03, rtol=0.02)
    vec, _ = _attention_case("cuda:0", H, G, D, Dv, T, 7, marks, dtype=torch.bfloat16, seed=H, tiles=False)
    assert torch.allclose(got, vec, atol=0.03, rtol=0.02)


@pytest.mark.gpu
def test_sigmoid_attention_split_key_ranges():
    """A decode-like launch (one row per sequence, few tiles, long contexts): the key ranges are split over more
    workgroups and the partial sums added; same result as the unsplit launch and the per-wave kernel."""
    dev = "cuda:0"
    g = torch.Generator().manual_seed(9)
    H, G, D, Dv, n_seq, ctx = 8, 2, 64, 64, 3, [1500, 700, 129]
    n_pages = sum(-(-c // 16) for c in ctx)
    kc, vt = _paged(dev, n_pages, G, D, Dv, torch.bfloat16)
    kc.copy_((0.3 * torch.randn(kc.shape, generator=g)).to(dev))
    vt.copy_(torch.randn(vt.shape, generator=g).to(dev))
    bt = torch.zeros(n_seq, -(-max(ctx) // 16), dtype=torch.int32)
    at = 0
    for i, c in enumerate(ctx):
        n = -(-c // 16)
        bt[i, :n] = torch.arange(at, at + n)
        at += n
    bt = bt.to(dev)
    q = torch.randn(n_seq, H * D, generator=g).to(device=dev, dtype=torch.bfloat16)
    pos = torch.tensor([c - 1 for c in ctx], dtype=torch.int64, device=dev)
    seg, ts = _seg(dev, [(1, c - 1, i) for i, c in enumerate(ctx)])
    tiles = torch.tensor([(i, 1, i, 0) for i in range(n_seq)], dtype=torch.int32, device=dev)
    r1, r2 = torch.rand(H, device=dev), 0.2 * torch.rand(H, device=dev)
    pb = torch.full((H,), -4.0, device=dev)
    outs = []
    for tl, mk in ((tiles, max(ctx)), (tiles, 0), (None, 0)):
        out = torch.zeros(n_seq, H * Dv, dtype=torch.bfloat16, device=dev)
        hops.sigmoid_attn(q, 0, kc, vt, bt, ts, pos, H, G, 0.2, 20.0, 0.3, 100.0, r1, r2, pb, out, tl, mk)
        outs.append(out.float().cpu())
    assert hops.sig_splits(n_seq * G, max(ctx)) > 1
    assert outs[0].abs().max() > 0.5
    assert torch.allclose(outs[0], outs[1], atol=0.02, rtol=0.02)
    assert torch.allclose(outs[0], outs[2], atol=0.03, rtol=0.02)


@pytest.mark.gpu
def test_matrix_core_attention_in_the_engine():
    """A bf16 model whose attention sizes the matrix-core kernel takes: whole prompts, portions and single tokens
    against the same engine's whole prompt, and against the float64 oracle on average."""
    cfg = {"architecture": "Lisorax", "vocab": 211, "width": 96, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
           "canon": {"taps": 3},
           "layers": [{"type": "attention", "mixer": _attn(8, 2, 32, 48, 4), "mlp": _moe()},
                      {"type": "rglru", "mixer": {"width": 64, "blocks": 2, "conv": 4}, "mlp": None},
                      {"type": "attention", "mixer": _attn(4, 2, 32, 48, 2, kv_from=0, every=5), "mlp": _moe(3, 1, 32)}]}
    b = Bench(cfg, seed=11, static_routes=True)
    t = toks(300, 211, 3)
    eng = b.engine("cuda:0", "bfloat16")
    whole = feed_all(eng, "w", t, [300])
    assert mean_err(whole, b.oracle(t)) < 0.05
    for cuts in ([130, 2, 77, 1], [7], [128, 1]):
        assert rel_err(feed_all(eng, "c", t, cuts), whole.cpu()) < 0.03, cuts


@pytest.mark.parametrize("device", DEVICES)
def test_sigmoid_attention_without_cap_and_temperature(device):
    g = torch.Generator().manual_seed(5)
    H, G, D, Dv, T = 2, 1, 10, 6, 40
    q, k, v = (torch.randn(T, n, generator=g) for n in (H * D, G * D, G * Dv))
    r1, r2, pb = torch.rand(H, generator=g), torch.rand(H, generator=g), torch.full((H,), -1.0)
    W = {"o": torch.eye(H * Dv).double(), "q.conv": torch.ones(H * D, 1).double(), "r1": r1.double(),
         "r2": r2.double(), "pb": pb.double()}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": 0.3}
    want = _plain_attention(q.double(), k.double(), v.double(), W, m).float()
    kc, vt = _paged(device, 3, G, D, Dv)
    seg, ts = _seg(device, [(T, 0, 0)])
    qkv = torch.cat([q, k, v], 1).to(device)
    hops.kv_store(qkv, H * D, H * D + G * D, kc, vt, torch.arange(T, device=device))
    out = torch.zeros(T, H * Dv, device=device)
    hops.sigmoid_attn(qkv, 0, kc, vt, torch.arange(3, dtype=torch.int32, device=device).view(1, 3), ts,
                      torch.arange(T, device=device), H, G, 0.3, 0.0, 0.0, 1.0, r1.to(device), r2.to(device),
                      pb.to(device), out)
    assert torch.allclose(out.cpu(), want, atol=1e-4, rtol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("Wd,nb,taps,T", [(60, 3, 3, 37), (130, 1, 4, 330), (64, 64, 1, 37)])
def test_rglru_portions(device, Wd, nb, taps, T):
    """Convolution tail and recurrence vector carried through portions of 1, 2, 3, 7, ... rows from NaN slots; the
    long case also runs the chunked form of the scan (portions of more than 64 rows: 330 at once, then 9 and 16 by
    turns - and 129 + 201 below)."""
    g = torch.Generator().manual_seed(Wd)
    d, bw = 40, Wd // nb
    W = {"y": torch.randn(Wd, d, generator=g) / 6, "y.b": 0.1 * torch.randn(Wd, generator=g),
         "x": torch.randn(Wd, d, generator=g) / 6, "x.b": 0.1 * torch.randn(Wd, generator=g),
         "conv": torch.randn(Wd, taps, generator=g) / taps, "conv.b": 0.1 * torch.randn(Wd, generator=g),
         "ra": torch.randn(nb, bw, bw, generator=g) / math.sqrt(bw), "ra.b": torch.randn(nb, bw, generator=g),
         "ri": torch.randn(nb, bw, bw, generator=g) / math.sqrt(bw), "ri.b": torch.randn(nb, bw, generator=g),
         "lam": -4 + 4 * torch.rand(Wd, generator=g), "o": torch.eye(Wd)}
    h = torch.randn(T, d, generator=g)
    want = plain.rglru(h.double(), {k: v.double() for k, v in W.items()}, "", {"width": Wd, "blocks": nb}).float()
    dev = {k: v.to(device) for k, v in W.items()}
    gate_w = torch.cat([dev["ra"].transpose(1, 2), dev["ri"].transpose(1, 2)], 2)
    gate_b = torch.cat([dev["ra.b"].reshape(-1), dev["ri.b"].reshape(-1)])
    rate = -lx.RGLRU_RATE * torch.nn.functional.softplus(dev["lam"])
    for cuts in CUTS + [[129, 201]]:
        conv_st = torch.full((3, taps - 1, Wd), float("nan"), device=device)
        rnn = torch.full((3, Wd), float("nan"), device=device)
        got = []
        for at, n in _portions(T, cuts):
            seg, ts = _seg(device, [(n, at, 2)])
            proj = torch.nn.functional.linear(h[at:at + n].to(device), torch.cat([dev["y"], dev["x"]]),
                                              torch.cat([dev["y.b"], dev["x.b"]]))
            u = torch.empty(n, Wd, device=device)
            hops.short_conv(proj, Wd, dev["conv"], dev["conv.b"], ts, seg, conv_st, u)
            gates = torch.bmm(u.view(n, nb, bw).transpose(0, 1), gate_w).view(nb, n, 2, bw).permute(1, 2, 0, 3)
            gates = gates.reshape(n, 2 * Wd) + gate_b
            out = torch.empty(n, Wd, device=device)
            hops.rglru_scan(gates.contiguous(), proj, u, rate, ts, seg, rnn, out, n)
            got.append(out.cpu())
        assert torch.allclose(torch.cat(got), want, atol=2e-5, rtol=1e-4), cuts


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,Dv", [(3, 12, 20), (1, 16, 16), (2, 130, 70), (2, 5, 150)])
def test_mlstm_portions(device, H, D, Dv):
    """Matrix memory, normaliser and running maximum carried through portions from NaN slots; forget gates that keep
    and input gates that spike, so that the maximum moves and old content is rescaled."""
    g = torch.Generator().manual_seed(D)
    d, T, eps = 32, 41, 1e-5
    W = {"q": torch.randn(H * D, d, generator=g) / 4, "k": torch.randn(H * D, d, generator=g) / 4,
         "v": torch.randn(H * Dv, d, generator=g) / 4, "g": torch.randn(H * Dv, d, generator=g) / 4,
         "i": torch.randn(H, d, generator=g), "i.b": torch.randn(H, generator=g),
         "f": torch.randn(H, d, generator=g), "f.b": 2 + torch.randn(H, generator=g),
         "norm": 1 + 0.1 * torch.randn(H * Dv, generator=g), "o": torch.eye(H * Dv)}
    h = torch.randn(T, d, generator=g)
    m = {"heads": H, "dim": D, "vdim": Dv, "gate_cap": 6.0}
    want = plain.mlstm(h.double(), {k: v.double() for k, v in W.items()}, "", m, eps).float()
    dev = {k: v.to(device) for k, v in W.items()}
    w_in = torch.cat([dev[n] for n in ("q", "k", "v", "g")])
    for cuts in CUTS:
        S = torch.full((2, H, D, Dv), float("nan"), device=device)
        nrm = torch.full((2, H, D), float("nan"), device=device)
        mx = torch.full((2, H), float("nan"), device=device)
        got = []
        for at, n in _portions(T, cuts):
            seg, ts = _seg(device, [(n, at, 1)])
            x = h[at:at + n].to(device)
            proj = x @ w_in.T
            gates = torch.cat([x @ dev["i"].T + dev["i.b"], x @ dev["f"].T + dev["f.b"]], 1).contiguous()
            o = torch.empty(n, H * Dv, device=device)
            hops.mlstm_scan(proj, gates, H, D, Dv, 6.0, ts, seg, S, nrm, mx, o)
            out = torch.empty(n, H * Dv, device=device)
            hops.head_norm_gate(o, dev["norm"], proj, 2 * H * D + H * Dv, H, eps, out)
            got.append(out.cpu())
        assert torch.allclose(torch.cat(got), want, atol=5e-5, rtol=2e-4), cuts


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,k,d,ff", [(5, 2, 40, 28), (70, 5, 33, 9), (1, 1, 16, 8), (16, 8, 130, 70), (300, 12, 33, 9),
                                      (5, 4, 24, 2500)])
def test_router_and_experts(device, E, k, d, ff):
    g = torch.Generator().manual_seed(E)
    T = 29
    W = {"router": torch.randn(E, d, generator=g), "router.b": torch.randn(E, generator=g)}
    for e in range(E):
        W[f"e{e}.gate"] = torch.randn(ff, d, generator=g) / 5
        W[f"e{e}.up"] = torch.randn(ff, d, generator=g) / 5
        W[f"e{e}.down"] = torch.randn(d, ff, generator=g) / 5
    h = torch.randn(T, d, generator=g)
    mlp = {"router": {"experts": E, "top": k}, "expert": {"ff": ff}}
    want = plain.moe(h.double(), {n: t.double() for n, t in W.items()}, "", mlp).float()
    tw, te = hops.moe_router(h.to(device), W["router"].to(device), W["router.b"].to(device), k)
    z = h.double() @ W["router"].double().T + W["router.b"].double()
    val, idx = torch.topk(z, k, -1)
    assert (te.cpu().long() == idx).all()
    assert torch.allclose(tw.cpu().double(), torch.softmax(val, -1), atol=1e-5)
    w_gu = torch.stack([torch.cat([W[f"e{e}.gate"], W[f"e{e}.up"]]) for e in range(E)]).to(device)
    w_dn = torch.stack([W[f"e{e}.down"] for e in range(E)]).to(device)
    out = torch.empty(T, d, device=device)
    hops.moe_rows(h.to(device), w_gu, w_dn, tw, te, out)
    assert torch.allclose(out.cpu(), want, atol=1e-4, rtol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("E,k,d,ff,T", [(8, 2, 128, 64, 300), (20, 5, 256, 128, 70), (3, 1, 256, 256, 1),
                                        (8, 2, 512, 256, 70), (4, 4, 256, 512, 700)])
def test_experts_on_the_matrix_cores(E, k, d, ff, T):
    """bf16 sizes the expert-sorted kernels take (entries sorted by expert, any number of experts), with and without
    tiled expert weights, against the plain function on the same bf16 weights and against the per-pair kernel."""
    from kafka_llm_service_amd import ops

    dev = "cuda:0"
    g = torch.Generator().manual_seed(E)
    W = {"router": torch.randn(E, d, generator=g), "router.b": torch.randn(E, generator=g)}
    for e in range(E):
        W[f"e{e}.gate"] = (torch.randn(ff, d, generator=g) / 8).bfloat16().float()
        W[f"e{e}.up"] = (torch.randn(ff, d, generator=g) / 8).bfloat16().float()
        W[f"e{e}.down"] = (torch.randn(d, ff, generator=g) / 8).bfloat16().float()
    h = torch.randn(T, d, generator=g).bfloat16()
    mlp = {"router": {"experts": E, "top": k}, "expert": {"ff": ff}}
    want = plain.moe(h.double(), {n: t.double() for n, t in W.items()}, "", mlp).float()
    hd = h.to(dev)
    tw, te = hops.moe_router(hd, W["router"].to(dev), W["router.b"].to(dev), k)
    w_gu = torch.stack([torch.cat([W[f"e{e}.gate"], W[f"e{e}.up"]]) for e in range(E)]).to(dev, torch.bfloat16)
    w_dn = torch.stack([W[f"e{e}.down"] for e in range(E)]).to(dev, torch.bfloat16)
    assert hops.moe_grouped_ok(hd, w_gu, w_dn)
    outs = []
    tiled = (ops.tile_experts(w_gu, glu=True), ops.tile_experts(w_dn)) if d % 256 == 0 and ff % 256 == 0 else (None, None)
    for wt in ((None, None), tiled):
        out = torch.full((T, d), float("nan"), device=dev)
        hops.moe_experts(hd, w_gu, w_dn, tw, te, out, *wt)
        outs.append(out.cpu())
        assert torch.isfinite(outs[-1]).all() and rel_err(outs[-1], want) < 0.02   # (the activations pass through bf16)
    rows = torch.empty(T, d, device=dev)
    hops.moe_rows(hd, w_gu, w_dn, tw, te, rows)
    assert rel_err(rows.cpu(), want) < 0.02


@pytest.mark.parametrize("device", DEVICES)
def test_router_ties_take_the_lower_index(device):
    h = torch.ones(3, 8, device=device)
    w = torch.zeros(6, 8, device=device)
    b = torch.tensor([1.0, 3.0, 3.0, -1.0, 3.0, 0.0], device=device)
    tw, te = hops.moe_router(h, w, b, 4)
    assert te.cpu().tolist() == [[1, 2, 4, 0]] * 3
    assert torch.allclose(tw.cpu(), torch.softmax(torch.tensor([3.0, 3.0, 3.0, 1.0]), 0).expand(3, 4), atol=1e-6)


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
        want_l = []
        plain.forward(bench_a.cfg, bench_a.W, t, layers_out=want_l)
        assert len(lay) == len(want_l) == 4
        for i, x in enumerate(lay):
            assert torch.allclose(x.cpu().double(), want_l[i], atol=2e-3, rtol=1e-4), f"layer {i}"


@pytest.mark.parametrize("device", DEVICES)
def test_other_sizes_and_ones(device):
    b = Bench(cfg_b(), seed=5)
    t = toks(37, 97, 2)
    eng = b.engine(device)
    assert rel_err(feed_all(eng, "w", t, [len(t)]), b.oracle(t)) < TOL["float32"]
    assert rel_err(feed_all(eng, "c", t, [2, 3, 16, 1, 1, 5]), b.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_models_of_one_layer_kind(device):
    """Only recurrent layers (the page pool stays unused) with a one-tap input convolution, only attention layers
    without an input convolution."""
    only_r = {"architecture": "Lisorax", "vocab": 131, "width": 40, "norm": {"eps": 1e-6},
              "embedding": {"scale": 0.5}, "canon": {"taps": 1},
              "layers": [{"type": "rglru", "mixer": {"width": 24, "blocks": 2, "conv": 2}, "mlp": None},
                         {"type": "mlstm", "mixer": {"heads": 2, "dim": 6, "vdim": 10, "gate_cap": 9.0},
                          "mlp": _moe(3, 2, 12)}]}
    only_a = {"architecture": "Lisorax", "vocab": 131, "width": 40, "norm": {"eps": 1e-6},
              "embedding": {"scale": 4.0},
              "layers": [{"type": "attention", "mixer": _attn(2, 1, 8, 6, 3), "mlp": None},
                         {"type": "attention", "mixer": _attn(7, 1, 8, 6, 2, kv_from=0, every=3), "mlp": _moe(2, 1, 16)}]}
    for cfg in (only_r, only_a):
        b = Bench(cfg, seed=21)
        t = toks(50, 131, 8)
        eng = b.engine(device)
        assert rel_err(feed_all(eng, "w", t, [50]), b.oracle(t)) < TOL["float32"]
        assert rel_err(feed_all(eng, "c", t, [7, 2, 20, 1]), b.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2], [16], [17, 15, 1, 2], [31, 1, 1, 1, 33], [64, 2]])
def test_portions_and_decoding(bench_sharp, device, cuts):
    """Prompt portions of several sizes (down to two tokens, [1] = everything decoded token by token: 100 steps) give
    the whole prompt's logits at every position."""
    t = toks(100, 211, 7)
    eng = bench_sharp.engine(device)
    assert rel_err(feed_all(eng, "r", t, cuts), bench_sharp.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_and_reuse(bench_a, bench_sharp, device, dtype):
    """Four unequal requests interleaved in shared steps (portions beside single tokens, a request sitting out a
    step), then more requests through the same two slots and a pool of few pages: every request's logits equal the
    request alone. In bf16 a rounding of a score moves an unnormalised sigmoid weight by several percent, so single
    rows stray from the float64 oracle by more than the batch could explain: there each request is compared with the
    same engine's result for the request alone (milder weights), and with the oracle on average."""
    b = bench_sharp if dtype == "float32" else bench_a
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
        if dtype == "float32":
            assert rel_err(torch.cat(got[k]), b.oracle(t)) < TOL[dtype], k
        else:
            alone = eng.feed([(k, t, list(range(len(t))))], [k])
            assert rel_err(torch.cat(got[k]), alone.cpu()) < 0.03, k
            assert mean_err(alone, b.oracle(t)) < 0.05, k
    assert eng.slots.stats()["acquired_total"] == (6 if dtype == "float32" else 12)


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_and_dirty_state(bench_a, device):
    """A short prompt, then 150 single-token steps (every state is carried 150 times, the temperature steps up every
    few tokens); the state tensors start out as NaN: a sequence's first portion must not read its slot."""
    t = toks(160, 211, 20)
    eng = bench_a.engine(device)
    for st in eng.v_cache.layers:
        for s in st.values():
            s.fill_(float("nan"))
    got = feed_all(eng, "r", t, [10, 1])
    assert torch.isfinite(got).all()
    assert rel_err(got, bench_a.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_long_prompt(bench_sharp, device):
    """300 tokens at once and in portions that end inside pages: keys up to 18 pages back."""
    t = toks(300, 211, 40)
    eng = bench_sharp.engine(device)
    assert rel_err(feed_all(eng, "w", t, [300]), bench_sharp.oracle(t)) < TOL["float32"]
    assert rel_err(feed_all(eng, "c", t, [130, 2, 77, 1]), bench_sharp.oracle(t)) < TOL["float32"]


def cfg_c():
    """Sizes between the small benches and a served model: head sizes the matrix-core attention takes (in bf16), two
    query heads per key/value head, more experts than the expert-sorted router kernel's 16, a memory wider than one
    slice of value columns, a key size that is not a power of two, the layers in another order."""
    return {"architecture": "Lisorax", "vocab": 301, "width": 160, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.5},
            "canon": {"taps": 4},
            "layers": [{"type": "mlstm", "mixer": {"heads": 2, "dim": 80, "vdim": 112, "gate_cap": 10.0},
                        "mlp": _moe(24, 4, 24)},
                       {"type": "attention", "mixer": _attn(10, 5, 64, 32, 3, every=64), "mlp": _moe(24, 4, 24)},
                       {"type": "rglru", "mixer": {"width": 192, "blocks": 6, "conv": 2}, "mlp": _moe(6, 3, 40)},
                       {"type": "attention", "mixer": _attn(5, 5, 64, 32, 4, kv_from=1, every=100, coef=0.25),
                        "mlp": None},
                       {"type": "rglru", "mixer": {"width": 96, "blocks": 1, "conv": 5}, "mlp": _moe(6, 3, 40)}]}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_medium_model_prompt_portions_and_batch(device, dtype):
    """420 tokens (keys 26 pages back, the temperature stepping inside the prompt, chunked recurrences), whole, in
    portions that end inside pages and chunks with decoded tokens at the end, and two requests side by side."""
    b = Bench(cfg_c(), seed=31, static_routes=dtype == "bfloat16")
    t, u = toks(420, 301, 50), toks(150, 301, 51)
    eng = b.engine(device, dtype, blocks=40)
    whole = feed_all(eng, "w", t, [420])
    if dtype == "float32":
        ok = lambda got, tk: rel_err(got, b.oracle(tk)) < TOL["float32"]  # noqa: E731
    else:
        assert mean_err(whole, b.oracle(t)) < 0.05
        alone = {tuple(t): whole.cpu(), tuple(u): feed_all(eng, "u", u, [150]).cpu()}
        ok = lambda got, tk: rel_err(got, alone[tuple(tk)]) < 0.05  # noqa: E731
    assert ok(whole, t)
    assert ok(feed_all(eng, "c", t, [200, 3, 65, 130, 2, 1]), t)
    got_t, got_u, at_t, at_u = [], [], 0, 0
    for nt, nu in ((100, 1), (1, 70), (150, 1), (2, 77), (167, 1)):
        last = at_t + nt == 420
        out = eng.feed([("t", t[at_t:at_t + nt], list(range(nt))), ("u", u[at_u:at_u + nu], list(range(nu)))],
                       ["t", "u"] if last else [])
        got_t.append(out[:nt])
        got_u.append(out[nt:])
        at_t, at_u = at_t + nt, at_u + nu
    assert at_t == 420 and at_u == 150
    assert ok(torch.cat(got_t), t) and ok(torch.cat(got_u), u)
    assert eng.kvm.num_free() == 40


@pytest.mark.gpu
def test_preset_sizes_and_streamed_projections():
    """The smallest preset in bf16 (128-wide heads on the matrix-core attention, tiled projections and experts on the
    weight-streaming kernels for steps of few rows, hipBLASLt and the expert-sorted kernels for the long ones): single
    tokens and short portions against the whole prompt, the whole prompt against the oracle on average."""
    from kafka_llm_service_amd.models.config import LISORAX_PRESETS

    cfg = copy.deepcopy(LISORAX_PRESETS["lisorax-tiny"])
    cfg["vocab"] = 1000
    b = Bench(cfg, seed=2, static_routes=True)
    t = toks(200, 1000, 4)
    eng = b.engine("cuda:0", "bfloat16")
    eng.model.enable_stream_weights()
    assert eng.model.stream and hasattr(eng.model.layers[0], "w_gu_t")
    whole = feed_all(eng, "w", t, [200])
    assert mean_err(whole, b.oracle(t)) < 0.05
    for cuts in ([150, 1], [3, 64, 5]):
        assert rel_err(feed_all(eng, "c", t, cuts), whole.cpu()) < 0.05, cuts


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
    lx.save_checkpoint(b.mc, b.W, tmp_path / "m")
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "lisorax" and mc.num_layers == 4 and mc.vocab_size == 97 and mc.canon_taps == 2
    eng = LLMEngine(EngineConfig(model=str(tmp_path / "m"), weights=str(tmp_path / "m"), device="cpu",
                                 num_kv_blocks=8, max_num_seqs=2, max_model_len=128, dtype="float32"))
    t = toks(20, 97, 9)
    assert rel_err(feed_all(eng, "x", t, [20]), b.oracle(t)) < TOL["float32"]
    bad = copy.deepcopy(b.W)
    bad["l0.mix.q"] = bad["l0.mix.q"][:-1]
    with pytest.raises(ValueError):
        lx.LisoraxLM(b.mc, "cpu").load_tensors(bad)
    del bad["l0.mix.q"]
    with pytest.raises(KeyError):
        lx.LisoraxLM(b.mc, "cpu").load_tensors(bad)
    late = copy.deepcopy(cfg_a())
    late["layers"][1]["mixer"]["kv_from"] = 3
    with pytest.raises((ValueError, KeyError)):
        mc2 = lx.LisoraxConfig.from_dict(late)
        lx.LisoraxLM(mc2, "cpu").load_tensors(lx.random_tensors(mc2))
    tiny = get_config("lisorax-tiny")
    assert tiny.arch == "lisorax" and math.isclose(tiny.norm_eps, 1e-6) and tiny.canon_taps == 4


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
    lx.save_checkpoint(b.mc, b.W, tmp_path / "m")
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
