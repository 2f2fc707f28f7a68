"""Lisorax: a hybrid decoder of sigmoid-attention, gated linear recurrence and matrix-memory layers with routed experts.

Every layer is PARALLEL: one RMS norm, both sublayers read it, one residual add:

    h  = rms_norm(x) * w                       hm = h + conv_canon(h)        (causal, per channel, ``canon.taps`` taps)
    x += mixer(hm) + experts(h)

  attention   q, k, v projections, each followed by a short causal per-channel convolution; no rotation. The query is
              scaled by a temperature that grows with its position, 1 + c ln(floor((p + 1) / every) + 1); the score
              (q . k) scale is soft-capped (cap tanh(s / cap)), a distance bias r1_h ln(1 + r2_h (i - j)) is taken
              off, a head bias is added, and the weight of every visible key is the SIGMOID of that - no softmax, no
              normalisation over keys. Grouped key/value heads. A layer with ``kv_from`` has no key/value tensors and
              reads the cache of the named earlier layer with its own queries and biases.
  rglru       y = gelu(W_y h + b), u = conv(W_x h + b); block-diagonal gates r = sigmoid(A_r u + b_r), i = sigmoid(A_i
              u + b_i); a = exp(-8 r softplus(lambda)); S_t = a S_(t-1) + sqrt(1 - a^2) i u; output W_o (S y).
  mlstm       per head a matrix memory S (dim x vdim), a normaliser n and a running maximum m that starts at 0, with
              capped exponential input and sigmoid forget gates; the read-out S^T q / (max(|n . q|, e^-m) + 1e-6) is
              unit-RMS-normed per head, weighted, gated by sigmoid(W_g h) and projected.
  experts     router logits in fp32, the ``top`` largest chosen, softmax over the chosen logits only; expert =
              W_down (silu(W_gate h) * W_up h).

The logits are the final RMS norm times the (unscaled) embedding table; the embedding output is scaled.

Per sequence the engine keeps paged keys and values (one page pool pair per attention layer that owns its keys, page
ids shared by all of them; values page-wise transposed) and one state slot: the last ``canon.taps - 1`` normed rows
of every layer, the last conv inputs of every convolved projection, the recurrence vector of an rglru layer, and
(S, n, m) of an mlstm layer. The residual stream, norms, attention scores and weights, router logits, gates and the
recurrent states are fp32; projections run in the model dtype (bf16, or fp32 throughout).

Steps are planned as segments (``SegMeta``, models/budurax.py): one run of consecutive rows per sequence, a decoded
token being a run of one, so prompt portions and single tokens go through the same kernels.
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path

import torch
import torch.nn.functional as F

from kafka_llm_service_amd import ops
from kafka_llm_service_amd.models.budurax import SegMeta
from kafka_llm_service_amd.ops import hybrid as hops

PAGE = 16
RGLRU_RATE = 8.0          # the recurrence gate's exponent: log a = -RGLRU_RATE * r * softplus(lambda)


@dataclass
class LisoraxConfig:
    name: str = "lisorax"
    arch: str = "lisorax"
    vocab_size: int = 0
    hidden_size: int = 0
    layers: list = field(default_factory=list)   # config.json's entries: {"type", "mixer": {...}, "mlp": {...}|None}
    norm_eps: float = 1e-5
    embed_scale: float = 1.0
    canon_taps: int = 0                          # taps of the input convolution; 0 = the config has none
    max_position_embeddings: int = 1 << 20
    bos_token_id: int = 0
    eos_token_ids: list = field(default_factory=list)
    tie_word_embeddings: bool = True
    num_experts: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_dict(c: dict, name: str = "lisorax") -> "LisoraxConfig":
        return LisoraxConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                             layers=list(c["layers"]), norm_eps=float(c["norm"]["eps"]),
                             embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                             canon_taps=int(c["canon"]["taps"]) if c.get("canon") else 0)

    @staticmethod
    def from_json(path: str | Path) -> "LisoraxConfig":
        path = Path(path)
        return LisoraxConfig.from_dict(json.loads(path.read_text()), name=path.parent.name)

    def to_dict(self) -> dict:
        d = {"architecture": "Lisorax", "vocab": self.vocab_size, "width": self.hidden_size, "layers": self.layers,
             "norm": {"eps": self.norm_eps}, "embedding": {"scale": self.embed_scale}}
        if self.canon_taps:
            d["canon"] = {"taps": self.canon_taps}
        return d

    def num_params(self) -> int:
        return sum(math.prod(s) for s in tensor_shapes(self).values())


def _moe_sizes(mlp: dict) -> tuple[int, int, int]:
    if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
    return int(mlp["router"]["experts"]), int(mlp["router"]["top"]), int(mlp["expert"]["ff"])


def tensor_shapes(cfg: LisoraxConfig) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a model with this config."""
    d, V = cfg.hidden_size, cfg.vocab_size
    s: dict[str, tuple] = {"embed": (V, d)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L["mixer"]
        s[p + "norm1"] = (d,)
        if cfg.canon_taps >= 1:
            s[p + "canon1"] = (d, cfg.canon_taps)
        if L["type"] == "attention":
            H, G, D, Dv, taps = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim", "conv"))
            names = [("q", H * D)] + ([("k", G * D), ("v", G * Dv)] if m.get("kv_from") is None else [])
            for n, rows in names:
                s[p + "mix." + n] = (rows, d)
                s[p + "mix." + n + ".conv"] = (rows, taps)
            for n in ("r1", "r2", "pb"):
                s[p + "mix." + n] = (H,)
            s[p + "mix.o"] = (d, H * Dv)
        elif L["type"] == "rglru":
            Wd, nb, taps = int(m["width"]), int(m["blocks"]), int(m["conv"])
            for n in ("y", "x"):
                s[p + "mix." + n] = (Wd, d)
                s[p + "mix." + n + ".b"] = (Wd,)
            s[p + "mix.conv"], s[p + "mix.conv.b"] = (Wd, taps), (Wd,)
            for n in ("ra", "ri"):
                s[p + "mix." + n] = (nb, Wd // nb, Wd // nb)
                s[p + "mix." + n + ".b"] = (nb, Wd // nb)
            s[p + "mix.lam"] = (Wd,)
            s[p + "mix.o"] = (d, Wd)
        elif L["type"] == "mlstm":
            H, D, Dv = (int(m[k]) for k in ("heads", "dim", "vdim"))
            s[p + "mix.q"], s[p + "mix.k"] = (H * D, d), (H * D, d)
            s[p + "mix.v"], s[p + "mix.g"] = (H * Dv, d), (H * Dv, d)
            s[p + "mix.o"], s[p + "mix.norm"] = (d, H * Dv), (H * Dv,)
            for n in ("i", "f"):
                s[p + "mix." + n], s[p + "mix." + n + ".b"] = (H, d), (H,)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        if L.get("mlp"):
            E, _, ff = _moe_sizes(L["mlp"])
            for e in range(E):
                q = f"{p}mlp.e{e}."
                s[q + "gate"], s[q + "up"], s[q + "down"] = (ff, d), (ff, d), (d, ff)
            s[p + "mlp.router"], s[p + "mlp.router.b"] = (E, d), (E,)
    s["final.norm"] = (d,)
    return s


def random_tensors(cfg: LisoraxConfig, seed: int = 0, device="cpu") -> dict[str, torch.Tensor]:
    """Seeded bf16 weights with the value ranges each kind of tensor needs (negative head biases so that unnormalised
    sigmoid weights stay small, non-negative distance-bias factors, forget gates that mostly keep), drawn on
    ``device`` (large models: on the GPU)."""
    g = torch.Generator(device=device).manual_seed(seed)

    def rn(shape):
        return torch.randn(shape, generator=g, device=device)

    def ru(shape):
        return torch.rand(shape, generator=g, device=device)

    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm") or name == "final.norm":
            t = 1.0 + 0.1 * rn(shape)
        elif name.endswith("f.b"):
            t = 2.0 + 3.0 * ru(shape)
        elif name.endswith("router.b"):
            t = rn(shape)
        elif leaf == "b":
            t = 0.1 * rn(shape)
        elif leaf == "pb":
            t = -5.0 + rn(shape) * 0.3
        elif leaf == "r1":
            t = 2.0 * ru(shape)
        elif leaf == "r2":
            t = 0.1 + 0.4 * ru(shape)
        elif leaf == "lam":
            t = -4.0 + 4.0 * ru(shape)
        elif leaf in ("conv", "canon1"):
            t = rn(shape) / math.sqrt(shape[1])
        elif leaf == "embed":
            t = 0.3 * rn(shape)
        elif leaf == "router":
            t = rn(shape) * 4.0 / math.sqrt(shape[-1])
        else:
            t = rn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


class LayerState:
    """Per-layer tensors with one row per state slot: ``canon`` (the layer's last normed rows), ``conv`` (last inputs
    of the convolved projections), ``rnn`` (the rglru vector, fp32), ``S`` / ``n`` / ``m`` (mlstm, fp32)."""

    def __init__(self):
        self.layers: list[dict] = []

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for d in self.layers for t in d.values())


class _Layer:
    pass


class LisoraxLM:
    plan = "segments"  # the model runner plans its steps as SegMeta runs (engine/model_runner.py)

    def __init__(self, cfg: LisoraxConfig, device, dtype=torch.bfloat16, tp: int = 1, tp_rank: int = 0,
                 max_positions: int | None = None):
        if tp != 1:
            raise ValueError("Lisorax runs unsharded (tp = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lisorax runs in bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.tp, self.tp_rank, self.ep, self.ep_rank = 1, 0, 1, 0
        self.dp_attention = False
        self.stream = self.tiled_only = False
        self.stream_max_m = 0
        self.max_positions = int(max_positions or 8192)
        self.layers: list[_Layer] = []
        self.attn_tile_tokens: list[int] = []

    # engine hooks shared with the other model classes ---------------------------------------------------------------
    STREAMED = ("w_in", "o")

    def _streamable(self, w) -> bool:
        return w is not None and w.dtype == torch.bfloat16 and w.is_cuda and \
            ops.stream_plan(1, w.shape[0], w.shape[1]) is not None

    def stream_weight_bytes(self) -> int:
        ws = [getattr(lw, n, None) for lw in self.layers for n in self.STREAMED] + [self.head]
        return sum(w.numel() * w.element_size() for w in ws if self._streamable(w))

    def enable_stream_weights(self, tiled_only: bool = False) -> int:
        """Wave-tiled copies of the projections (ops.tile_weight) so that decode-sized steps (<= ops.STREAM_MAX_M
        rows) run them on the framework's weight-streaming MFMA GEMM; prefill-sized steps and shapes the kernel does
        not take stay on hipBLASLt. bf16 only. Returns the added bytes."""
        added = 0
        for lw in self.layers:
            for n in self.STREAMED:
                w = getattr(lw, n, None)
                if self._streamable(w):
                    setattr(lw, n + "_t", ops.tile_weight(w))
                    added += w.numel() * w.element_size()
            if lw.E and lw.w_gu.is_cuda and lw.w_gu.dtype == torch.bfloat16 and \
                    hops.moe_grouped_ok(torch.empty(1, lw.w_gu.shape[2], dtype=lw.w_gu.dtype, device=self.device),
                                        lw.w_gu, lw.w_down) and \
                    ops.stream_moe_supported(lw.w_gu.shape[1], lw.w_gu.shape[2]) and \
                    ops.stream_moe_supported(lw.w_down.shape[1], lw.w_down.shape[2]):
                lw.w_gu_t = ops.tile_experts(lw.w_gu, glu=True)   # expert feed-forwards: grouped streaming kernel
                lw.w_down_t = ops.tile_experts(lw.w_down)
                added += (lw.w_gu.numel() + lw.w_down.numel()) * lw.w_gu.element_size()
        if self._streamable(self.head):
            self.head_t = ops.tile_weight(self.head)
            added += self.head.numel() * self.head.element_size()
        self.stream = added > 0
        self.stream_max_m = ops.STREAM_MAX_M
        return added

    def _lin(self, x, w, wt=None, bias=None):
        """x @ w^T (+ bias): the weight-streaming kernel for decode-sized steps when the weight has a tiled copy, else
        hipBLASLt."""
        M = x.shape[0]
        if self.stream and wt is not None and 0 < M <= self.stream_max_m and \
                ops.stream_plan(M, w.shape[0], w.shape[1]) is not None:
            y = ops.linear_stream(x, wt)
            y = ops.slab_reduce(y) if ops.is_slab(y) else y
            return y if bias is None else y.add_(bias)
        return F.linear(x, w, bias)

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._tensors)

    # weights --------------------------------------------------------------------------------------------------
    def load_tensors(self, W: dict[str, torch.Tensor]) -> "LisoraxLM":
        """Checkpoint tensors (any float dtype) -> device tensors: projections that read the same input fused into
        one GEMM weight in the model dtype, experts stacked, everything that feeds a gate, a bias of the attention or
        the router kept in fp32."""
        cfg, dev, dt = self.cfg, self.device, self.dtype
        want = tensor_shapes(cfg)
        for k, shp in want.items():
            if k not in W:
                raise KeyError(f"checkpoint lacks tensor {k!r}")
            if tuple(W[k].shape) != tuple(shp):
                raise ValueError(f"tensor {k!r}: shape {tuple(W[k].shape)}, config says {tuple(shp)}")
        self._tensors = []

        def keep(t):
            t = t.contiguous()
            self._tensors.append(t)
            return t

        def act(name):  # model dtype
            return keep(W[name].to(device=dev, dtype=dt))

        def f32(name):
            return keep(W[name].to(device=dev, dtype=torch.float32))

        def fused(names, dtype=dt):
            return keep(torch.cat([W[n].to(device=dev, dtype=dtype) for n in names], 0))

        d = cfg.hidden_size
        # the residual stream is fp32 from the start: bf16 table values times the scale, in fp32
        self.embed = keep(W["embed"].to(device=dev, dtype=torch.float32) * float(cfg.embed_scale))
        self.final_norm = act("final.norm")
        # the output projection is the embedding table itself (unscaled); the sampler reads logits rows in 8-element
        # vectors, so it is padded with zero rows to a multiple of 8 and the extra columns are cut off as a view
        pad = -cfg.vocab_size % 8
        hw = W["embed"].to(device=dev, dtype=dt)
        self.head = keep(torch.cat([hw, torch.zeros(pad, d, dtype=dt, device=dev)], 0))
        self.layers = []
        tiles = set()
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L["mixer"]
            lw = _Layer()
            lw.type, lw.m = L["type"], m
            lw.norm1 = act(p + "norm1")
            lw.canon = act(p + "canon1") if cfg.canon_taps >= 1 else None
            if lw.type == "attention":
                H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
                if G < 1 or H % G:
                    raise ValueError(f"layer {i}: {H} query heads over {G} key/value heads")
                lw.kv_from = m.get("kv_from")
                if lw.kv_from is not None:
                    j = int(lw.kv_from)
                    src = cfg.layers[j] if 0 <= j < i else None
                    if src is None or src["type"] != "attention" or src["mixer"].get("kv_from") is not None:
                        raise ValueError(f"layer {i}: kv_from must name an earlier attention layer that owns its keys")
                    sm = src["mixer"]
                    if (int(sm["kv_heads"]), int(sm["dim"]), int(sm["vdim"])) != (G, D, Dv):
                        raise ValueError(f"layer {i}: the borrowed cache has other head sizes")
                names = ["q"] + (["k", "v"] if lw.kv_from is None else [])
                lw.w_in = fused([p + "mix." + n for n in names])
                lw.conv = fused([p + "mix." + n + ".conv" for n in names])
                lw.r1, lw.r2, lw.pb = f32(p + "mix.r1"), f32(p + "mix.r2"), f32(p + "mix.pb")
                lw.o = act(p + "mix.o")
                qt = m.get("q_temp") or {}
                lw.t_coef, lw.t_every = float(qt.get("coef", 0.0)), float(qt.get("every", 1.0))
                if lw.t_coef and lw.t_every <= 0:
                    raise ValueError(f"layer {i}: q_temp.every must be positive")
                lw.scale, lw.softcap = float(m["scale"]), float(m.get("softcap") or 0.0)
                tiles.add(hops.sig_tile_tokens(H, G))
            elif lw.type == "rglru":
                Wd, nb = int(m["width"]), int(m["blocks"])
                if nb < 1 or Wd % nb:
                    raise ValueError(f"layer {i}: width {Wd} does not split into {nb} blocks")
                lw.w_in = fused([p + "mix.y", p + "mix.x"])
                lw.b_in = fused([p + "mix.y.b", p + "mix.x.b"])
                lw.conv, lw.conv_b = act(p + "mix.conv"), act(p + "mix.conv.b")
                # both gates of a block in one batched fp32 product: [blocks, in, 2 * out] = recurrence gate | input gate
                ga = torch.cat([W[p + "mix.ra"].to(device=dev, dtype=torch.float32).transpose(1, 2),
                                W[p + "mix.ri"].to(device=dev, dtype=torch.float32).transpose(1, 2)], 2)
                lw.gate_w = keep(ga)
                lw.gate_b = keep(torch.cat([W[p + "mix.ra.b"].to(device=dev, dtype=torch.float32).reshape(-1),
                                            W[p + "mix.ri.b"].to(device=dev, dtype=torch.float32).reshape(-1)]))
                lw.rate = keep(-RGLRU_RATE * F.softplus(W[p + "mix.lam"].to(device=dev, dtype=torch.float32)))
                lw.o = act(p + "mix.o")
            else:
                H, D, Dv = (int(m[k]) for k in ("heads", "dim", "vdim"))
                lw.w_in = fused([p + "mix." + n for n in ("q", "k", "v", "g")])
                lw.gate_w = fused([p + "mix.i", p + "mix.f"], torch.float32)
                lw.gate_b = fused([p + "mix.i.b", p + "mix.f.b"], torch.float32)
                lw.mnorm, lw.o = act(p + "mix.norm"), act(p + "mix.o")
                lw.cap = float(m["gate_cap"])
                if lw.cap <= 0:
                    raise ValueError(f"layer {i}: gate_cap must be positive")
            if L.get("mlp"):
                E, top, ff = _moe_sizes(L["mlp"])
                if not 1 <= top <= E:
                    raise ValueError(f"layer {i}: top {top} of {E} experts")
                lw.E, lw.top, lw.ff = E, top, ff
                lw.router, lw.router_b = f32(p + "mlp.router"), f32(p + "mlp.router.b")
                lw.w_gu = keep(torch.stack([torch.cat([W[f"{p}mlp.e{e}.gate"], W[f"{p}mlp.e{e}.up"]], 0)
                                            for e in range(E)]).to(device=dev, dtype=dt))       # [E, 2 ff, d]
                lw.w_down = keep(torch.stack([W[f"{p}mlp.e{e}.down"] for e in range(E)]).to(device=dev, dtype=dt))
            else:
                lw.E = 0
            self.layers.append(lw)
        self.attn_tile_tokens = sorted(tiles)
        return self

    # caches ---------------------------------------------------------------------------------------------------
    def _owners(self):
        return [(i, L["mixer"]) for i, L in enumerate(self.cfg.layers)
                if L["type"] == "attention" and L["mixer"].get("kv_from") is None]

    def page_bytes(self) -> int:
        """Bytes of one 16-token page over every layer that owns keys and values."""
        es = torch.empty(0, dtype=self.dtype).element_size()
        return sum(PAGE * int(m["kv_heads"]) * (int(m["dim"]) + int(m["vdim"])) * es for _, m in self._owners()) or 1

    def alloc_cache(self, num_blocks: int, num_slots: int):
        """(per-layer (keys [blocks, 16, G dim], values [blocks, G vdim, 16]) or None, per-layer slot state). Zeroed
        once: a masked key's row is never used, but fresh memory must not hold NaN patterns for the debug checks."""
        dev, dt, d = self.device, self.dtype, self.cfg.hidden_size
        pages, state = [], LayerState()
        ct = self.cfg.canon_taps
        for lw in self.layers:
            m, st = lw.m, {}
            if lw.type == "attention" and lw.kv_from is None:
                G, D, Dv = (int(m[k]) for k in ("kv_heads", "dim", "vdim"))
                pages.append((torch.zeros(num_blocks, PAGE, G * D, dtype=dt, device=dev),
                              torch.zeros(num_blocks, G * Dv, PAGE, dtype=dt, device=dev)))
            else:
                pages.append(None)
            if ct >= 1:
                st["canon"] = torch.zeros(num_slots, ct - 1, d, dtype=dt, device=dev)
            if lw.type in ("attention", "rglru"):
                st["conv"] = torch.zeros(num_slots, lw.conv.shape[1] - 1, lw.conv.shape[0], dtype=dt, device=dev)
            if lw.type == "rglru":
                st["rnn"] = torch.zeros(num_slots, int(m["width"]), dtype=torch.float32, device=dev)
            if lw.type == "mlstm":
                H, D, Dv = (int(m[k]) for k in ("heads", "dim", "vdim"))
                st["S"] = torch.zeros(num_slots, H, D, Dv, dtype=torch.float32, device=dev)
                st["n"] = torch.zeros(num_slots, H, D, dtype=torch.float32, device=dev)
                st["m"] = torch.zeros(num_slots, H, dtype=torch.float32, device=dev)
            state.layers.append(st)
        return pages, state

    # one step ---------------------------------------------------------------------------------------------------
    def forward(self, inp, pages: list, state: LayerState, gather: bool = True,
                layers_out: list | None = None) -> torch.Tensor:
        """Logits fp32 [n, V] for ``inp.logit_rows``. ``layers_out``: a list that receives the residual stream after
        every layer (fp32 [T, d] copies; debugging and the per-layer tests)."""
        cfg, dt, dev = self.cfg, self.dtype, self.device
        m: SegMeta = inp.attn
        T, d, eps = inp.tokens.shape[0], cfg.hidden_size, cfg.norm_eps
        x = F.embedding(inp.tokens, self.embed)  # fp32 [T, d] residual stream (the table holds the scale)
        h = torch.empty(T, d, dtype=dt, device=dev)
        hm = torch.empty(T, d, dtype=dt, device=dev) if cfg.canon_taps >= 1 else h
        if self.layers:
            hops.rms_norm(x, self.layers[0].norm1, eps, h)
        for i, lw in enumerate(self.layers):
            st = state.layers[i]   # (h = this layer's norm of x: from above, or from the previous layer's add)
            if lw.canon is not None:
                hops.short_conv(h, 0, lw.canon, None, m.tok_seg, m.seg, st["canon"], hm, residual=True)
            if lw.type == "attention":
                y = self._attention(i, lw, hm, inp, m, pages, st)
            elif lw.type == "rglru":
                y = self._rglru(lw, hm, m, st)
            else:
                y = self._mlstm(lw, hm, m, st)
            ye = self._experts(lw, h) if lw.E else None
            nxt = self.layers[i + 1].norm1 if i + 1 < len(self.layers) else None
            hops.add2(x, y, ye, nxt, eps, h if nxt is not None else None)
            if layers_out is not None:
                layers_out.append(x.clone())
        xs = x.index_select(0, inp.logit_rows)
        hf = torch.empty(xs.shape[0], d, dtype=dt, device=dev)
        hops.rms_norm(xs, self.final_norm, eps, hf)
        return self._lin(hf, self.head, getattr(self, "head_t", None)).float()[:, :cfg.vocab_size]

    def _attention(self, i: int, lw, hm, inp, m: SegMeta, pages: list, st: dict) -> torch.Tensor:
        mm = lw.m
        H, G, D, Dv = (int(mm[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        T, dt, dev = hm.shape[0], self.dtype, self.device
        raw = self._lin(hm, lw.w_in, getattr(lw, "w_in_t", None))   # [q | k | v] (q alone when the keys are borrowed)
        qkv = torch.empty_like(raw)
        hops.short_conv(raw, 0, lw.conv, None, m.tok_seg, m.seg, st["conv"], qkv)
        src = i if lw.kv_from is None else int(lw.kv_from)
        k_cache, v_cache_t = pages[src]
        if lw.kv_from is None:
            hops.kv_store(qkv, H * D, H * D + G * D, k_cache, v_cache_t, inp.slot_mapping)
        ao = torch.empty(T, H * Dv, dtype=dt, device=dev)
        hops.sigmoid_attn(qkv, 0, k_cache, v_cache_t, m.block_tables, m.tok_seg, inp.positions, H, G, lw.scale,
                          lw.softcap, lw.t_coef, lw.t_every, lw.r1, lw.r2, lw.pb, ao,
                          m.tiles.get(hops.sig_tile_tokens(H, G)), m.max_keys)
        return self._lin(ao, lw.o, getattr(lw, "o_t", None))

    def _rglru(self, lw, hm, m: SegMeta, st: dict) -> torch.Tensor:
        Wd, nb = int(lw.m["width"]), int(lw.m["blocks"])
        T, dt, dev = hm.shape[0], self.dtype, self.device
        proj = self._lin(hm, lw.w_in, getattr(lw, "w_in_t", None), lw.b_in)       # [gelu branch | recurrent branch]
        u = torch.empty(T, Wd, dtype=dt, device=dev)
        hops.short_conv(proj, Wd, lw.conv, lw.conv_b, m.tok_seg, m.seg, st["conv"], u)
        # the gates' block-diagonal products in fp32: [blocks, T, in] x [blocks, in, 2 out]
        ub = u.float().view(T, nb, Wd // nb).transpose(0, 1)
        g = torch.bmm(ub, lw.gate_w)                                               # [blocks, T, 2 bw]
        bw = Wd // nb
        gates = g.view(nb, T, 2, bw).permute(1, 2, 0, 3).reshape(T, 2 * Wd)
        gates = gates + lw.gate_b
        out = torch.empty(T, Wd, dtype=dt, device=dev)
        rows = int(m.seg_host[:, 1].max()) if m.seg_host is not None and len(m.seg_host) else 0
        hops.rglru_scan(gates, proj, u, lw.rate, m.tok_seg, m.seg, st["rnn"], out, rows)
        return self._lin(out, lw.o, getattr(lw, "o_t", None))

    def _mlstm(self, lw, hm, m: SegMeta, st: dict) -> torch.Tensor:
        H, D, Dv = (int(lw.m[k]) for k in ("heads", "dim", "vdim"))
        T, dt, dev = hm.shape[0], self.dtype, self.device
        proj = self._lin(hm, lw.w_in, getattr(lw, "w_in_t", None))                # [q | k | v | output gate]
        gates = torch.addmm(lw.gate_b, hm.float(), lw.gate_w.t())                  # fp32 [T, 2 H]: input | forget
        o = torch.empty(T, H * Dv, dtype=torch.float32, device=dev)
        hops.mlstm_scan(proj, gates, H, D, Dv, lw.cap, m.tok_seg, m.seg, st["S"], st["n"], st["m"], o)
        on = torch.empty(T, H * Dv, dtype=dt, device=dev)
        hops.head_norm_gate(o, lw.mnorm, proj, 2 * H * D + H * Dv, H, self.cfg.norm_eps, on)
        return self._lin(on, lw.o, getattr(lw, "o_t", None))

    def _experts(self, lw, h) -> torch.Tensor:
        tw, te = hops.moe_router(h, lw.router, lw.router_b, lw.top)
        out = torch.empty(h.shape[0], self.cfg.hidden_size, dtype=torch.float32, device=self.device)
        hops.moe_experts(h, lw.w_gu, lw.w_down, tw, te, out, getattr(lw, "w_gu_t", None), getattr(lw, "w_down_t", None))
        return out


def load_checkpoint(model: LisoraxLM, path: str | Path) -> LisoraxLM:
    """``path``: a folder holding model.safetensors (or any *.safetensors), or such a file."""
    from safetensors import safe_open

    path = Path(path)
    files = sorted(path.glob("*.safetensors")) if path.is_dir() else [path]
    W = {}
    for f in files:
        with safe_open(str(f), framework="pt", device="cpu") as h:
            for k in h.keys():
                W[k] = h.get_tensor(k)
    return model.load_tensors(W)


def save_checkpoint(cfg: LisoraxConfig, W: dict[str, torch.Tensor], folder: str | Path) -> None:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in W.items()}, str(folder / "model.safetensors"))
    (folder / "config.json").write_text(json.dumps(cfg.to_dict(), indent=1))
