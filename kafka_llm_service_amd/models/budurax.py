"""Budurax: a hybrid decoder of latent-attention and Mamba-2 layers for the serving engine.

Every layer is  x += norm1b(mixer(shift(norm1(x)))),  x += norm2b(ff(norm2(x)))  with layer norms (weight + bias)
before AND after each sublayer, then a per-layer token input and a learned average over the depth:

  token shift     the mixer reads h_t + (h_{t-1} - h_t) * mu per channel (h = norm1(x), zeros before the first token)
  latent attention  a low-rank KV: per token only the RMS-normed latent c (kv_rank) and ONE rotary key part (rot_dim,
                  shared by all heads) are cached; keys / values per head are W_uk c / W_uv c. The engine attends in
                  the latent space: q_lat = W_uk^T q per head, scores = q_lat . c + q_rot . k_rot, output = W_uv
                  (sum_j p_j c_j) - all heads read the same cached rows, and nothing per head is ever materialised
                  for the context. Rotary with YaRN frequency blending; sigmoid output gate; a layer may borrow
                  another layer's cache (``kv_from``) and then has no down-projection of its own.
  mamba2          in-projection -> [z | x | B | C | dt]; causal short convolution + silu over x, B, C; the selective
                  state-space recurrence S_t = exp(-exp(A_log) dt_t) S_{t-1} + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t
                  per head (fp32 state); y * silu(z), RMS norm in groups, out-projection.
  feed-forward    W_down (gelu_tanh(W_gate h) * W_up h)
  token input     x += rms_unit(W_proj (gelu_tanh(W_gate x) * e_tok[layer part])) * w
  depth average   the next layer reads sum_j a_ij X_j over the embedding output X_0 and every layer result so far.

Per sequence the engine keeps paged latent rows (one page pool per attention layer that owns a down-projection, page
ids shared by all of them) and one state slot: the previous normed row of every shifted layer, the last taps - 1
convolution inputs and the state-space matrix of every Mamba-2 layer. The residual stream, norms, softmax, rotary
angles and everything inside the recurrence are fp32; projections run in the model dtype (bf16, or fp32 throughout).

Steps are planned as segments (``SegMeta``): one run of consecutive rows per sequence, a decoded token being a run of
one, so prompt portions and single tokens go through the same kernels.
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path

import torch
import torch.nn.functional as F

from kafka_llm_service_amd import ops
from kafka_llm_service_amd.ops import hybrid as hops

PAGE = 16


@dataclass
class BuduraxConfig:
    name: str = "budurax"
    arch: str = "budurax"
    vocab_size: int = 0
    hidden_size: int = 0
    layers: list = field(default_factory=list)   # config.json's entries: {"type", "mixer": {...}, "mlp": {...}|None}
    norm_eps: float = 1e-6
    token_side_dim: int = 0                      # 0 = no per-layer token input
    max_position_embeddings: int = 1 << 20
    bos_token_id: int = 0
    eos_token_ids: list = field(default_factory=list)
    tie_word_embeddings: bool = False
    num_experts: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_dict(c: dict, name: str = "budurax") -> "BuduraxConfig":
        side = c.get("token_side") or {}
        return BuduraxConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                             layers=list(c["layers"]), norm_eps=float(c["norm"]["eps"]),
                             token_side_dim=int(side.get("dim", 0)))

    @staticmethod
    def from_json(path: str | Path) -> "BuduraxConfig":
        path = Path(path)
        return BuduraxConfig.from_dict(json.loads(path.read_text()), name=path.parent.name)

    def to_dict(self) -> dict:
        d = {"architecture": "Budurax", "vocab": self.vocab_size, "width": self.hidden_size, "layers": self.layers,
             "norm": {"eps": self.norm_eps}}
        if self.token_side_dim:
            d["token_side"] = {"dim": self.token_side_dim}
        return d

    def num_params(self) -> int:
        return sum(math.prod(s) for s in tensor_shapes(self).values())


def tensor_shapes(cfg: BuduraxConfig, shift: bool = True, dwa: bool = True) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a model with this config."""
    d, V = cfg.hidden_size, cfg.vocab_size
    s: dict[str, tuple] = {"embed": (V, d)}
    if cfg.token_side_dim:
        s["side.embed"] = (V, cfg.token_side_dim * cfg.num_layers)
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if L.get("mlp") else ()):
            s[p + n] = (d,)
            s[p + n + ".b"] = (d,)
        if L["type"] == "latent_attention":
            H, D, rd, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            s[p + "mix.q"] = (H * (D + rd), d)
            if m.get("kv_from") is None:
                s[p + "mix.dkv"] = (R + rd, d)
                s[p + "mix.dkv.norm"] = (R,)
            s[p + "mix.uk"] = (H * D, R)
            s[p + "mix.uv"] = (H * vd, R)
            s[p + "mix.g"] = (H * vd, d)
            s[p + "mix.o"] = (d, H * vd)
        elif L["type"] == "mamba2":
            Hh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, C = Hh * P, Hh * P + 2 * G * N
            s[p + "mix.in"] = (inner + C + Hh, d)
            s[p + "mix.conv"] = (C, m["conv"])
            s[p + "mix.conv.b"] = (C,)
            for n in ("dt_bias", "A_log", "D"):
                s[p + "mix." + n] = (Hh,)
            s[p + "mix.norm"] = (inner,)
            s[p + "mix.o"] = (d, inner)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        if L.get("mlp"):
            if L["mlp"].get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unknown feed-forward kind {L['mlp'].get('kind')!r}")
            ff = L["mlp"]["ff"]
            s[p + "mlp.gate"], s[p + "mlp.up"], s[p + "mlp.down"] = (ff, d), (ff, d), (d, ff)
        if shift:
            s[p + "shift"] = (d,)
        if dwa:
            s[p + "dwa"] = (i + 2,)
        if cfg.token_side_dim:
            s[p + "side.gate"] = (cfg.token_side_dim, d)
            s[p + "side.proj"] = (d, cfg.token_side_dim)
            s[p + "side.norm"] = (d,)
    s["final.norm"], s["final.norm.b"], s["head"] = (d,), (d,), (V, d)
    return s


def random_tensors(cfg: BuduraxConfig, seed: int = 0, shift: bool = True, dwa: bool = True,
                   device="cpu") -> dict[str, torch.Tensor]:
    """Seeded bf16 weights with the value ranges each kind of tensor needs (decays in (0, 1), positive step sizes),
    drawn on ``device`` (large models: on the GPU)."""
    g = torch.Generator(device=device).manual_seed(seed)

    def rn(shape):
        return torch.randn(shape, generator=g, device=device)

    def ru(shape):
        return torch.rand(shape, generator=g, device=device)


    out = {}
    for name, shape in tensor_shapes(cfg, shift, dwa).items():
        leaf = name.split(".")[-1]
        if name.endswith(".b"):
            t = 0.1 * rn(shape)
        elif leaf in ("norm1", "norm2", "norm1b", "norm2b") or name in ("final.norm",) or name.endswith("side.norm") \
                or name.endswith("dkv.norm") or name.endswith("mix.norm"):
            t = 1.0 + 0.1 * rn(shape)
            if leaf in ("norm1b", "norm2b") or name.endswith("side.norm"):
                t = t * 0.5
        elif leaf == "shift":
            t = ru(shape)
        elif leaf == "dwa":
            t = ru(shape) + 0.2
            t = t / t.sum()
        elif leaf == "A_log":
            t = torch.log(1.0 + 7.0 * ru(shape))
        elif leaf == "dt_bias":
            t = torch.log(torch.expm1(0.01 + 0.2 * ru(shape)))
        elif leaf == "D":
            t = 1.0 + 0.1 * rn(shape)
        elif leaf == "conv":
            t = rn(shape) / math.sqrt(shape[1])
        elif leaf == "embed":
            t = rn(shape)
        else:
            t = rn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


def rotary_table(n_pos: int, rot: dict, device) -> torch.Tensor:
    """fp32 [n_pos, dims]: cos | sin of position * frequency (rotate-half pairing, ``dims / 2`` frequencies
    base^(-2i/dims)). With ``rot["scaling"]`` (YaRN: factor, original, fast, slow) frequency i is blended between
    f_i (fast-turning dimensions) and f_i / factor (slow ones) by a linear ramp between the dimensions that make
    ``fast`` and ``slow`` turns over the original context, and cos / sin are scaled by 0.1 ln(factor) + 1."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turns_dim(t: float) -> float:
            return dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))

        lo = max(math.floor(turns_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turns_dim(float(sc["slow"]))), dims - 1)
        ramp = ((torch.arange(half, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(n_pos, dtype=torch.float32)[:, None] * f.to(torch.float32)[None]  # fp32 angles
    return (torch.cat([torch.cos(ang), torch.sin(ang)], 1) * mag).to(device).contiguous()


@dataclass
class SegMeta:
    """A step's rows as per-sequence runs: ``seg`` int32 [R, 4] = (first row, rows, first position, state slot),
    ``tok_seg`` int32 [T] = the run of each row, ``block_tables`` int32 [R, W] the runs' page lists."""
    num_tokens: int
    num_segs: int
    seg: torch.Tensor
    tok_seg: torch.Tensor
    block_tables: torch.Tensor
    # attention tiles per tile size in tokens: int32 [n, 4] = (first row, tokens, run, 0), each within one run
    tiles: dict = field(default_factory=dict)
    seg_host: object = None   # numpy copy of ``seg`` (the plan's host side), for launch-shape decisions
    max_keys: int = 0         # longest context of the step (first position + rows over the runs)
    cache: dict = field(default_factory=dict)   # per-step device tables derived from seg_host (chunk plans)


@dataclass
class RecurrentState:
    """Per-layer state tensors, one row per state slot (None where a layer keeps none)."""
    shift: list          # fp32 [slots, d]: the previous token's normed mixer input
    conv: list           # model dtype [slots, taps - 1, channels]: the last raw convolution inputs
    ssm: list            # fp32 [slots, heads, N, P]

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for ts in (self.shift, self.conv, self.ssm) for t in ts
                   if t is not None)


class _Layer:
    pass


class BuduraxLM:
    plan = "segments"  # the model runner plans its steps as SegMeta runs (engine/model_runner.py)

    def __init__(self, cfg: BuduraxConfig, device, dtype=torch.bfloat16, tp: int = 1, tp_rank: int = 0,
                 max_positions: int | None = None):
        if tp != 1:
            raise ValueError("Budurax runs unsharded (tp = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Budurax runs in bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.tp, self.tp_rank, self.ep, self.ep_rank = 1, 0, 1, 0
        self.dp_attention = False
        self.stream = self.tiled_only = False
        self.stream_max_m = 0
        self.max_positions = int(max_positions or 8192)
        self.layers: list[_Layer] = []
        self._rot: dict[str, torch.Tensor] = {}
        self.has_dwa = False

    # engine hooks shared with TransformerLM ------------------------------------------------------------------
    STREAMED = ("qgd", "in_w", "o", "gate_up", "down")

    def _streamable(self, w) -> bool:
        return w is not None and w.dtype == torch.bfloat16 and w.is_cuda and \
            ops.stream_plan(1, w.shape[0], w.shape[1]) is not None

    def stream_weight_bytes(self) -> int:
        ws = [getattr(lw, n, None) for lw in self.layers for n in self.STREAMED] + [self.head]
        return sum(w.numel() * w.element_size() for w in ws if self._streamable(w))

    def enable_stream_weights(self, tiled_only: bool = False) -> int:
        """Wave-tiled copies of the projections (ops.tile_weight) so that decode-sized steps (<= ops.STREAM_MAX_M
        rows) run them on the framework's weight-streaming MFMA GEMM, as the Llama path does; prefill-sized steps and
        shapes the kernel does not take stay on hipBLASLt. bf16 only. Returns the added bytes."""
        added = 0
        for lw in self.layers:
            for n in self.STREAMED:
                w = getattr(lw, n, None)
                if self._streamable(w):
                    setattr(lw, n + "_t", ops.tile_weight(w))
                    added += w.numel() * w.element_size()
        if self._streamable(self.head):
            self.head_t = ops.tile_weight(self.head)
            added += self.head.numel() * self.head.element_size()
        self.stream = added > 0
        self.stream_max_m = ops.STREAM_MAX_M
        return added

    def _lin(self, x, w, wt=None):
        """x @ w^T: the weight-streaming kernel for decode-sized steps when the weight has a tiled copy (its split-K
        slabs summed to bf16 by slab_reduce), else hipBLASLt."""
        M = x.shape[0]
        if self.stream and wt is not None and 0 < M <= self.stream_max_m and \
                ops.stream_plan(M, w.shape[0], w.shape[1]) is not None:
            y = ops.linear_stream(x, wt)
            return ops.slab_reduce(y) if ops.is_slab(y) else y
        return F.linear(x, w)

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._tensors)

    # weights --------------------------------------------------------------------------------------------------
    def load_tensors(self, W: dict[str, torch.Tensor]) -> "BuduraxLM":
        """Checkpoint tensors (any float dtype) -> device tensors in the model dtype, projections that read the same
        input fused into one GEMM weight, per-head up-projections reshaped for the batched latent GEMMs."""
        cfg, dev, dt = self.cfg, self.device, self.dtype
        want = tensor_shapes(cfg, shift=any(k.endswith(".shift") for k in W), dwa=any(k.endswith(".dwa") for k in W))
        for k, shp in want.items():
            if k not in W:
                raise KeyError(f"checkpoint lacks tensor {k!r}")
            if tuple(W[k].shape) != tuple(shp):
                raise ValueError(f"tensor {k!r}: shape {tuple(W[k].shape)}, config says {tuple(shp)}")
        self._tensors = []

        def act(name):  # model dtype
            t = W[name].to(device=dev, dtype=dt).contiguous()
            self._tensors.append(t)
            return t

        def f32(name):
            t = W[name].to(device=dev, dtype=torch.float32).contiguous()
            self._tensors.append(t)
            return t

        def fused(names):
            t = torch.cat([W[n].to(device=dev, dtype=dt) for n in names], 0).contiguous()
            self._tensors.append(t)
            return t

        self.embed = f32("embed")  # the residual stream starts (and stays) fp32; bf16 values are exact in it
        self.side_embed = act("side.embed") if cfg.token_side_dim else None
        self.final_norm, self.final_norm_b = act("final.norm"), act("final.norm.b")
        # the sampler reads logits rows in 8-element vectors: the head is padded with zero rows to a multiple of 8
        # and the extra columns are cut off as a view
        pad = -cfg.vocab_size % 8
        hw = W["head"].to(device=dev, dtype=dt)
        self.head = torch.cat([hw, torch.zeros(pad, cfg.hidden_size, dtype=dt, device=dev)], 0).contiguous()
        self._tensors.append(self.head)
        self.layers = []
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L["mixer"]
            lw = _Layer()
            lw.type, lw.m = L["type"], m
            for n in ("norm1", "norm1b", "norm2", "norm2b"):
                has = (p + n) in want
                setattr(lw, n, act(p + n) if has else None)
                setattr(lw, n + "_b", act(p + n + ".b") if has else None)
            lw.shift = act(p + "shift") if p + "shift" in want else None
            lw.dwa = f32(p + "dwa") if p + "dwa" in want else None
            if lw.type == "latent_attention":
                H, D, rd, vd, R = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
                lw.kv_from = m.get("kv_from")
                if lw.kv_from is not None:
                    src = cfg.layers[int(lw.kv_from)]
                    if src["type"] != "latent_attention" or src["mixer"].get("kv_from") is not None or \
                            int(lw.kv_from) >= i:
                        raise ValueError(f"layer {i}: kv_from must name an earlier latent-attention layer that owns "
                                         "its cache")
                    sm = src["mixer"]
                    if (int(sm["kv_rank"]), int(sm["rot_dim"])) != (R, rd) or sm["rot"] != m["rot"]:
                        raise ValueError(f"layer {i}: borrowed cache has another latent size or rotation")
                names = [p + "mix.q", p + "mix.g"] + ([p + "mix.dkv"] if lw.kv_from is None else [])
                lw.qgd = fused(names)
                lw.g_off = H * (D + rd)
                lw.dkv_off = lw.g_off + H * vd if lw.kv_from is None else -1
                lw.dkv_norm = act(p + "mix.dkv.norm") if lw.kv_from is None else None
                lw.uk_h = act(p + "mix.uk").view(H, D, R)                          # q_lat = q_u @ uk_h  (per head)
                t = W[p + "mix.uv"].to(device=dev, dtype=dt).view(H, vd, R).transpose(1, 2).contiguous()
                self._tensors.append(t)
                lw.uv_ht = t                                                       # out = o_lat @ uv_ht (per head)
                lw.o = act(p + "mix.o")
                lw.scale = float(m["scale"])
                lw.rot_dims = int(m["rot"]["dims"])
                if lw.rot_dims > rd or lw.rot_dims % 2:
                    raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
                lw.cos_sin = self._rot_table(m["rot"])
            else:
                Hh, P, N, G = (int(m[k]) for k in ("heads", "vdim", "state", "groups"))
                if Hh % G or (Hh * P) % int(m["norm_groups"]):
                    raise ValueError(f"layer {i}: heads / groups / norm_groups do not divide")
                lw.in_w, lw.conv, lw.conv_b = act(p + "mix.in"), act(p + "mix.conv"), act(p + "mix.conv.b")
                lw.dt_bias, lw.A_log, lw.D = f32(p + "mix.dt_bias"), f32(p + "mix.A_log"), f32(p + "mix.D")
                lw.mnorm, lw.o = act(p + "mix.norm"), act(p + "mix.o")
            if L.get("mlp"):
                lw.gate_up = fused([p + "mlp.gate", p + "mlp.up"])
                lw.down = act(p + "mlp.down")
                lw.ff = int(L["mlp"]["ff"])
            else:
                lw.gate_up = lw.down = None
            if cfg.token_side_dim:
                lw.side_gate, lw.side_proj, lw.side_norm = act(p + "side.gate"), act(p + "side.proj"), \
                    act(p + "side.norm")
            else:
                lw.side_gate = lw.side_proj = lw.side_norm = None
            self.layers.append(lw)
        self.has_dwa = any(lw.dwa is not None for lw in self.layers)
        # tile sizes (tokens) the step plan must carry for the attention layers (ops.hybrid.tile_tokens)
        self.attn_tile_tokens = sorted({hops.tile_tokens(int(lw.m["heads"])) for lw in self.layers
                                        if lw.type == "latent_attention"})
        return self

    def _rot_table(self, rot: dict) -> torch.Tensor:
        key = json.dumps(rot, sort_keys=True)
        if key not in self._rot:
            self._rot[key] = rotary_table(self.max_positions, rot, self.device)
        return self._rot[key]

    # caches ---------------------------------------------------------------------------------------------------
    def page_bytes(self) -> int:
        """Bytes of one 16-token page over every layer that owns a latent cache."""
        es = torch.empty(0, dtype=self.dtype).element_size()
        # (the latent part is kept twice where the matrix-core kernel runs: row-major and page-wise transposed)
        return sum(PAGE * (2 * int(L["mixer"]["kv_rank"]) + int(L["mixer"]["rot_dim"])) * es
                   for L in self.cfg.layers
                   if L["type"] == "latent_attention" and L["mixer"].get("kv_from") is None) or 1

    def alloc_cache(self, num_blocks: int, num_slots: int) -> tuple[list, RecurrentState]:
        """(per-layer latent page pools [blocks, 16, kv_rank + rot_dim] or None, per-layer slot state). Zeroed once:
        a masked key's row is never read, but fresh memory must not hold NaN patterns for the debug checks."""
        dev, dt, d = self.device, self.dtype, self.cfg.hidden_size
        pages, shift, conv, ssm = [], [], [], []
        self.pages_t = []  # page-wise transposed latent copies [blocks, kv_rank, 16] where the MFMA kernel applies
        for lw in self.layers:
            m = lw.m
            own = lw.type == "latent_attention" and lw.kv_from is None
            pages.append(torch.zeros(num_blocks, PAGE, int(m["kv_rank"]) + int(m["rot_dim"]), dtype=dt, device=dev)
                         if own else None)
            self.pages_t.append(torch.zeros(num_blocks, int(m["kv_rank"]), PAGE, dtype=dt, device=dev)
                                if own and hops.latent_mfma_ok(pages[-1], int(m["kv_rank"]), int(m["rot_dim"]))
                                else None)
            shift.append(torch.zeros(num_slots, d, dtype=torch.float32, device=dev) if lw.shift is not None else None)
            if lw.type == "mamba2":
                Hh, P, N, G = (int(m[k]) for k in ("heads", "vdim", "state", "groups"))
                conv.append(torch.zeros(num_slots, int(m["conv"]) - 1, Hh * P + 2 * G * N, dtype=dt, device=dev))
                ssm.append(torch.zeros(num_slots, Hh, N, P, dtype=torch.float32, device=dev))
            else:
                conv.append(None)
                ssm.append(None)
        return pages, RecurrentState(shift, conv, ssm)

    # one step ---------------------------------------------------------------------------------------------------
    def forward(self, inp, pages: list, state: RecurrentState, gather: bool = True,
                layers_out: list | None = None) -> torch.Tensor:
        """Logits fp32 [n, V] for ``inp.logit_rows``. ``layers_out``: a list that receives the residual stream after
        every layer (fp32 [T, d] copies; debugging and the per-layer tests)."""
        cfg, dt, dev = self.cfg, self.dtype, self.device
        m: SegMeta = inp.attn
        T, d, eps = inp.tokens.shape[0], cfg.hidden_size, cfg.norm_eps
        x = F.embedding(inp.tokens, self.embed)  # fp32 [T, d] residual stream
        stack = None
        if self.has_dwa:
            stack = torch.empty(len(self.layers) + 1, T, d, dtype=torch.float32, device=dev)
            stack[0].copy_(x)
        h = torch.empty(T, d, dtype=dt, device=dev)
        h2 = torch.empty(T, d, dtype=dt, device=dev)
        last = torch.empty(m.num_segs, d, dtype=torch.float32, device=dev)
        for i, lw in enumerate(self.layers):
            hops.ln_shift(x, lw.norm1, lw.norm1_b, eps, h, lw.shift, m.tok_seg, m.seg, state.shift[i], last)
            if lw.shift is not None:
                hops.scatter_rows(state.shift[i], m.seg, last)
            if lw.type == "latent_attention":
                y = self._latent_attention(i, lw, h, inp, m, pages)
            else:
                y = self._mamba2(i, lw, h, m, state)
            if lw.gate_up is not None:
                hops.add_ln(x, y, lw.norm1b, lw.norm1b_b, eps, h2, lw.norm2, lw.norm2_b)
                a = torch.empty(T, lw.ff, dtype=dt, device=dev)
                hops.gelu_mul(self._lin(h2, lw.gate_up, getattr(lw, "gate_up_t", None)), a)
                y = self._lin(a, lw.down, getattr(lw, "down_t", None))
                nw, nb = lw.norm2b, lw.norm2b_b
            else:
                nw, nb = lw.norm1b, lw.norm1b_b
            ys = None
            if lw.side_gate is not None:
                hops.add_ln(x, y, nw, nb, eps, h2)  # h2 = the new x in the model dtype (the gate GEMM's input)
                g = torch.empty(T, cfg.token_side_dim, dtype=dt, device=dev)
                hops.side_gate(F.linear(h2, lw.side_gate), inp.tokens, self.side_embed, i * cfg.token_side_dim, g)
                ys = F.linear(g, lw.side_proj)
            else:
                hops.add_ln(x, y, nw, nb, eps)
            if ys is not None or stack is not None:
                hops.side_dwa(x, ys, lw.side_norm, eps, stack, i, lw.dwa)
            if layers_out is not None:
                layers_out.append(x.clone())
        xs = x.index_select(0, inp.logit_rows)
        hf = torch.empty(xs.shape[0], d, dtype=dt, device=dev)
        hops.ln_shift(xs, self.final_norm, self.final_norm_b, eps, hf)
        return self._lin(hf, self.head, getattr(self, "head_t", None)).float()[:, :cfg.vocab_size]

    def _latent_attention(self, i: int, lw, h, inp, m: SegMeta, pages: list) -> torch.Tensor:
        mm = lw.m
        H, D, rd, vd, R = (int(mm[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
        T, dt, dev = h.shape[0], self.dtype, self.device
        qgd = self._lin(h, lw.qgd, getattr(lw, "qgd_t", None))  # [q heads (dim | rot) | output gate | latent, shared rotary key]
        src = i if lw.kv_from is None else int(lw.kv_from)
        cache, cache_t = pages[src], self.pages_t[src]
        q_rot = torch.empty(T, H, rd, dtype=dt, device=dev)
        hops.latent_prep(qgd, H, D, rd, R, lw.dkv_off, lw.dkv_norm, self.cfg.norm_eps, inp.positions, lw.cos_sin,
                         lw.rot_dims, cache, inp.slot_mapping, q_rot, cache_t if lw.kv_from is None else None)
        q_u = qgd[:, :H * (D + rd)].view(T, H, D + rd)[:, :, :D].transpose(0, 1)  # [H, T, dim] (strided view)
        q_lat = torch.bmm(q_u, lw.uk_h)                                           # [H, T, R]
        o_lat = torch.empty(H, T, R, dtype=dt, device=dev)
        hops.latent_attn(q_lat, q_rot, cache, m.block_tables, m.tok_seg, m.seg, inp.positions, lw.scale, o_lat,
                         cache_t, m.tiles.get(hops.tile_tokens(H)), m.max_keys)
        a = torch.bmm(o_lat, lw.uv_ht)                                            # [H, T, vdim]
        ao = torch.empty(T, H * vd, dtype=dt, device=dev)
        hops.sigmoid_mul(a, qgd[:, lw.g_off:lw.g_off + H * vd], ao)
        return self._lin(ao, lw.o, getattr(lw, "o_t", None))

    def _chunk_plan(self, m: SegMeta, heads: int):
        """Device chunk tables of this step for layers of ``heads`` heads (built once per step), None = plain scan."""
        key = ("chunks", heads)
        if key not in m.cache:
            p = hops.scan_chunks(m.seg_host, heads)
            if p is not None:
                fresh, cont, cs, mx = p
                up = torch.from_numpy(__import__("numpy").concatenate([fresh.reshape(-1), cont.reshape(-1),
                                                                       cs.reshape(-1)])).to(self.device)
                a, b = fresh.size, fresh.size + cont.size
                p = (up[:a].view(-1, 4), up[a:b].view(-1, 4), up[b:].view(-1, 4), mx)
            m.cache[key] = p
        return m.cache[key]

    def _mamba2(self, i: int, lw, h, m: SegMeta, state: RecurrentState) -> torch.Tensor:
        mm = lw.m
        Hh, P, N, G = (int(mm[k]) for k in ("heads", "vdim", "state", "groups"))
        inner, C = Hh * P, Hh * P + 2 * G * N
        T, dt, dev = h.shape[0], self.dtype, self.device
        proj = self._lin(h, lw.in_w, getattr(lw, "in_w_t", None))  # [z | x | B | C | dt]
        xbc = torch.empty(T, C, dtype=dt, device=dev)
        hops.conv_silu(proj, inner, lw.conv, lw.conv_b, m.tok_seg, m.seg, state.conv[i], xbc)
        y = torch.empty(T, inner, dtype=torch.float32, device=dev)
        plan = self._chunk_plan(m, Hh) if dev.type == "cuda" else None
        if plan is not None:  # long prompt portions, few sequences: chunk-parallel scan
            hops.ssm_scan_chunked(xbc, proj, inner + C, lw.dt_bias, lw.A_log, lw.D, Hh, P, N, G, plan, state.ssm[i], y)
        else:
            hops.ssm_scan(xbc, proj, inner + C, lw.dt_bias, lw.A_log, lw.D, Hh, P, N, G, m.tok_seg, m.seg,
                          state.ssm[i], y)
        yn = torch.empty(T, inner, dtype=dt, device=dev)
        hops.gated_norm(y, proj, lw.mnorm, int(mm["norm_groups"]), self.cfg.norm_eps, yn)
        return self._lin(yn, lw.o, getattr(lw, "o_t", None))


def load_checkpoint(model: BuduraxLM, path: str | Path) -> BuduraxLM:
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


def save_checkpoint(cfg: BuduraxConfig, W: dict[str, torch.Tensor], folder: str | Path) -> None:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in W.items()}, str(folder / "model.safetensors"))
    (folder / "config.json").write_text(json.dumps(cfg.to_dict(), indent=1))
