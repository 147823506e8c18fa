"""Mozidra: a decoder of windowed softmax-attention layers over hyper-connected residual streams, every layer with a
group-routed mixture of clamped experts.

Residual streams. Instead of one residual x the model carries ``streams`` copies x_1 .. x_S (all equal to the
embedding at the start). A sublayer (mixer or feed-forward) with coefficients a (read, [S]), M (mix, [S, S], indexed
[from, to]) and b (write, [S]) does

    u = sum_s a_s x_s      y = sublayer(rms_norm(u) * (1 + w))      x_r <- sum_s M[s, r] x_s + b_r y   (all r at once)

and the model's output reads the sum of the streams through the final norm (weights stored around zero: 1 + w). A
config without ``streams`` is the plain pre-norm residual, which is the same computation with S = 1 and a = M = b = 1.

Mixers
  attention         grouped-query softmax attention: q, k, v projections with biases; RMS norm over the WHOLE q and the
                    whole k projection (plain weights) before they are split into heads; rotation of dimension pairs
                    (2i, 2i + 1), i < rot.dims / 2, by position * base^(-2i / rot.dims); a sliding window (row i sees
                    keys j with 0 <= i - j < mask.size); a per-head sink logit that joins the softmax denominator only.
                    Layers marked ``v_mix`` after the first such layer cache (1 - l) v + l v_first, v_first being the
                    first marked layer's values of the same token.
  latent_attention  one RMS-normed latent row c (kv_rank) per token is cached; keys and values per head are W_uk c and
                    W_uv c. No positions. The engine attends in the latent space (q_lat = W_uk^T q per head, scores
                    q_lat . c, output W_uv (sum p c)), with the same window and sink.
Feed-forward      router logits in fp32 -> softmax over all experts s; the choice adds a per-expert correction to s and
                  only looks at the experts of the ``groups.keep`` best of ``groups.count`` groups of neighbours (a
                  group scores its largest corrected value); the ``top`` chosen experts weigh s / (sum of the chosen s +
                  1e-20). Expert: W_down (g' sigmoid(1.702 g') (u' + 1)) with g' = min(W_gate h, limit), u' = W_up h
                  clamped to +-limit. A shared expert of the same form runs for every row, times sigmoid(w_sg . h).

Per sequence the engine keeps pages only (no recurrent state): the latent rows of every latent-attention layer, the
keys and page-wise transposed values of every attention layer; page ids are shared by all layers. Pages behind every
window stay allocated until the request ends. The streams, norms, rotation, scores, softmax, router and the stream
arithmetic are fp32; projections run in the model dtype (bf16, or fp32 throughout).

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
from kafka_llm_service_amd.models.budurax import SegMeta, rotary_table
from kafka_llm_service_amd.ops import hybrid as hops

PAGE = 16
SWISH_ALPHA = 1.702       # the experts' gate is g sigmoid(SWISH_ALPHA g)
ROUTE_EPS = 1e-20         # added to the sum of the chosen scores before the division


@dataclass
class MozidraConfig:
    name: str = "mozidra"
    arch: str = "mozidra"
    vocab_size: int = 0
    hidden_size: int = 0
    layers: list = field(default_factory=list)   # config.json's entries: {"type", "mixer": {...}, "mlp": {...}|None}
    norm_eps: float = 1e-5
    streams: int = 0                             # residual streams; 0 = the config has none (plain residual)
    max_position_embeddings: int = 1 << 20
    bos_token_id: int = 0
    eos_token_ids: list = field(default_factory=list)
    tie_word_embeddings: bool = False
    num_experts: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_dict(c: dict, name: str = "mozidra") -> "MozidraConfig":
        return MozidraConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                             layers=list(c["layers"]), norm_eps=float(c["norm"]["eps"]),
                             streams=int(c.get("streams") or 0))

    @staticmethod
    def from_json(path: str | Path) -> "MozidraConfig":
        path = Path(path)
        return MozidraConfig.from_dict(json.loads(path.read_text()), name=path.parent.name)

    def to_dict(self) -> dict:
        d = {"architecture": "Mozidra", "vocab": self.vocab_size, "width": self.hidden_size, "layers": self.layers,
             "norm": {"eps": self.norm_eps}}
        if self.streams:
            d["streams"] = self.streams
        return d

    def num_params(self) -> int:
        return sum(math.prod(s) for s in tensor_shapes(self).values())


def _moe_sizes(mlp: dict) -> dict:
    """Sizes and constants of a layer's feed-forward entry."""
    if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
    r = mlp["router"]
    gr = r.get("groups") or {}
    sh = mlp.get("shared") or None
    return {"E": int(r["experts"]), "top": int(r["top"]), "ff": int(mlp["expert"]["ff"]),
            "limit": float(mlp["expert"]["limit"]), "groups": int(gr.get("count", 1)), "keep": int(gr.get("keep", 1)),
            "shared_ff": int(sh["ff"]) if sh else 0, "shared_limit": float(sh["limit"]) if sh else 0.0}


def tensor_shapes(cfg: MozidraConfig) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a model with this config."""
    d, V, S = cfg.hidden_size, cfg.vocab_size, cfg.streams
    s: dict[str, tuple] = {"embed": (V, d)}
    for i, L in enumerate(cfg.layers):
        p, m = f"l{i}.", L["mixer"]
        s[p + "norm1"] = (d,)
        if L["type"] == "attention":
            H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
            for n, rows in (("q", H * D), ("k", G * D), ("v", G * Dv)):
                s[p + "mix." + n] = (rows, d)
                s[p + "mix." + n + ".b"] = (rows,)
            s[p + "mix.q.norm"], s[p + "mix.k.norm"] = (H * D,), (G * D,)
            if m.get("v_mix"):
                s[p + "mix.vmix"] = ()
            s[p + "mix.sink"] = (H,)
            s[p + "mix.o"] = (d, H * Dv)
        elif L["type"] == "latent_attention":
            H, D, Dv, R = (int(m[k]) for k in ("heads", "dim", "vdim", "kv_rank"))
            s[p + "mix.q"] = (H * D, d)
            s[p + "mix.dkv"], s[p + "mix.dkv.norm"] = (R, d), (R,)
            s[p + "mix.uk"], s[p + "mix.uv"] = (H * D, R), (H * Dv, R)
            s[p + "mix.sink"] = (H,)
            s[p + "mix.o"] = (d, H * Dv)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        subs = ["hc1"]
        if L.get("mlp"):
            z = _moe_sizes(L["mlp"])
            s[p + "norm2"] = (d,)
            for e in range(z["E"]):
                q = f"{p}mlp.e{e}."
                s[q + "gate"], s[q + "up"], s[q + "down"] = (z["ff"], d), (z["ff"], d), (d, z["ff"])
            s[p + "mlp.router"], s[p + "mlp.correction"] = (z["E"], d), (z["E"],)
            if z["shared_ff"]:
                q, fs = p + "mlp.shared.", z["shared_ff"]
                s[q + "gate"], s[q + "up"], s[q + "down"], s[q + "sg"] = (fs, d), (fs, d), (d, fs), (1, d)
            subs.append("hc2")
        if S:
            for q in subs:
                s[p + q + ".in"], s[p + q + ".out"], s[p + q + ".mix"] = (S,), (S,), (S, S)
    s["final.norm"], s["head"] = (d,), (V, d)
    return s


def random_tensors(cfg: MozidraConfig, seed: int = 0, device="cpu") -> dict[str, torch.Tensor]:
    """Seeded bf16 weights with the value ranges each kind of tensor needs (norm weights around zero, stream mixes
    near the identity, read / write weights that keep the streams' size), drawn on ``device``."""
    g = torch.Generator(device=device).manual_seed(seed)

    def rn(shape):
        return torch.randn(shape, generator=g, device=device)

    S = max(1, cfg.streams)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2") or name == "final.norm":
            t = 0.1 * rn(shape)
        elif name.endswith("q.norm") or name.endswith("k.norm") or name.endswith("dkv.norm"):
            t = 1.0 + 0.1 * rn(shape)
        elif leaf == "b":
            t = 0.1 * rn(shape)
        elif leaf == "sink":
            t = rn(shape)
        elif leaf == "vmix":
            t = 0.3 + 0.1 * rn(shape)
        elif leaf == "correction":
            t = 0.05 * rn(shape)
        elif leaf == "in":
            t = (1.0 + 0.2 * rn(shape)) / S
        elif leaf == "out":
            t = 1.0 + 0.2 * rn(shape)
        elif leaf == "mix":
            t = torch.eye(S, device=device) + 0.1 * rn(shape)
        elif leaf == "embed":
            t = rn(shape)
        elif leaf == "router":
            t = rn(shape) * 2.0 / math.sqrt(shape[-1])
        else:
            t = rn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


class PageState:
    """The per-slot state of a model that keeps none: the engine's slot bookkeeping stays as for the other segment
    models."""

    def nbytes(self) -> int:
        return 0


class _Layer:
    pass


class _Streams:
    """Coefficients of one sublayer's stream step on the device (fp32): read [S], mix [S, S] ([from, to]), write [S]."""

    def __init__(self, a, M, b):
        self.a, self.M, self.b = a, M, b


class MozidraLM:
    plan = "segments"  # the model runner plans its steps as SegMeta runs (engine/model_runner.py)

    def __init__(self, cfg: MozidraConfig, device, dtype=torch.bfloat16, tp: int = 1, tp_rank: int = 0,
                 max_positions: int | None = None):
        if tp != 1:
            raise ValueError("Mozidra runs unsharded (tp = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Mozidra runs in bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.tp, self.tp_rank, self.ep, self.ep_rank = 1, 0, 1, 0
        self.dp_attention = False
        self.stream = self.tiled_only = False
        self.stream_max_m = 0
        self.max_positions = int(max_positions or 8192)
        self.layers: list[_Layer] = []
        self.attn_tile_tokens: list[int] = []
        self._rot: dict = {}

    # engine hooks shared with the other model classes ---------------------------------------------------------------
    STREAMED = ("w_in", "o", "sh_gu", "sh_down")

    def _streamable(self, w) -> bool:
        return w is not None and w.dtype == torch.bfloat16 and w.is_cuda and \
            ops.stream_plan(1, w.shape[0], w.shape[1]) is not None

    def stream_weight_bytes(self) -> int:
        ws = [getattr(lw, n, None) for lw in self.layers for n in self.STREAMED] + [self.head]
        return sum(w.numel() * w.element_size() for w in ws if self._streamable(w))

    def enable_stream_weights(self, tiled_only: bool = False) -> int:
        """Wave-tiled copies of the projections (ops.tile_weight) and of the experts (ops.tile_experts) so that
        decode-sized steps (<= ops.STREAM_MAX_M rows; experts: <= hops.MOE_STREAM_MAX_T) run them on the framework's
        weight-streaming MFMA kernels; prefill-sized steps and shapes the kernels do not take stay on hipBLASLt and
        the expert-sorted GEMMs. bf16 only. Returns the added bytes."""
        added = 0
        for lw in self.layers:
            for n in self.STREAMED:
                w = getattr(lw, n, None)
                if self._streamable(w):
                    setattr(lw, n + "_t", ops.tile_weight(w))
                    added += w.numel() * w.element_size()
            if lw.z is not None and lw.w_gu.is_cuda and lw.w_gu.dtype == torch.bfloat16 and \
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
    def load_tensors(self, W: dict[str, torch.Tensor]) -> "MozidraLM":
        """Checkpoint tensors (any float dtype) -> device tensors: projections that read the same input fused into
        one GEMM weight in the model dtype, per-head up-projections reshaped for the batched latent products, experts
        stacked; norm weights (as 1 + w), stream coefficients, sinks, the router (with the shared expert's gate row
        appended) and its correction kept in fp32."""
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

        def plus_one(name):
            return keep(1.0 + W[name].to(device=dev, dtype=torch.float32))

        def fused(names, dtype=dt):
            return keep(torch.cat([W[n].to(device=dev, dtype=dtype) for n in names], 0))

        def streams(prefix):
            if cfg.streams:
                return _Streams(f32(prefix + ".in"), f32(prefix + ".mix"), f32(prefix + ".out"))
            one = torch.ones(1, dtype=torch.float32, device=dev)
            return _Streams(one, one.view(1, 1), one)

        d = cfg.hidden_size
        self.S = max(1, cfg.streams)
        self.embed = f32("embed")  # the streams start (and stay) fp32; bf16 table values are exact in it
        self.final_norm = plus_one("final.norm")
        self.sum_in = keep(torch.ones(self.S, dtype=torch.float32, device=dev))   # the output reads the plain sum
        # the sampler reads logits rows in 8-element vectors: the head is padded with zero rows to a multiple of 8
        # and the extra columns are cut off as a view
        pad = -cfg.vocab_size % 8
        hw = W["head"].to(device=dev, dtype=dt)
        self.head = keep(torch.cat([hw, torch.zeros(pad, d, dtype=dt, device=dev)], 0))
        self.layers = []
        first_vmix = None
        for i, L in enumerate(cfg.layers):
            p, m = f"l{i}.", L["mixer"]
            lw = _Layer()
            lw.type, lw.m = L["type"], m
            lw.norm1, lw.hc1 = plus_one(p + "norm1"), streams(p + "hc1")
            mask = m.get("mask") or {}
            lw.window = int(mask["size"]) if mask.get("size") is not None else 0   # 0 = every earlier position
            if mask.get("size") is not None and lw.window < 1:
                raise ValueError(f"layer {i}: mask.size must be at least 1")
            lw.scale = float(m["scale"])
            lw.sink = f32(p + "mix.sink")
            if lw.type == "attention":
                H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
                if G < 1 or H % G:
                    raise ValueError(f"layer {i}: {H} query heads over {G} key/value heads")
                lw.w_in = fused([p + "mix.q", p + "mix.k", p + "mix.v"])
                lw.b_in = fused([p + "mix.q.b", p + "mix.k.b", p + "mix.v.b"])
                lw.q_norm, lw.k_norm = f32(p + "mix.q.norm"), f32(p + "mix.k.norm")
                rot = m.get("rot") or None
                lw.rot_dims = int(rot["dims"]) if rot else 0
                if lw.rot_dims > D or lw.rot_dims % 2:
                    raise ValueError(f"layer {i}: rot.dims must be even and at most the head size")
                lw.cos_sin = self._rot_table(rot) if lw.rot_dims else None
                lw.vmix_from, lw.lam = None, 0.0
                if m.get("v_mix"):
                    if first_vmix is None:
                        first_vmix = i
                    else:
                        fm = cfg.layers[first_vmix]["mixer"]
                        if int(fm["kv_heads"]) * int(fm["vdim"]) != G * Dv:
                            raise ValueError(f"layer {i}: its values and layer {first_vmix}'s differ in size")
                        lw.vmix_from, lw.lam = first_vmix, float(W[p + "mix.vmix"].float())
                lw.o = act(p + "mix.o")
            else:
                H, D, Dv, R = (int(m[k]) for k in ("heads", "dim", "vdim", "kv_rank"))
                lw.w_in = fused([p + "mix.q", p + "mix.dkv"])                      # row = [q heads | latent]
                lw.dkv_norm = act(p + "mix.dkv.norm")
                lw.uk_h = act(p + "mix.uk").view(H, D, R)                          # q_lat = q @ uk_h  (per head)
                lw.uv_ht = keep(W[p + "mix.uv"].to(device=dev, dtype=dt).view(H, Dv, R).transpose(1, 2))
                lw.o = act(p + "mix.o")
            if L.get("mlp"):
                z = _moe_sizes(L["mlp"])
                E = z["E"]
                if not 1 <= z["top"] <= E or z["groups"] < 1 or E % z["groups"] or \
                        not 1 <= z["keep"] <= z["groups"] or z["keep"] * (E // z["groups"]) < z["top"]:
                    raise ValueError(f"layer {i}: {z['top']} of {E} experts in {z['keep']} of {z['groups']} groups")
                lw.z = z
                lw.norm2, lw.hc2 = plus_one(p + "norm2"), streams(p + "hc2")
                rows = [p + "mlp.router"] + ([p + "mlp.shared.sg"] if z["shared_ff"] else [])
                lw.router = fused(rows, torch.float32)                              # [E (+ 1), d] fp32
                lw.correction = f32(p + "mlp.correction")
                lw.w_gu = keep(torch.stack([torch.cat([W[f"{p}mlp.e{e}.gate"], W[f"{p}mlp.e{e}.up"]], 0)
                                            for e in range(E)]).to(device=dev, dtype=dt))       # [E, 2 ff, d]
                lw.w_down = keep(torch.stack([W[f"{p}mlp.e{e}.down"] for e in range(E)]).to(device=dev, dtype=dt))
                if z["shared_ff"]:
                    lw.sh_gu = fused([p + "mlp.shared.gate", p + "mlp.shared.up"])
                    lw.sh_down = act(p + "mlp.shared.down")
                else:
                    lw.sh_gu = lw.sh_down = None
            else:
                lw.z = None
            self.layers.append(lw)
        # tile sizes (tokens) the step plan must carry for the matrix-core attention kernels
        self.attn_tile_tokens = sorted({hops.tile_tokens(int(lw.m["heads"])) if lw.type == "latent_attention" else
                                        hops.sig_tile_tokens(int(lw.m["heads"]), int(lw.m["kv_heads"]))
                                        for lw in self.layers})
        return self

    def _rot_table(self, rot: dict) -> torch.Tensor:
        """fp32 [positions, dims]: cos | sin of fp32 position x fp32 frequency, one table per (dims, base)."""
        key = (int(rot["dims"]), float(rot["base"]))
        if key not in self._rot:
            self._rot[key] = rotary_table(self.max_positions, {"dims": key[0], "base": key[1]}, self.device)
        return self._rot[key]

    # caches ---------------------------------------------------------------------------------------------------
    def page_bytes(self) -> int:
        """Bytes of one 16-token page over every layer."""
        es = torch.empty(0, dtype=self.dtype).element_size()
        n = 0
        for L in self.cfg.layers:
            m = L["mixer"]
            if L["type"] == "attention":
                n += int(m["kv_heads"]) * (int(m["dim"]) + int(m["vdim"]))
            else:  # (the latent is kept twice where the matrix-core kernel runs: row-major and page-wise transposed)
                n += 2 * int(m["kv_rank"])
        return PAGE * n * es or 1

    def alloc_cache(self, num_blocks: int, num_slots: int):
        """(per layer: the latent pool [blocks, 16, kv_rank], or (keys [blocks, 16, G dim], values [blocks, G vdim,
        16]); no slot state). Zeroed once: a masked key's row is never used, but fresh memory must not hold NaN
        patterns for the debug checks."""
        dev, dt = self.device, self.dtype
        pages = []
        self.pages_t = []  # page-wise transposed latent copies [blocks, kv_rank, 16] for the matrix-core kernel
        for lw in self.layers:
            m = lw.m
            if lw.type == "attention":
                G, D, Dv = (int(m[k]) for k in ("kv_heads", "dim", "vdim"))
                pages.append((torch.zeros(num_blocks, PAGE, G * D, dtype=dt, device=dev),
                              torch.zeros(num_blocks, G * Dv, PAGE, dtype=dt, device=dev)))
                self.pages_t.append(None)
            else:
                R = int(m["kv_rank"])
                pages.append(torch.zeros(num_blocks, PAGE, R, dtype=dt, device=dev))
                self.pages_t.append(torch.zeros(num_blocks, R, PAGE, dtype=dt, device=dev)
                                    if hops.latent_mfma_ok(pages[-1], R, 0) else None)
        return pages, PageState()

    # one step ---------------------------------------------------------------------------------------------------
    def forward(self, inp, pages: list, state: PageState, gather: bool = True,
                layers_out: list | None = None) -> torch.Tensor:
        """Logits fp32 [n, V] for ``inp.logit_rows``. ``layers_out``: a list that receives the sum of the streams
        after every layer (fp32 [T, d] copies; debugging and the per-layer tests)."""
        cfg, dt, dev = self.cfg, self.dtype, self.device
        m: SegMeta = inp.attn
        T, d, eps, S = inp.tokens.shape[0], cfg.hidden_size, cfg.norm_eps, self.S
        xs = F.embedding(inp.tokens, self.embed).unsqueeze(0).repeat(S, 1, 1)   # fp32 [S, T, d] streams
        h = torch.empty(T, d, dtype=dt, device=dev)
        step = {}   # what later layers of this step read from earlier ones (the first value-mixing layer's values)
        if self.layers:
            lw = self.layers[0]
            hops.stream_step(xs, read=lw.hc1.a, norm_w=lw.norm1, eps=eps, out=h)
        for i, lw in enumerate(self.layers):
            y = self._attention(i, lw, h, inp, m, pages, step) if lw.type == "attention" else \
                self._latent_attention(i, lw, h, inp, m, pages)
            nxt = self.layers[i + 1] if i + 1 < len(self.layers) else None
            total = torch.empty(T, d, dtype=torch.float32, device=dev) if layers_out is not None else None
            if lw.z is not None:
                # the mixer's write, the feed-forward's read and its norm in one pass over the streams
                hops.stream_step(xs, y, lw.hc1.M, lw.hc1.b, lw.hc2.a, lw.norm2, eps, h)
                ye, ys, gate = self._experts(lw, h)
                last = lw.hc2
            else:
                ye, ys, gate, last = y, None, None, lw.hc1
            if nxt is not None:
                hops.stream_step(xs, ye, last.M, last.b, nxt.hc1.a, nxt.norm1, eps, h, y2=ys, row_scale=gate,
                                 total=total)
            else:
                hops.stream_step(xs, ye, last.M, last.b, y2=ys, row_scale=gate, total=total)
            if layers_out is not None:
                layers_out.append(total)
        xsel = xs.index_select(1, inp.logit_rows)
        hf = torch.empty(xsel.shape[1], d, dtype=dt, device=dev)
        hops.stream_step(xsel, read=self.sum_in, norm_w=self.final_norm, eps=eps, out=hf)
        return self._lin(hf, self.head, getattr(self, "head_t", None)).float()[:, :cfg.vocab_size]

    def _attention(self, i: int, lw, h, inp, m: SegMeta, pages: list, step: dict) -> torch.Tensor:
        mm = lw.m
        H, G, D, Dv = (int(mm[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        T, dt, dev = h.shape[0], self.dtype, self.device
        qkv = self._lin(h, lw.w_in, getattr(lw, "w_in_t", None), lw.b_in)   # [q | k | v], biases added
        k_cache, v_cache_t = pages[i]
        q = torch.empty(T, H * D, dtype=dt, device=dev)
        vf = step.get(lw.vmix_from) if lw.vmix_from is not None else None          # (rows, first value column)
        hops.qk_norm_rope_store(qkv, H, G, D, Dv, lw.q_norm, lw.k_norm, self.cfg.norm_eps, inp.positions, lw.cos_sin,
                                lw.rot_dims, vf[0] if vf else None, vf[1] if vf else 0, lw.lam, k_cache, v_cache_t,
                                inp.slot_mapping, q)
        if mm.get("v_mix") and lw.vmix_from is None:
            step[i] = (qkv, H * D + G * D)
        ao = torch.empty(T, H * Dv, dtype=dt, device=dev)
        hops.window_attn(q, k_cache, v_cache_t, m.block_tables, m.tok_seg, inp.positions, H, G, lw.scale, lw.window,
                         lw.sink, ao, m.tiles.get(hops.sig_tile_tokens(H, G)), m.max_keys)
        return self._lin(ao, lw.o, getattr(lw, "o_t", None))

    def _latent_attention(self, i: int, lw, h, inp, m: SegMeta, pages: list) -> torch.Tensor:
        mm = lw.m
        H, D, Dv, R = (int(mm[k]) for k in ("heads", "dim", "vdim", "kv_rank"))
        T, dt, dev = h.shape[0], self.dtype, self.device
        qd = self._lin(h, lw.w_in, getattr(lw, "w_in_t", None))                    # [q heads | latent]
        cache, cache_t = pages[i], self.pages_t[i]
        q_rot = torch.empty(T, H, 0, dtype=dt, device=dev)                         # (no rotated part in this family)
        hops.latent_prep(qd, H, D, 0, R, H * D, lw.dkv_norm, self.cfg.norm_eps, inp.positions, None, 0, cache,
                         inp.slot_mapping, q_rot, cache_t)
        q_u = qd[:, :H * D].view(T, H, D).transpose(0, 1)                          # [H, T, dim] (strided view)
        q_lat = torch.bmm(q_u, lw.uk_h)                                            # [H, T, R]
        o_lat = torch.empty(H, T, R, dtype=dt, device=dev)
        hops.latent_attn(q_lat, q_rot, cache, m.block_tables, m.tok_seg, m.seg, inp.positions, lw.scale, o_lat,
                         cache_t, m.tiles.get(hops.tile_tokens(H)), m.max_keys, window=lw.window, sink=lw.sink)
        ao = torch.empty(T, H * Dv, dtype=dt, device=dev)
        torch.bmm(o_lat, lw.uv_ht, out=ao.view(T, H, Dv).transpose(0, 1))          # head h -> its vdim columns
        return self._lin(ao, lw.o, getattr(lw, "o_t", None))

    def _experts(self, lw, h):
        """(routed experts' weighted sum fp32 [T, d], shared expert's output [T, d] or None, its gate fp32 [T])."""
        z = lw.z
        T, d, dt, dev = h.shape[0], self.cfg.hidden_size, self.dtype, self.device
        tw, te, gate = hops.moe_router_grouped(h, lw.router, lw.correction, z["top"], z["groups"], z["keep"],
                                               ROUTE_EPS, extra_gate=lw.sh_gu is not None)
        out = torch.empty(T, d, dtype=torch.float32, device=dev)
        hops.moe_experts(h, lw.w_gu, lw.w_down, tw, te, out, getattr(lw, "w_gu_t", None), getattr(lw, "w_down_t", None),
                         act="swish_clamp", limit=z["limit"], alpha=SWISH_ALPHA)
        ys = None
        if lw.sh_gu is not None:
            a = torch.empty(T, z["shared_ff"], dtype=dt, device=dev)
            hops.swish_clamp_mul(self._lin(h, lw.sh_gu, getattr(lw, "sh_gu_t", None)), z["shared_limit"], SWISH_ALPHA,
                                 a)
            ys = self._lin(a, lw.sh_down, getattr(lw, "sh_down_t", None))
        return out, ys, gate


def load_checkpoint(model: MozidraLM, path: str | Path) -> MozidraLM:
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


def save_checkpoint(cfg: MozidraConfig, W: dict[str, torch.Tensor], folder: str | Path) -> None:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in W.items()}, str(folder / "model.safetensors"))
    (folder / "config.json").write_text(json.dumps(cfg.to_dict(), indent=1))
