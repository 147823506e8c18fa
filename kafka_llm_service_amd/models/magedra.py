"""Magedra: a hybrid decoder over hyper-connected residual streams whose mixers are gated recurrences and softmax
attention, side by side or in turn, every layer with a clamped dense feed-forward.

Residual. ``streams`` copies x_1 .. x_S of the residual (all equal to the normed embedding at the start). A sublayer
(mixer or feed-forward) with coefficients a (read, [S]), M (mix, [S, S], indexed [from, to]) and b (write, [S]) does

    u = sum_s a_s x_s      y = sublayer(layer_norm(u) * w)      x_r <- sum_s M[s, r] x_s + mult * b_r * y   (all r at once)

with ``mult`` = config residual_mult and a layer norm that has a weight and no bias; the output reads the sum of the
streams through the same kind of norm and multiplies the logits by ``logit_scale``. A config without ``streams`` is
the plain pre-norm residual x += mult * y (S = 1, a = M = b = 1). The embedding rows pass through a layer norm too.

Mixers
  mingru            z = sigmoid(W_z h + b_z), u = W_x h + b_x, candidate c = u + 1/2 (u >= 0) or sigmoid(u) (u < 0);
                    S <- (1 - z) S + z c per channel; output W_o (S silu(W_g h)).
  parallel          two mixers read the same input, result = left_scale * left + right_scale * right.
                    left: grouped-query softmax attention; rotation of dimension i with i + rot.dims / 2 on the first
                    rot.dims dimensions of every q and k head; the scaled scores are mixed over the heads before the
                    softmax, s'_h = sum_g talk[h, g] s_g; the heads' outputs times sigmoid(W_g h), then W_o.
                    right: HGRN2 - q = silu(W_q h), forget gate f = l + (1 - l) sigmoid(W_f h + b_f) per head and key
                    channel with a learned lower bound l, S <- diag(f) S + (1 - f) v^T, read-out S^T q, RMS norm per
                    head (one weight vector for all heads), then W_o.
  latent_attention  queries through a normed latent (c_q = rms_norm(W_dq h), q = W_uq c_q, per head [dim | rot_dim]);
                    per token one RMS-normed latent row c (kv_rank) and one rotated key part (rot_dim, shared by all
                    heads; dimension 2i turns with 2i + 1) are cached; keys / values per head are W_uk c / W_uv c. The
                    engine attends in the latent space (q_lat = W_uk^T q per head, scores q_lat . c + q_rot . k_rot,
                    output W_uv (sum p c)).
Feed-forward      g = min(W_gate h + b, limit), u = clamp(W_up h + b, +-limit), W_down (g sigmoid(1.702 g) (u + 1)) + b.

A layer with ``weights_of: j`` runs layer j's tensors on a cache and state of its own.

How the head mix reaches the attention kernels: the mix is linear in the queries, so the attention-input kernel
(``ops.hybrid.rope_kv_store``) leaves for every head h the row q'[h] = [sum_{g in key head c} talk[h, g] q[g]]_c of the
whole key row's size, and q'[h] . (k_0 | .. | k_{G-1}) = s'_h. The windowed-attention kernels then run with
``shared_keys`` (all G key heads of a token are one key; values stay per key/value head).

The pair rotation of the latent layers runs on the kernel that turns dimension i with i + dims / 2: the rows of W_uq's
rotated parts and of W_dkv's key part are reordered at load (even members first, odd members second), which changes
no score because q and k are permuted alike.

Per sequence the engine keeps pages (latent rows of every latent layer; keys and page-wise transposed values of every
parallel layer; page ids shared by all layers) and one state slot (the minGRU vector, the HGRN2 matrices, fp32). The
streams, norms, rotation, scores, softmax, gates, candidates and states are fp32; projections run in the model dtype
(bf16, or fp32 throughout).

Steps are planned as segments (``SegMeta``, models/budurax.py): one run of consecutive rows per sequence, a decoded
token being a run of one, so prompt portions and single tokens go through the same kernels.
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path

import numpy as np
import torch
import torch.nn.functional as F

from kafka_llm_service_amd import ops
from kafka_llm_service_amd.models.budurax import SegMeta, rotary_table
from kafka_llm_service_amd.ops import hybrid as hops

PAGE = 16
SWISH_ALPHA = 1.702       # the feed-forward's gate is g sigmoid(SWISH_ALPHA g)
MIXERS = ("mingru", "parallel", "latent_attention")


@dataclass
class MagedraConfig:
    name: str = "magedra"
    arch: str = "magedra"
    vocab_size: int = 0
    hidden_size: int = 0
    layers: list = field(default_factory=list)   # config.json's entries: {"type", "mixer", "mlp"|None, "weights_of"?}
    norm_eps: float = 1e-6
    streams: int = 0                             # residual streams; 0 = the config has none (plain residual)
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    max_position_embeddings: int = 1 << 20
    bos_token_id: int = 0
    eos_token_ids: list = field(default_factory=list)
    tie_word_embeddings: bool = False
    num_experts: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    @staticmethod
    def from_dict(c: dict, name: str = "magedra") -> "MagedraConfig":
        return MagedraConfig(name=name, vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                             layers=list(c["layers"]), norm_eps=float(c["norm"]["eps"]),
                             streams=int(c.get("streams") or 0), residual_mult=float(c.get("residual_mult", 1.0)),
                             logit_scale=float(c.get("logit_scale", 1.0)))

    @staticmethod
    def from_json(path: str | Path) -> "MagedraConfig":
        path = Path(path)
        return MagedraConfig.from_dict(json.loads(path.read_text()), name=path.parent.name)

    def to_dict(self) -> dict:
        d = {"architecture": "Magedra", "vocab": self.vocab_size, "width": self.hidden_size, "layers": self.layers,
             "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "logit_scale": self.logit_scale}
        if self.streams:
            d["streams"] = self.streams
        return d

    def owner(self, i: int) -> int:
        """The layer whose tensors layer i runs."""
        j = self.layers[i].get("weights_of")
        return i if j is None else int(j)

    def num_params(self) -> int:
        return sum(math.prod(s) for s in tensor_shapes(self).values())


def _ff_sizes(mlp: dict) -> tuple[int, float]:
    if mlp.get("kind", "dense") != "dense":
        raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
    return int(mlp["ff"]), float(mlp["limit"])


def tensor_shapes(cfg: MagedraConfig) -> dict[str, tuple]:
    """Checkpoint tensor names -> shapes of a model with this config (layers with ``weights_of`` own none)."""
    d, V, S = cfg.hidden_size, cfg.vocab_size, cfg.streams
    s: dict[str, tuple] = {"embed": (V, d), "embed.norm": (d,)}
    for i, L in enumerate(cfg.layers):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", L["mixer"]
        s[p + "norm1"] = (d,)
        if L["type"] == "mingru":
            Wd = int(m["width"])
            for n in ("z", "x", "g"):
                s[p + "mix." + n] = (Wd, d)
            s[p + "mix.z.b"], s[p + "mix.x.b"] = (Wd,), (Wd,)
            s[p + "mix.o"] = (d, Wd)
        elif L["type"] == "parallel":
            a, b = m["left"], m["right"]
            H, G, D, Dv = (int(a[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
            q = p + "mix.left."
            s[q + "q"], s[q + "k"], s[q + "v"] = (H * D, d), (G * D, d), (G * Dv, d)
            s[q + "talk"], s[q + "g"], s[q + "o"] = (H, H), (H * Dv, d), (d, H * Dv)
            Hr, Dr, Dvr = (int(b[k]) for k in ("heads", "dim", "vdim"))
            q = p + "mix.right."
            s[q + "q"], s[q + "f"], s[q + "f.b"], s[q + "lower"] = (Hr * Dr, d), (Hr * Dr, d), (Hr * Dr,), (Hr * Dr,)
            s[q + "v"], s[q + "norm"], s[q + "o"] = (Hr * Dvr, d), (Dvr,), (d, Hr * Dvr)
        elif L["type"] == "latent_attention":
            H, D, rd, Dv, R, Rq = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
            q = p + "mix."
            s[q + "dq"], s[q + "dq.norm"], s[q + "uq"] = (Rq, d), (Rq,), (H * (D + rd), Rq)
            s[q + "dkv"], s[q + "dkv.norm"] = (R + rd, d), (R,)
            s[q + "uk"], s[q + "uv"], s[q + "o"] = (H * D, R), (H * Dv, R), (d, H * Dv)
        else:
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        subs = ["hc1"]
        if L.get("mlp"):
            ff, _ = _ff_sizes(L["mlp"])
            s[p + "norm2"] = (d,)
            q = p + "mlp."
            s[q + "gate"], s[q + "gate.b"], s[q + "up"], s[q + "up.b"] = (ff, d), (ff,), (ff, d), (ff,)
            s[q + "down"], s[q + "down.b"] = (d, ff), (d,)
            subs.append("hc2")
        if S:
            for q in subs:
                s[p + q + ".in"], s[p + q + ".out"], s[p + q + ".mix"] = (S,), (S,), (S, S)
    s["final.norm"], s["head"] = (d,), (V, d)
    return s


def random_tensors(cfg: MagedraConfig, seed: int = 0, device="cpu") -> dict[str, torch.Tensor]:
    """Seeded bf16 weights with the value ranges each kind of tensor needs (norm weights around one, stream mixes
    near the identity, read weights that keep the streams' size, lower bounds inside (0, 1), a head mix near the
    identity), drawn on ``device``."""
    g = torch.Generator(device=device).manual_seed(seed)

    def rn(shape):
        return torch.randn(shape, generator=g, device=device)

    S = max(1, cfg.streams)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.split(".")[-1]
        if leaf in ("norm1", "norm2", "norm") or name in ("final.norm", "embed.norm"):
            t = 1.0 + 0.1 * rn(shape)
        elif leaf == "b":
            t = 0.1 * rn(shape)
        elif leaf == "lower":
            t = torch.rand(shape, generator=g, device=device) * 0.9
        elif leaf == "talk":
            t = torch.eye(shape[0], device=device) + 0.3 * rn(shape) / math.sqrt(shape[0])
        elif leaf == "in":
            t = (1.0 + 0.2 * rn(shape)) / S
        elif leaf == "out":
            t = 1.0 + 0.2 * rn(shape)
        elif leaf == "mix":
            t = torch.eye(S, device=device) + 0.1 * rn(shape)
        elif leaf == "embed":
            t = rn(shape)
        else:
            t = rn(shape) / math.sqrt(shape[-1])
        out[name] = t.to(torch.bfloat16)
    return out


class LayerState:
    """Per-layer dicts of state tensors, one row per state slot (empty for layers that keep none)."""

    def __init__(self):
        self.layers: list[dict] = []

    def nbytes(self) -> int:
        return sum(t.numel() * t.element_size() for st in self.layers for t in st.values())


class _Weights:
    pass


class _Streams:
    """Coefficients of one sublayer's stream step on the device (fp32): read [S], mix [S, S] ([from, to]), write [S]
    (the residual multiplier folded in)."""

    def __init__(self, a, M, b):
        self.a, self.M, self.b = a, M, b


def _halves_order(n: int, dims: int) -> torch.Tensor:
    """Row order that moves the pair rotation's layout (2i with 2i + 1 over the first ``dims`` of ``n`` rows) to the
    layout of the rotation that turns i with i + dims / 2: even members, odd members, the rest."""
    return torch.tensor(list(range(0, dims, 2)) + list(range(1, dims, 2)) + list(range(dims, n)), dtype=torch.long)


class MagedraLM:
    plan = "segments"  # the model runner plans its steps as SegMeta runs (engine/model_runner.py)

    def __init__(self, cfg: MagedraConfig, device, dtype=torch.bfloat16, tp: int = 1, tp_rank: int = 0,
                 max_positions: int | None = None):
        if tp != 1:
            raise ValueError("Magedra runs unsharded (tp = 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Magedra runs in bfloat16 or float32")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.tp, self.tp_rank, self.ep, self.ep_rank = 1, 0, 1, 0
        self.dp_attention = False
        self.stream = self.tiled_only = False
        self.stream_max_m = 0
        self.max_positions = int(max_positions or 8192)
        self.layers: list[_Weights] = []          # one entry per layer; layers with ``weights_of`` share an object
        self.attn_tile_tokens: list[int] = []
        self._rot: dict = {}

    # engine hooks shared with the other model classes ---------------------------------------------------------------
    STREAMED = ("w_in", "uq", "o", "gate_up", "down")

    def _owned(self):
        return [lw for i, lw in enumerate(self.layers) if self.cfg.owner(i) == i]

    def _streamable(self, w) -> bool:
        return w is not None and w.dtype == torch.bfloat16 and w.is_cuda and \
            ops.stream_plan(1, w.shape[0], w.shape[1]) is not None

    def stream_weight_bytes(self) -> int:
        ws = [getattr(lw, n, None) for lw in self._owned() for n in self.STREAMED] + [self.head]
        return sum(w.numel() * w.element_size() for w in ws if self._streamable(w))

    def enable_stream_weights(self, tiled_only: bool = False) -> int:
        """Wave-tiled copies of the projections (ops.tile_weight) so that decode-sized steps (<= ops.STREAM_MAX_M
        rows) run them on the framework's weight-streaming MFMA GEMM; prefill-sized steps and shapes the kernel does
        not take stay on hipBLASLt. bf16 only. Returns the added bytes."""
        added = 0
        for lw in self._owned():
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
    def load_tensors(self, W: dict[str, torch.Tensor]) -> "MagedraLM":
        """Checkpoint tensors (any float dtype) -> device tensors: projections that read the same input fused into
        one GEMM weight in the model dtype (the parallel mixer's seven, its two output projections side by side along
        the input), per-head up-projections reshaped for the batched latent products; norm weights, stream
        coefficients (write weights times the residual multiplier), the head mix, gate biases and lower bounds fp32."""
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

        mult = cfg.residual_mult

        def streams(prefix):
            if cfg.streams:
                return _Streams(f32(prefix + ".in"), f32(prefix + ".mix"),
                                keep(mult * W[prefix + ".out"].to(device=dev, dtype=torch.float32)))
            one = torch.ones(1, dtype=torch.float32, device=dev)
            return _Streams(one, one.view(1, 1), keep(mult * one))

        d = cfg.hidden_size
        self.S = max(1, cfg.streams)
        self.embed = f32("embed")  # the streams start (and stay) fp32; bf16 table values are exact in it
        self.embed_norm, self.final_norm = f32("embed.norm"), f32("final.norm")
        self.one = keep(torch.ones(1, dtype=torch.float32, device=dev))
        self.sum_in = keep(torch.ones(self.S, dtype=torch.float32, device=dev))   # the output reads the plain sum
        # the sampler reads logits rows in 8-element vectors: the head is padded with zero rows to a multiple of 8
        # and the extra columns are cut off as a view
        pad = -cfg.vocab_size % 8
        hw = W["head"].to(device=dev, dtype=dt)
        self.head = keep(torch.cat([hw, torch.zeros(pad, d, dtype=dt, device=dev)], 0))
        owned: dict[int, _Weights] = {}
        self.layers = []
        tiles = set()
        for i, L in enumerate(cfg.layers):
            j = cfg.owner(i)
            if j != i:
                src = cfg.layers[j] if 0 <= j < len(cfg.layers) else None
                if src is None or src.get("weights_of") is not None or \
                        {k: v for k, v in L.items() if k != "weights_of"} != src:
                    raise ValueError(f"layer {i}: weights_of must name a layer of the same entry that owns its tensors")
                if j not in owned:
                    raise ValueError(f"layer {i}: weights_of names a later layer")
                self.layers.append(owned[j])
                continue
            p, m = f"l{i}.", L["mixer"]
            lw = _Weights()
            lw.type, lw.m = L["type"], m
            lw.norm1, lw.hc1 = f32(p + "norm1"), streams(p + "hc1")
            if lw.type == "mingru":
                lw.w_in = fused([p + "mix.z", p + "mix.x", p + "mix.g"])
                lw.b_in = fused([p + "mix.z.b", p + "mix.x.b"], torch.float32)
                lw.o = act(p + "mix.o")
            elif lw.type == "parallel":
                a, b = m["left"], m["right"]
                H, G, D, Dv = (int(a[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
                Hr, Dr, Dvr = (int(b[k]) for k in ("heads", "dim", "vdim"))
                if G < 1 or H % G:
                    raise ValueError(f"layer {i}: {H} query heads over {G} key/value heads")
                q, r = p + "mix.left.", p + "mix.right."
                lw.w_in = fused([q + "q", q + "k", q + "v", q + "g", r + "q", r + "f", r + "v"])
                lw.g_off = H * D + G * D + G * Dv
                lw.rq_off = lw.g_off + H * Dv
                lw.rf_off, lw.rv_off = lw.rq_off + Hr * Dr, lw.rq_off + 2 * Hr * Dr
                lw.talk = f32(q + "talk")
                rot = a.get("rot") or None
                lw.rot_dims = int(rot["dims"]) if rot else 0
                if lw.rot_dims > D or lw.rot_dims % 2:
                    raise ValueError(f"layer {i}: rot.dims must be even and at most the head size")
                lw.cos_sin = self._rot_table(rot) if lw.rot_dims else None
                lw.scale = float(a["scale"])
                lw.f_bias, lw.lower = f32(r + "f.b"), f32(r + "lower")
                lw.rnorm = keep(W[r + "norm"].to(device=dev, dtype=dt).repeat(Hr))   # one weight vector for all heads
                lw.left_scale, lw.right_scale = float(m["left_scale"]), float(m["right_scale"])
                # both output projections as one product over [left heads | right heads]
                lw.o = keep(torch.cat([W[q + "o"].to(device=dev, dtype=dt), W[r + "o"].to(device=dev, dtype=dt)], 1))
                tiles.add(hops.sig_tile_tokens(H, G))
            else:
                H, D, rd, Dv, R, Rq = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
                rot = m["rot"]
                lw.rot_dims = int(rot["dims"])
                if lw.rot_dims > rd or lw.rot_dims % 2:
                    raise ValueError(f"layer {i}: rot.dims must be even and at most rot_dim")
                # pair layout -> halves layout of the rotated parts (q and k alike: the scores do not change)
                order = _halves_order(rd, lw.rot_dims)
                dkv = W[p + "mix.dkv"]
                dkv = torch.cat([dkv[:R], dkv[R:][order]], 0)
                lw.w_in = keep(torch.cat([W[p + "mix.dq"], dkv], 0).to(device=dev, dtype=dt))   # [c_q | latent | key]
                uq = W[p + "mix.uq"].view(H, D + rd, Rq)
                uq = torch.cat([uq[:, :D], uq[:, D:][:, order]], 1).reshape(H * (D + rd), Rq)
                lw.uq = keep(uq.to(device=dev, dtype=dt))
                lw.dq_norm = f32(p + "mix.dq.norm")
                lw.dkv_norm = act(p + "mix.dkv.norm")
                lw.uk_h = act(p + "mix.uk").view(H, D, R)                          # q_lat = q @ uk_h  (per head)
                lw.uv_ht = keep(W[p + "mix.uv"].to(device=dev, dtype=dt).view(H, Dv, R).transpose(1, 2))
                lw.o = act(p + "mix.o")
                lw.scale = float(m["scale"])
                lw.cos_sin = self._rot_table(rot)
                tiles.add(hops.tile_tokens(H))
            if L.get("mlp"):
                lw.ff, lw.limit = _ff_sizes(L["mlp"])
                if not lw.limit > 0:
                    raise ValueError(f"layer {i}: the feed-forward's limit must be positive")
                lw.norm2, lw.hc2 = f32(p + "norm2"), streams(p + "hc2")
                lw.gate_up = fused([p + "mlp.gate", p + "mlp.up"])
                lw.gate_up_b = fused([p + "mlp.gate.b", p + "mlp.up.b"])
                lw.down, lw.down_b = act(p + "mlp.down"), act(p + "mlp.down.b")
            else:
                lw.ff = 0
            owned[i] = lw
            self.layers.append(lw)
        # tile sizes (tokens) the step plan must carry for the matrix-core attention kernels
        self.attn_tile_tokens = sorted(tiles)
        return self

    def _rot_table(self, rot: dict) -> torch.Tensor:
        """fp32 [positions, dims]: cos | sin of fp32 position x fp32 frequency, one table per (dims, base)."""
        key = (int(rot["dims"]), float(rot["base"]))
        if key not in self._rot:
            self._rot[key] = rotary_table(self.max_positions, {"dims": key[0], "base": key[1]}, self.device)
        return self._rot[key]

    # caches ---------------------------------------------------------------------------------------------------
    def page_bytes(self) -> int:
        """Bytes of one 16-token page over every layer (layers that share tensors still cache for themselves)."""
        es = torch.empty(0, dtype=self.dtype).element_size()
        n = 0
        for L in self.cfg.layers:
            m = L["mixer"]
            if L["type"] == "parallel":
                n += int(m["left"]["kv_heads"]) * (int(m["left"]["dim"]) + int(m["left"]["vdim"]))
            elif L["type"] == "latent_attention":
                # (the latent is kept twice where the matrix-core kernel runs: row-major and page-wise transposed)
                n += 2 * int(m["kv_rank"]) + int(m["rot_dim"])
        return PAGE * n * es or 1

    def alloc_cache(self, num_blocks: int, num_slots: int):
        """(per layer: the latent pool [blocks, 16, kv_rank + rot_dim], or (keys [blocks, 16, G dim], values
        [blocks, G vdim, 16]), or None; per-layer slot state: the minGRU vector [slots, width], the HGRN2 matrices
        [slots, heads, dim, vdim], fp32). Zeroed once: a masked key's row is never used, but fresh memory must not
        hold NaN patterns for the debug checks."""
        dev, dt = self.device, self.dtype
        pages, state = [], LayerState()
        self.pages_t = []  # page-wise transposed latent copies [blocks, kv_rank, 16] for the matrix-core kernel
        for lw in self.layers:
            m, st, pt = lw.m, {}, None
            if lw.type == "parallel":
                G, D, Dv = (int(m["left"][k]) for k in ("kv_heads", "dim", "vdim"))
                pages.append((torch.zeros(num_blocks, PAGE, G * D, dtype=dt, device=dev),
                              torch.zeros(num_blocks, G * Dv, PAGE, dtype=dt, device=dev)))
                Hr, Dr, Dvr = (int(m["right"][k]) for k in ("heads", "dim", "vdim"))
                st["S"] = torch.zeros(num_slots, Hr, Dr, Dvr, dtype=torch.float32, device=dev)
            elif lw.type == "latent_attention":
                R, rd = int(m["kv_rank"]), int(m["rot_dim"])
                pages.append(torch.zeros(num_blocks, PAGE, R + rd, dtype=dt, device=dev))
                if hops.latent_mfma_ok(pages[-1], R, rd):
                    pt = torch.zeros(num_blocks, R, PAGE, dtype=dt, device=dev)
            else:
                pages.append(None)
                st["rnn"] = torch.zeros(num_slots, int(m["width"]), dtype=torch.float32, device=dev)
            self.pages_t.append(pt)
            state.layers.append(st)
        return pages, state

    # one step ---------------------------------------------------------------------------------------------------
    def forward(self, inp, pages: list, state: LayerState, gather: bool = True,
                layers_out: list | None = None) -> torch.Tensor:
        """Logits fp32 [n, V] for ``inp.logit_rows``. ``layers_out``: a list that receives the sum of the streams
        after every layer (fp32 [T, d] copies; debugging and the per-layer tests)."""
        cfg, dt, dev = self.cfg, self.dtype, self.device
        m: SegMeta = inp.attn
        T, d, eps, S = inp.tokens.shape[0], cfg.hidden_size, cfg.norm_eps, self.S
        xs = torch.empty(S, T, d, dtype=torch.float32, device=dev)      # fp32 streams
        e = F.embedding(inp.tokens, self.embed).unsqueeze(0)
        hops.stream_step(e, read=self.one, norm_w=self.embed_norm, eps=eps, out=xs[0], center=True)
        if S > 1:
            xs[1:] = xs[0]
        h = torch.empty(T, d, dtype=dt, device=dev)
        if self.layers:
            lw = self.layers[0]
            hops.stream_step(xs, read=lw.hc1.a, norm_w=lw.norm1, eps=eps, out=h, center=True)
        for i, lw in enumerate(self.layers):
            st = state.layers[i]
            if lw.type == "mingru":
                y = self._mingru(lw, h, m, st)
            elif lw.type == "parallel":
                y = self._parallel(i, lw, h, inp, m, pages, st)
            else:
                y = self._latent_attention(i, lw, h, inp, m, pages)
            nxt = self.layers[i + 1] if i + 1 < len(self.layers) else None
            total = torch.empty(T, d, dtype=torch.float32, device=dev) if layers_out is not None else None
            last = lw.hc1
            if lw.ff:
                # the mixer's write, the feed-forward's read and its norm in one pass over the streams
                hops.stream_step(xs, y, lw.hc1.M, lw.hc1.b, lw.hc2.a, lw.norm2, eps, h, center=True)
                a = torch.empty(T, lw.ff, dtype=dt, device=dev)
                hops.swish_clamp_mul(self._lin(h, lw.gate_up, getattr(lw, "gate_up_t", None), lw.gate_up_b), lw.limit,
                                     SWISH_ALPHA, a)
                y = self._lin(a, lw.down, getattr(lw, "down_t", None), lw.down_b)
                last = lw.hc2
            if nxt is not None:
                hops.stream_step(xs, y, last.M, last.b, nxt.hc1.a, nxt.norm1, eps, h, total=total, center=True)
            else:
                hops.stream_step(xs, y, last.M, last.b, total=total)
            if layers_out is not None:
                layers_out.append(total)
        xsel = xs.index_select(1, inp.logit_rows)
        hf = torch.empty(xsel.shape[1], d, dtype=dt, device=dev)
        hops.stream_step(xsel, read=self.sum_in, norm_w=self.final_norm, eps=eps, out=hf, center=True)
        logits = self._lin(hf, self.head, getattr(self, "head_t", None)).float()
        if cfg.logit_scale != 1.0:
            logits.mul_(cfg.logit_scale)
        return logits[:, :cfg.vocab_size]   # (a view: the padded row stride is what the sampler reads)

    def _max_rows(self, m: SegMeta) -> int:
        return int(m.seg_host[:, 1].max()) if m.seg_host is not None and len(m.seg_host) else 0

    def _chunk_plan(self, m: SegMeta, work: int):
        """Device chunk tables of this step for a scan with ``work`` workgroups per segment (built once per step), None
        = the plain scan fills the GPU or the segments are short."""
        key = ("chunks", work)
        if key not in m.cache:
            p = hops.scan_chunks(m.seg_host, work)
            if p is not None:
                fresh, cont, cs, mx = p
                up = torch.from_numpy(np.concatenate([fresh.reshape(-1), cont.reshape(-1),
                                                      cs.reshape(-1)])).to(self.device)
                a, b = fresh.size, fresh.size + cont.size
                p = (up[:a].view(-1, 4), up[a:b].view(-1, 4), up[b:].view(-1, 4), mx)
            m.cache[key] = p
        return m.cache[key]

    def _mingru(self, lw, h, m: SegMeta, st: dict) -> torch.Tensor:
        Wd = int(lw.m["width"])
        proj = self._lin(h, lw.w_in, getattr(lw, "w_in_t", None))                 # [update gate | candidate | gate]
        out = torch.empty(h.shape[0], Wd, dtype=self.dtype, device=self.device)
        hops.mingru_scan(proj, lw.b_in, Wd, m.tok_seg, m.seg, st["rnn"], out, self._max_rows(m))
        return self._lin(out, lw.o, getattr(lw, "o_t", None))

    def _parallel(self, i: int, lw, h, inp, m: SegMeta, pages: list, st: dict) -> torch.Tensor:
        a, b = lw.m["left"], lw.m["right"]
        H, G, D, Dv = (int(a[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
        Hr, Dr, Dvr = (int(b[k]) for k in ("heads", "dim", "vdim"))
        T, dt, dev = h.shape[0], self.dtype, self.device
        # [q | k | v | output gate || raw q | raw forget gate | v of the recurrence]
        proj = self._lin(h, lw.w_in, getattr(lw, "w_in_t", None))
        k_cache, v_cache_t = pages[i]
        q = torch.empty(T, H * G * D, dtype=dt, device=dev)                       # head-mixed queries
        hops.rope_kv_store(proj, H, G, D, Dv, inp.positions, lw.cos_sin, lw.rot_dims, False, lw.talk, k_cache,
                           v_cache_t, inp.slot_mapping, q)
        ao = torch.empty(T, H * Dv, dtype=dt, device=dev)
        hops.window_attn(q, k_cache, v_cache_t, m.block_tables, m.tok_seg, inp.positions, H, G, lw.scale, 0, None, ao,
                         m.tiles.get(hops.sig_tile_tokens(H, G)), m.max_keys, shared_keys=True)
        both = torch.empty(T, H * Dv + Hr * Dvr, dtype=dt, device=dev)            # [left heads | right heads]
        hops.gate_mul(ao, proj, lw.g_off, lw.left_scale, both[:, :H * Dv])
        o = torch.empty(T, Hr * Dvr, dtype=torch.float32, device=dev)
        plan = self._chunk_plan(m, Hr * -(-Dvr // 64)) if dev.type == "cuda" else None
        if plan is not None:  # long prompt portions, few sequences: chunk-parallel scan
            hops.hgrn2_scan_chunked(proj, lw.rq_off, lw.rf_off, lw.rv_off, lw.f_bias, lw.lower, Hr, Dr, Dvr, plan,
                                    st["S"], o)
        else:
            hops.hgrn2_scan(proj, lw.rq_off, lw.rf_off, lw.rv_off, lw.f_bias, lw.lower, Hr, Dr, Dvr, m.tok_seg, m.seg,
                            st["S"], o)
        hops.head_norm_gate(o, lw.rnorm, None, 0, Hr, self.cfg.norm_eps, both[:, H * Dv:], lw.right_scale)
        return self._lin(both, lw.o, getattr(lw, "o_t", None))

    def _latent_attention(self, i: int, lw, h, inp, m: SegMeta, pages: list) -> torch.Tensor:
        mm = lw.m
        H, D, rd, Dv, R, Rq = (int(mm[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank", "q_rank"))
        T, dt, dev = h.shape[0], self.dtype, self.device
        first = self._lin(h, lw.w_in, getattr(lw, "w_in_t", None))                # [query latent | latent | rotated key]
        cq = torch.empty(T, Rq, dtype=dt, device=dev)
        hops.act_norm(first, 0, Rq, lw.dq_norm, self.cfg.norm_eps, cq)
        q = self._lin(cq, lw.uq, getattr(lw, "uq_t", None))                       # heads of [dim | rot_dim]
        cache, cache_t = pages[i], self.pages_t[i]
        q_rot = torch.empty(T, H, rd, dtype=dt, device=dev)
        hops.latent_prep(q, H, D, rd, R, -1, None, self.cfg.norm_eps, inp.positions, lw.cos_sin, lw.rot_dims, cache,
                         inp.slot_mapping, q_rot)
        hops.latent_prep(first, 0, D, rd, R, Rq, lw.dkv_norm, self.cfg.norm_eps, inp.positions, lw.cos_sin,
                         lw.rot_dims, cache, inp.slot_mapping, q_rot[:, :0], cache_t)
        q_u = q.view(T, H, D + rd)[:, :, :D].transpose(0, 1)                      # [H, T, dim] (strided view)
        q_lat = torch.bmm(q_u, lw.uk_h)                                           # [H, T, R]
        o_lat = torch.empty(H, T, R, dtype=dt, device=dev)
        hops.latent_attn(q_lat, q_rot, cache, m.block_tables, m.tok_seg, m.seg, inp.positions, lw.scale, o_lat,
                         cache_t, m.tiles.get(hops.tile_tokens(H)), m.max_keys)
        ao = torch.empty(T, H * Dv, dtype=dt, device=dev)
        torch.bmm(o_lat, lw.uv_ht, out=ao.view(T, H, Dv).transpose(0, 1))         # head h -> its vdim columns
        return self._lin(ao, lw.o, getattr(lw, "o_t", None))


def load_checkpoint(model: MagedraLM, path: str | Path) -> MagedraLM:
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


def save_checkpoint(cfg: MagedraConfig, W: dict[str, torch.Tensor], folder: str | Path) -> None:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    save_file({k: v.contiguous() for k, v in W.items()}, str(folder / "model.safetensors"))
    (folder / "config.json").write_text(json.dumps(cfg.to_dict(), indent=1))
