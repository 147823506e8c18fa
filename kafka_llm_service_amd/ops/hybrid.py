"""Ops of the segment-planned decoder families (layer norm, token shift, latent attention, Mamba-2, depth average;
gated mixers and routed experts; residual streams, windowed attention with sinks, group-limited routing): GPU tensors
run the HIP kernels of ``csrc/hybrid.hip``, ``hybrid_gated.hip`` and ``hybrid_streams.hip``, CPU tensors the fp32
references of ``hybrid_reference.py``.

Activations are bf16 or fp32 (the model's dtype, the kernels are built for both); the residual stream, recurrent
state, norms, softmax and every gate of a recurrence are fp32 in both. A step's rows are described by ``seg`` int32
[R, 4] = (first row, rows, first position, state slot) and ``tok_seg`` int32 [T] (see hybrid_reference.py).
"""
from __future__ import annotations

import torch

from . import hybrid_reference as ref
from ._ext import ext

SCAN_MAX_TAPS = 16


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
    if rd == 0 and (rot_dims or cos_sin is not None):
        raise ValueError("latent_prep: a rotation needs a rotated part")
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
                tiles=None, max_keys: int = 0, window: int = 0, sink=None) -> None:
    """Causal softmax attention of every row's heads over its sequence's cached [latent | rotated key] rows:
    out[h, t] = sum_j softmax_j((q_lat[h, t] . c_j + q_rot[t, h] . k_j) scale) c_j over the keys j <= position[t].
    With the transposed latent copy ``cache_t`` and ``tiles`` (int32 [n, 4] = (first row, tokens, segment, 0), at
    most ``tile_tokens(H)`` tokens of one segment each) bf16 runs on the matrix cores; else one wave per (row, 4
    heads) on the vector units (fp32, odd sizes). ``max_keys`` (the step's longest context) lets a launch of few
    tiles split its key ranges over more workgroups (``attn_splits``).
    ``window`` > 0: a row at position p sees only the keys p - window < j <= p. ``sink`` fp32 [H]: a per-head logit
    (not scaled) that joins the softmax denominator without a key or a value."""
    if window < 0:
        raise ValueError("latent_attn: window must be positive (0 = every earlier position)")
    if _gpu(q_lat):
        if cache_t is not None and tiles is not None and q_lat.dtype == torch.bfloat16:
            H, T, R = q_lat.shape
            if window:  # a key range is at most the window long
                max_keys = min(max_keys, window + tile_tokens(H))
            ns = attn_splits(tiles.shape[0], H, max_keys) if max_keys else 1
            po = pml = None
            if ns > 1:
                po = torch.empty(ns, H, T, R, dtype=torch.float32, device=q_lat.device)
                pml = torch.empty(ns, H, T, 2, dtype=torch.float32, device=q_lat.device)
            ext().hy_latent_attn_mfma(q_lat, q_rot, cache, cache_t, block_tables, tiles, tile_tokens(H), positions,
                                      float(scale), out, ns, po, pml, int(window), sink)
        else:
            ext().hy_latent_attn(q_lat, q_rot, cache, block_tables, tok_seg, positions, float(scale), out, int(window),
                                 sink)
    else:
        ref.latent_attn(q_lat, q_rot, cache, block_tables, tok_seg, seg, positions, scale, out, window, sink)


def sigmoid_mul(a, g, out) -> None:
    if _gpu(a):
        ext().hy_sigmoid_mul(a, g, out)
    else:
        ref.sigmoid_mul(a, g, out)


def conv_silu(proj, c0: int, w, b, tok_seg, seg, state, out) -> None:
    """Causal per-channel convolution + silu over columns [c0, c0 + C) of ``proj``; ``state`` [slots, taps - 1, C]
    holds each sequence's last raw inputs and is advanced."""
    short_conv(proj, c0, w, b, tok_seg, seg, state, out, act="silu")


def short_conv(u, c0: int, w, b, tok_seg, seg, state, out, act: str = "none", residual: bool = False) -> None:
    """out_t = act(b + sum_k w[:, k] u_(t - taps + 1 + k)) (+ u_t with ``residual``) per channel of columns
    [c0, c0 + C) of ``u``, zeros before a sequence's start; ``b`` may be None, ``act`` is "none" or "silu".
    ``state`` [slots, taps - 1, C] holds each sequence's last inputs and is advanced (taps = 1: no state)."""
    if w.shape[1] > SCAN_MAX_TAPS:
        raise ValueError(f"short convolution of {w.shape[1]} taps (at most {SCAN_MAX_TAPS})")
    if act not in ("none", "silu"):
        raise ValueError(f"short convolution: unknown activation {act!r}")
    if _gpu(u):
        ext().hy_short_conv(u, int(c0), w, b, tok_seg, seg, state, out, act == "silu", bool(residual))
    else:
        ref.short_conv(u, c0, w, b, tok_seg, seg, state, out, act, residual)


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


# ---- gated mixers: sigmoid attention, real-gated linear recurrence, matrix memory, routed experts --------------------
def rms_norm(x, w, eps, out) -> None:
    """out = x / sqrt(mean(x^2) + eps) * w over rows of the fp32 stream."""
    if _gpu(x):
        ext().hy_rms_norm(x, w, float(eps), out)
    else:
        ref.rms_norm(x, w, eps, out)


def kv_store(src, k_off: int, v_off: int, k_cache, v_cache_t, slot_mapping) -> None:
    """Row t's key columns [k_off, k_off + Ck) -> k_cache [pages, page, Ck] at its slot, its value columns
    [v_off, v_off + Cv) -> v_cache_t [pages, Cv, page] (every page transposed: a channel's tokens are consecutive,
    the layout the value product of the attention kernels reads)."""
    if _gpu(src):
        ext().hy_kv_store(src, int(k_off), int(v_off), k_cache, v_cache_t, slot_mapping)
    else:
        ref.kv_store(src, k_off, v_off, k_cache, v_cache_t, slot_mapping)


SIG_TILE_ROWS = 32     # query rows ((token, head) pairs of one key/value head) of a matrix-core attention tile


def sig_tile_tokens(heads: int, kv_heads: int) -> int:
    """Tokens per tile of the matrix-core sigmoid attention: as many whole tokens (all query heads of one key/value
    head) as fit 32 rows, at least one."""
    return max(1, SIG_TILE_ROWS // max(1, heads // kv_heads))


def sigmoid_attn_mfma_ok(q, k_cache, v_cache_t, H: int, G: int) -> bool:
    """bf16 GPU tensors of sizes the matrix-core kernel takes (16-token pages, key size a multiple of 16, sizes up
    to 256, at most 32 query heads per key/value head, 16-byte aligned query rows)."""
    if not (q.is_cuda and q.dtype == torch.bfloat16):
        return False
    if q.stride(0) % 8 or q.data_ptr() % 16:  # query rows are read in 16-byte pieces
        return False
    return bool(ext().hy_sigmoid_attn_mfma_ok(k_cache.shape[1], k_cache.shape[2] // G, v_cache_t.shape[1] // G,
                                              H // G))


def sig_splits(wgs: int, max_keys: int, target: int = ATTN_SPLIT_WGS) -> int:
    """Key-range splits of a matrix-core sigmoid attention launch: few workgroups (a decode step has one tile per
    sequence and key/value head) against long contexts are dealt over more (up to ``target`` in all), each at least
    two 128-key blocks long; the partial sums are added in order by a second launch."""
    blocks = -(-max_keys // 128)
    if wgs >= target // 2 or blocks < 4:
        return 1
    return max(1, min(ATTN_SPLIT_MAX, target // max(1, wgs), blocks // 2))


def sigmoid_attn(q, q_off: int, k_cache, v_cache_t, block_tables, tok_seg, positions, H: int, G: int, scale: float,
                 softcap: float, t_coef: float, t_every: float, r1, r2, pb, out, tiles=None, max_keys: int = 0) -> None:
    """Causal attention with sigmoid weights (no softmax, no normalisation over keys). For row t at position p, head h
    (key/value head h // (H / G)) and every key j <= p:
        s = (q . k_j) scale (1 + t_coef ln(floor((p + 1) / t_every) + 1));  s = softcap tanh(s / softcap) if softcap;
        out = sum_j sigmoid(s - r1[h] ln(1 + r2[h] (p - j)) + pb[h]) v_j.
    q rows start at column ``q_off`` of ``q``; out [T, H Dv]. Scores, biases and weights are fp32. With ``tiles``
    (int32 [n, 4] = (first row, tokens, segment, 0), at most ``sig_tile_tokens`` tokens of one segment each) and
    sizes it takes, bf16 runs on the matrix cores; else one wave per (row, head) on the vector units. ``max_keys``
    (the step's longest context) lets a launch of few tiles split its key ranges over more workgroups."""
    if _gpu(q):
        if tiles is not None and q_off % 8 == 0 and sigmoid_attn_mfma_ok(q, k_cache, v_cache_t, H, G):
            ns = sig_splits(tiles.shape[0] * G, max_keys) if max_keys else 1
            po = None
            if ns > 1:
                po = torch.empty(ns, q.shape[0], out.shape[1], dtype=torch.float32, device=q.device)
            ext().hy_sigmoid_attn_mfma(q, int(q_off), k_cache, v_cache_t, block_tables, tiles,
                                       sig_tile_tokens(H, G), positions, int(H), int(G), float(scale), float(softcap),
                                       float(t_coef), float(t_every), r1, r2, pb, out, ns, po)
        else:
            ext().hy_sigmoid_attn(q, int(q_off), k_cache, v_cache_t, block_tables, tok_seg, positions, int(H), int(G),
                                  float(scale), float(softcap), float(t_coef), float(t_every), r1, r2, pb, out)
    else:
        ref.sigmoid_attn(q, q_off, k_cache, v_cache_t, block_tables, tok_seg, positions, H, G, scale, softcap, t_coef,
                         t_every, r1, r2, pb, out)


def rglru_scan(gates, proj, u, rate, tok_seg, seg, state, out, max_rows: int = 0) -> None:
    """The real-gated linear recurrent unit over a step's segments. gates fp32 [T, 2 W] = pre-activations of the
    recurrence gate | the input gate (biases included), proj [T, >= W] whose first W columns are the raw gelu branch,
    u [T, W] the convolved branch, rate fp32 [W] (= -c softplus(lambda)):
        a = exp(rate sigmoid(g_r)),  S <- a S + sqrt(1 - a^2) sigmoid(g_i) u,  out = S gelu_tanh(branch).
    state fp32 [slots, W], zero before a sequence's first token (the slot is then written, not read). ``max_rows``:
    an upper bound of the longest segment's rows, when the caller knows one: steps with segments of more than 64 rows
    run in chunks (everything but the multiply-adds in parallel over rows, the chunks' entry states carried in
    order; ``gates`` is then overwritten), which re-associates the sums - fp32 rounding only."""
    if _gpu(u):
        ext().hy_rglru_scan(gates, proj, u, rate, seg, state, out, int(max_rows))
    else:
        ref.rglru_scan(gates, proj, u, rate, tok_seg, seg, state, out)


def mlstm_scan(qkv, gates, H: int, D: int, Dv: int, cap: float, tok_seg, seg, S, nrm, mx, out) -> None:
    """The matrix-memory recurrence (mLSTM) over a step's segments. qkv [T, >= H (2 D + Dv)] = q | k | v heads,
    gates fp32 [T, 2 H] = raw input | forget gate (biases included). Per head, with i = cap tanh(g_i / cap),
    f = logsigmoid(cap tanh(g_f / cap)), q' = q D^(-1/2):
        m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n <- e^(f + m - m') n + e^(i - m') k;
        out = S^T q' / (max(|n . q'|, e^(-m')) + 1e-6).
    State per slot, all fp32 and all zero (m too) before a sequence's first token: S [slots, H, D, Dv],
    nrm [slots, H, D], mx [slots, H]. out fp32 [T, H Dv]."""
    if _gpu(qkv):
        ext().hy_mlstm_scan(qkv, gates, int(H), int(D), int(Dv), float(cap), seg, S, nrm, mx, out)
    else:
        ref.mlstm_scan(qkv, gates, H, D, Dv, cap, tok_seg, seg, S, nrm, mx, out)


def head_norm_gate(o, w, g, g_off: int, H: int, eps, out, scale: float = 1.0) -> None:
    """out = o / rms_per_head(o) * w * sigmoid(g[:, g_off : g_off + H Dv]) * scale for o fp32 [T, H Dv]; ``g`` None:
    no gate. ``out`` may be a column slice of a wider buffer."""
    if _gpu(o):
        ext().hy_head_norm_gate(o, w, g, int(g_off), int(H), float(eps), out, float(scale))
    else:
        ref.head_norm_gate(o, w, g, g_off, H, eps, out, scale)


def moe_router(h, w, b, k: int):
    """Router of a routed feed-forward: fp32 logits h W^T + b (W, b fp32), the k largest per row (ties: the lower
    index) and a softmax over those k. Returns (weights fp32 [T, k], experts int32 [T, k])."""
    T = h.shape[0]
    tw = torch.empty(T, k, dtype=torch.float32, device=h.device)
    te = torch.empty(T, k, dtype=torch.int32, device=h.device)
    if k > w.shape[0]:
        raise ValueError("router: more experts per token than experts")
    if _gpu(h):
        # logits as one fp32 matrix product (full-precision fp32: PyTorch's default for fp32 operands, and the engine
        # switches reduced-precision matrix modes off explicitly for fp32 models), then the top-k kernel
        ext().hy_moe_topk(torch.addmm(b, h.float(), w.t()), tw, te)
    else:
        ref.moe_router(h, w, b, k, tw, te)
    return tw, te


GLU_ACTS = ("silu", "swish_clamp")


def _glu_act(act: str, limit: float, alpha: float) -> tuple[float, float]:
    """(limit, alpha) as the kernels take them: limit 0 selects silu(g) * u."""
    if act not in GLU_ACTS:
        raise ValueError(f"unknown gated activation {act!r}")
    if act == "silu":
        return 0.0, 1.0
    if not limit > 0:
        raise ValueError("swish_clamp needs a positive limit")
    return float(limit), float(alpha)


def moe_rows(h, w_gu, w_down, topk_w, topk_e, out, act: str = "silu", limit: float = 0.0, alpha: float = 1.0) -> None:
    """Routed experts evaluated per (row, chosen expert) pair, any sizes and both dtypes:
    out[t] = sum_j topk_w[t, j] W_down[e_tj] act(W_gate[e_tj] h_t, W_up[e_tj] h_t) with w_gu [E, 2 F, d] = gate
    rows then up rows and w_down [E, d, F]; the pairs of a row are summed in order j = 0, 1, ... (fp32).
    ``act``: "silu" = silu(g) * u, or "swish_clamp" (see ``swish_clamp_mul``)."""
    lim, al = _glu_act(act, limit, alpha)
    if _gpu(h):
        T, k = topk_e.shape
        a = torch.empty(T * k, w_down.shape[2], dtype=h.dtype, device=h.device)
        ext().hy_moe_rows(h, w_gu, w_down, topk_w, topk_e, a, out, lim, al)
    else:
        ref.moe_rows(h, w_gu, w_down, topk_w, topk_e, out, lim, al)


MOE_STREAM_MAX_T = 640  # steps of up to this many rows run tiled expert weights on the grouped streaming kernel


def moe_grouped_ok(h, w_gu, w_down) -> bool:
    """bf16 GPU tensors of sizes the expert-sorted matrix-core kernels take (ops.grouped_gemm)."""
    E, F2, d = w_gu.shape
    return bool(h.is_cuda and h.dtype == torch.bfloat16 and F2 % 128 == 0 and d % 128 == 0 and (F2 // 2) % 64 == 0 and
                h.stride(0) % 8 == 0)


def moe_experts(h, w_gu, w_down, topk_w, topk_e, out, w_gu_t=None, w_down_t=None, act: str = "silu",
                limit: float = 0.0, alpha: float = 1.0) -> None:
    """out (fp32 [T, d]) = the routed experts' weighted sum for every row. Sizes the framework's expert-sorted
    matrix-core kernels take (bf16) go through them - entries sorted by expert (``ops.moe_sort``), gate/up GEMM on
    gathered rows, silu * up, down GEMM with the weighted combine in its epilogue (fp32 adds, two entries per row
    commute), or the grouped weight-streaming kernels when tiled expert weights are given and the step is small -
    everything else is evaluated per (row, expert) pair by ``moe_rows``. ``act`` as in ``moe_rows`` (the streaming
    kernel applies it in its epilogue; between the two expert-sorted GEMMs it is a launch of its own)."""
    from kafka_llm_service_amd import ops

    T = h.shape[0]
    if T and moe_grouped_ok(h, w_gu, w_down):
        r = ops.moe_sort(topk_w, topk_e, w_gu.shape[0])
        out.zero_()
        if w_gu_t is not None and w_down_t is not None and T <= MOE_STREAM_MAX_T:
            lim, al = _glu_act(act, limit, alpha)
            a = ops.grouped_stream_glu(h, w_gu_t, r, limit=lim, alpha=al)
            ops.grouped_stream_combine(a, w_down_t, r, T, out)
        else:
            gu = ops.grouped_gemm(h, w_gu, r, gather=True)
            if act == "silu":
                a = ops.silu_mul(gu)
            else:
                a = torch.empty(gu.shape[0], gu.shape[1] // 2, dtype=gu.dtype, device=gu.device)
                swish_clamp_mul(gu, limit, alpha, a)
            ops.grouped_gemm(a, w_down, r, gather=False, combine_out=out)
    else:
        moe_rows(h, w_gu, w_down, topk_w, topk_e, out, act, limit, alpha)


def add2(x, y1, y2=None, norm_w=None, eps=0.0, out=None) -> None:
    """x += y1 (+ y2) on the fp32 stream, the sublayer outputs summed in fp32 first; with ``norm_w`` also
    out = rms_norm(new x) * norm_w in the same pass over the row (the next layer's norm)."""
    if _gpu(x):
        ext().hy_add2(x, y1, y2, norm_w, float(eps), out)
    else:
        ref.add2(x, y1, y2)
        if norm_w is not None:
            ref.rms_norm(x, norm_w, eps, out)


# ---- hyper-connected residual streams, windowed softmax attention with sinks, group-limited routing -----------------
STREAM_MAX = 16   # residual streams the stream kernel takes


def stream_step(xs, y=None, mix=None, write=None, read=None, norm_w=None, eps=0.0, out=None, y2=None,
                row_scale=None, total=None, center: bool = False) -> None:
    """One pass over the residual streams xs fp32 [S, T, d] (hyper-connections), every part optional:
      write   with ``mix`` fp32 [S, S] (indexed [from, to]) and ``write`` fp32 [S]: all streams at once from the old
              ones, xs[r] <- sum_s mix[s, r] xs[s] + write[r] * (y + row_scale[:, None] * y2); y / y2 [T, d] in the
              activation dtype or fp32, row_scale fp32 [T] (y2 and row_scale come together or not at all);
      read    with ``read`` fp32 [S] and ``norm_w`` fp32 [d] (a one-plus weight is passed as 1 + w): out = u /
              sqrt(mean(u^2) + eps) * norm_w for u = sum_s read[s] xs[s] of the NEW streams, in out's dtype; with
              ``center`` the row's mean is taken off u first (a layer norm with a weight and no bias);
      total   fp32 [T, d] <- sum_s xs[s] of the new streams.
    All arithmetic is fp32. A plain residual is S = 1 with mix = write = read = 1."""
    S = xs.shape[0]
    if S > STREAM_MAX:
        raise ValueError(f"stream_step: at most {STREAM_MAX} streams")
    if (mix is None) != (write is None) or (mix is not None and y is None):
        raise ValueError("stream_step: a write needs mix, write and y")
    if (y2 is None) != (row_scale is None) or (y2 is not None and mix is None):
        raise ValueError("stream_step: y2 and row_scale come together, with a write")
    if (read is None) != (norm_w is None) or (read is None) != (out is None):
        raise ValueError("stream_step: a read needs read, norm_w and out")
    if _gpu(xs):
        ext().hy_stream_step(xs, y, mix, write, read, norm_w, float(eps), out, y2, row_scale, total, bool(center))
    else:
        ref.stream_step(xs, y, mix, write, read, norm_w, eps, out, y2, row_scale, total, center)


def swish_clamp_mul(gu, limit: float, alpha: float, out) -> None:
    """out = g' sigmoid(alpha g') (u' + 1) with g' = min(gu[:, :F], limit), u' = clamp(gu[:, F:], -limit, limit)."""
    if not limit > 0:
        raise ValueError("swish_clamp_mul needs a positive limit")
    if _gpu(gu):
        ext().hy_swish_clamp_mul(gu, float(limit), float(alpha), out)
    else:
        ref.swish_clamp_mul(gu, limit, alpha, out)


def qk_norm_rope_store(qkv, H: int, G: int, D: int, Dv: int, q_w, k_w, eps, positions, cos_sin, rot_dims: int,
                       v_first, v_first_off: int, lam: float, k_cache, v_cache_t, slot_mapping, q_out) -> None:
    """Attention inputs from the fused projection row [q (H D) | k (G D) | v (G Dv)]:
      * RMS norm over the WHOLE q part and over the whole k part (weights fp32 [H D], [G D]), before the head split;
      * rotation of the dimension pairs (2i, 2i + 1), i < rot_dims / 2, of every q and k head by the row's position
        (``cos_sin`` fp32 [positions, rot_dims] = cos | sin per frequency; rot_dims = 0 and no table: no rotation);
      * values: with ``v_first`` (rows [T, ...] whose value columns start at ``v_first_off``) v <- (1 - lam) v + lam
        v_first;
      * q -> q_out [T, H D]; k -> k_cache [pages, page, G D] at the row's slot; v -> v_cache_t [pages, G Dv, page].
    Norms, rotation and the mix are fp32."""
    if rot_dims % 2 or rot_dims > D or (rot_dims > 0) != (cos_sin is not None):
        raise ValueError("qk_norm_rope_store: rot_dims even, at most the head size, with its table")
    if _gpu(qkv):
        ext().hy_qk_norm_rope_store(qkv, int(H), int(G), int(D), int(Dv), q_w, k_w, float(eps), positions, cos_sin,
                                    int(rot_dims), v_first, int(v_first_off), float(lam), k_cache, v_cache_t,
                                    slot_mapping, q_out)
    else:
        ref.qk_norm_rope_store(qkv, H, G, D, Dv, q_w, k_w, eps, positions, cos_sin, rot_dims, v_first, v_first_off,
                               lam, k_cache, v_cache_t, slot_mapping, q_out)


SHARED_SPLIT_WGS = 1024   # workgroups a shared-keys attention launch is split towards


def window_attn_mfma_ok(q, k_cache, v_cache_t, H: int, G: int, shared_keys: bool = False) -> bool:
    """bf16 GPU tensors of sizes the matrix-core kernel takes (16-token pages, key size a multiple of 16, sizes up
    to 256, at most 32 query heads per key/value head, 16-byte aligned query rows). With ``shared_keys`` the key size
    is the whole key row's."""
    if not (q.is_cuda and q.dtype == torch.bfloat16):
        return False
    if q.stride(0) % 8 or q.data_ptr() % 16:  # query rows are read in 16-byte pieces
        return False
    return bool(ext().hy_window_attn_mfma_ok(k_cache.shape[1], k_cache.shape[2] // (1 if shared_keys else G),
                                             v_cache_t.shape[1] // G, H // G))


def window_attn(q, k_cache, v_cache_t, block_tables, tok_seg, positions, H: int, G: int, scale: float, window: int,
                sink, out, tiles=None, max_keys: int = 0, shared_keys: bool = False) -> None:
    """Causal softmax attention over paged keys [pages, page, G D] and page-wise transposed values [pages, G Dv, page]:
    row t at position p, head h (key/value head h // (H / G)) sees the keys p - window < j <= p (window 0: all j <= p);
        out = sum_j e^(s_j) v_j / (sum_j e^(s_j) + e^(sink[h])),  s_j = (q . k_j) scale
    with ``sink`` fp32 [H] (None: no such term). q [T, H D], out [T, H Dv]; scores and weights fp32. With ``tiles``
    (int32 [n, 4] = (first row, tokens, segment, 0), at most ``sig_tile_tokens(H, G)`` tokens of one segment each) and
    sizes it takes, bf16 runs on the matrix cores; else one wave per (row, head) on the vector units, keys in order,
    whatever the batch. ``max_keys`` (the step's longest context) lets a launch of few tiles split its key ranges
    over more workgroups (``sig_splits``); a merge pass combines them.
    ``shared_keys``: q is [T, H G D] - every query head is a row of the whole key row's size and its score is the
    product with ALL G key heads of a token (queries that hold a mix over the heads, see ``rope_kv_store``); values
    stay per key/value head."""
    if window < 0:
        raise ValueError("window_attn: window must be positive (0 = every earlier position)")
    if _gpu(q):
        if tiles is not None and window_attn_mfma_ok(q, k_cache, v_cache_t, H, G, shared_keys):
            tt = sig_tile_tokens(H, G)
            if window and max_keys:  # a tile's key range is at most the window and its own tokens long
                max_keys = min(max_keys, window + tt)
            # (shared keys: few key/value heads, every workgroup walks the whole key row - more, shorter ranges)
            ns = sig_splits(tiles.shape[0] * G, max_keys, SHARED_SPLIT_WGS if shared_keys else ATTN_SPLIT_WGS) \
                if max_keys else 1
            po = pml = None
            if ns > 1:
                po = torch.empty(ns, q.shape[0], out.shape[1], dtype=torch.float32, device=q.device)
                pml = torch.empty(ns, q.shape[0], H, 2, dtype=torch.float32, device=q.device)
            ext().hy_window_attn_mfma(q, k_cache, v_cache_t, block_tables, tiles, tt, positions, int(H), int(G),
                                      float(scale), int(window), sink, out, ns, po, pml, bool(shared_keys))
        else:
            ext().hy_window_attn(q, k_cache, v_cache_t, block_tables, tok_seg, positions, int(H), int(G), float(scale),
                                 int(window), sink, out, bool(shared_keys))
    else:
        ref.window_attn(q, k_cache, v_cache_t, block_tables, tok_seg, positions, H, G, scale, window, sink, out,
                        shared_keys)


def moe_router_grouped(h, w, correction, k: int, groups: int, keep: int, eps: float = 0.0, extra_gate: bool = False):
    """Group-limited router: fp32 logits h W^T over the first E rows of ``w`` (fp32 [E (+ 1), d]); s = softmax over
    all E; the choice looks at s + correction, only within the ``keep`` groups (of ``groups`` equal groups of
    neighbouring experts) whose largest corrected score is largest, and takes the k largest there (ties: the lower
    index); the weights are s of the chosen divided by (their sum + eps). With ``extra_gate`` the last row of ``w`` is
    a gate vector and sigmoid of its product is returned per row. Returns (weights fp32 [T, k], experts int32
    [T, k], gate fp32 [T] or None)."""
    T = h.shape[0]
    E = w.shape[0] - (1 if extra_gate else 0)
    if E < 1 or groups < 1 or E % groups or not 1 <= keep <= groups or not 1 <= k <= keep * (E // groups):
        raise ValueError("router: experts, groups and choices do not fit")
    if correction.shape[0] != E:
        raise ValueError("router: one correction per expert")
    tw = torch.empty(T, k, dtype=torch.float32, device=h.device)
    te = torch.empty(T, k, dtype=torch.int32, device=h.device)
    gate = torch.empty(T, dtype=torch.float32, device=h.device) if extra_gate else None
    if _gpu(h):
        # logits as one full-precision fp32 matrix product (the engine switches reduced-precision matrix modes off),
        # then the choice kernel
        ext().hy_moe_topk_grouped(torch.mm(h.float(), w.t()), int(E), correction, int(groups), int(keep), float(eps),
                                  tw, te, gate)
    else:
        ref.moe_router_grouped(h, w, E, correction, k, groups, keep, eps, tw, te, gate)
    return tw, te, gate


# ---- gated recurrences beside attention (minGRU, HGRN2), rotation + head mix + paged store --------------------------
def act_norm(x, c0: int, n: int, w, eps, out, center: bool = False) -> None:
    """out [T, n] = norm(x[:, c0 : c0 + n]) * w over rows of activations (x in the activation dtype or fp32, w fp32
    [n]): an RMS norm, or with ``center`` a layer norm with a weight and no bias. Statistics in fp32."""
    if c0 < 0 or c0 + n > x.shape[1]:
        raise ValueError("act_norm: columns outside the row")
    if _gpu(x):
        ext().hy_act_norm(x, int(c0), int(n), w, float(eps), out, bool(center))
    else:
        ref.act_norm(x, c0, n, w, eps, out, center)


def gate_mul(a, g, g_off: int, scale: float, out) -> None:
    """out = a * sigmoid(g[:, g_off : g_off + n]) * scale for a [T, n]; ``out`` may be a column slice."""
    if _gpu(a):
        ext().hy_gate_mul(a, g, int(g_off), float(scale), out)
    else:
        ref.gate_mul(a, g, g_off, scale, out)


def mingru_scan(proj, bias, W: int, tok_seg, seg, state, out, max_rows: int = 0) -> None:
    """minGRU over a step's segments: a gated recurrence whose gates read only the current token. proj [T, >= 3 W] =
    pre-activations of the update gate | the candidate | the output gate, bias fp32 [2 W] for the first two:
        z = sigmoid(p_z + b_z);  u = p_x + b_x;  c = u + 1/2 where u >= 0, sigmoid(u) where u < 0;
        S <- (1 - z) S + z c;  out = S silu(p_g).
    state fp32 [slots, W], zero before a sequence's first token (the slot is then written, not read). Gates, the
    candidate and the state are fp32. ``max_rows``: an upper bound of the longest segment's rows when the caller
    knows one: long segments run in chunks (per-chunk scans from zero with the chunk's decay product, entry states
    carried in order, a second pass from the entry states), which re-associates the sums - fp32 rounding only."""
    if _gpu(proj):
        ext().hy_mingru_scan(proj, bias, int(W), seg, state, out, int(max_rows))
    else:
        ref.mingru_scan(proj, bias, W, tok_seg, seg, state, out)


def hgrn2_scan(proj, q_off: int, f_off: int, v_off: int, f_bias, lower, H: int, D: int, Dv: int, tok_seg, seg, S,
               out) -> None:
    """HGRN2 over a step's segments: linear attention whose forget gate is also (one minus) its key. proj [T, ...]
    holds the raw queries (H D columns at q_off), raw forget gates (H D at f_off) and values (H Dv at v_off);
    f_bias, lower fp32 [H D]. Per head:
        f = lower + (1 - lower) sigmoid(p_f + b_f);  S <- diag(f) S + (1 - f) v^T;  out = S^T silu(p_q).
    S fp32 [slots, H, D, Dv], zero before a sequence's first token; out fp32 [T, H Dv]."""
    if _gpu(proj):
        ext().hy_hgrn2_scan(proj, int(q_off), int(f_off), int(v_off), f_bias, lower, int(H), int(D), int(Dv), seg, S,
                            out)
    else:
        ref.hgrn2_scan(proj, q_off, f_off, v_off, f_bias, lower, H, D, Dv, tok_seg, seg, S, out)


def hgrn2_scan_chunked(proj, q_off: int, f_off: int, v_off: int, f_bias, lower, H: int, D: int, Dv: int, plan, S,
                       out) -> None:
    """The recurrence of ``hgrn2_scan`` in launches that expose more parallelism for long segments: every chunk
    scanned from a zero state (and the product of its forget gates taken), the chunks' entry states rebuilt in order
    (and the sequence's state advanced), every chunk scanned again from its entry state. ``plan``: device tensors
    (vseg_fresh, vseg_cont, cs) + max chunks from ``scan_chunks``. Twice the arithmetic of the plain scan over
    (chunks) times the workgroups; the result differs from the token-by-token order only by fp32 rounding (the entry
    states are re-associated)."""
    fresh, cont, cs, max_chunks = plan
    tmp = torch.empty(fresh.shape[0], H, D, Dv, dtype=torch.float32, device=proj.device)
    F = torch.empty(fresh.shape[0], H * D, dtype=torch.float32, device=proj.device)
    e = ext()
    e.hy_hgrn2_scan(proj, int(q_off), int(f_off), int(v_off), f_bias, lower, int(H), int(D), int(Dv), fresh, tmp, out)
    e.hy_hgrn2_chunk_decay(proj, int(f_off), f_bias, lower, fresh, F)
    e.hy_hgrn2_chunk_combine(cs, F, tmp, S)
    e.hy_hgrn2_scan(proj, int(q_off), int(f_off), int(v_off), f_bias, lower, int(H), int(D), int(Dv), cont, tmp, out)


def rope_kv_store(qkv, H: int, G: int, D: int, Dv: int, positions, cos_sin, rot_dims: int, pairs: bool, talk,
                  k_cache, v_cache_t, slot_mapping, q_out) -> None:
    """Attention inputs from the fused projection row [q (H D) | k (G D) | v (G Dv)] (further columns are ignored):
      * rotation of the first ``rot_dims`` dimensions of every q and k head by the row's position (``cos_sin`` fp32
        [positions, rot_dims] = cos | sin per frequency): dimension i with i + rot_dims / 2, or with ``pairs``
        dimension 2i with 2i + 1; rot_dims = 0 and no table: no rotation;
      * k -> k_cache [pages, page, G D] at the row's slot; v -> v_cache_t [pages, G Dv, page];
      * q -> q_out [T, H D]; or with ``talk`` fp32 [H, H] (scores mixed over the heads before the softmax,
        s'_h = sum_g talk[h, g] s_g) -> q_out [T, H G D]: q'[h] = for every key head c the sum over its query heads g
        of talk[h, g] q[g], so that q'[h] . (the whole key row) = s'_h (``window_attn`` with ``shared_keys``).
    Rotation and the mix are fp32."""
    if rot_dims % 2 or rot_dims > D or (rot_dims > 0) != (cos_sin is not None):
        raise ValueError("rope_kv_store: rot_dims even, at most the head size, with its table")
    if G < 1 or H % G:
        raise ValueError("rope_kv_store: query heads must split evenly over the key heads")
    if _gpu(qkv):
        ext().hy_rope_kv_store(qkv, int(H), int(G), int(D), int(Dv), positions, cos_sin, int(rot_dims), bool(pairs),
                               talk, k_cache, v_cache_t, slot_mapping, q_out)
    else:
        ref.rope_kv_store(qkv, H, G, D, Dv, positions, cos_sin, rot_dims, pairs, talk, k_cache, v_cache_t,
                          slot_mapping, q_out)
