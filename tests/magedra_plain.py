"""Plain, slow Magedra forward for the tests: one function per mechanism, whole sequences only, no cache, nothing
carried between calls, float64 by default. It shares nothing with the package: the engine's chunked, paged and batched
results are compared with what these functions give for the whole token list at once.

``cfg`` is the model's config.json as a dict, ``W`` maps tensor names to torch tensors.
"""
from __future__ import annotations

import math

import torch


def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w, the variance around the mean, no bias."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def angles(T, dims, base):
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    return torch.arange(T, dtype=torch.float64)[:, None] * f[None]


def rotate_halves(x, dims, base):
    """x [T, heads, D]: dimension i turns with dimension i + dims / 2 (i < dims / 2) by position * base^(-2i/dims)."""
    half = dims // 2
    ang = angles(x.shape[0], dims, base)
    c, s = torch.cos(ang).to(x.dtype)[:, None], torch.sin(ang).to(x.dtype)[:, None]
    a, b = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = a * c - b * s
    out[..., half:dims] = b * c + a * s
    return out


def rotate_pairs(x, dims, base):
    """x [T, heads, D]: dimension 2i turns with dimension 2i + 1 (i < dims / 2) by position * base^(-2i/dims)."""
    ang = angles(x.shape[0], dims, base)
    c, s = torch.cos(ang).to(x.dtype)[:, None], torch.sin(ang).to(x.dtype)[:, None]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def causal_softmax(s):
    """s [H, T, T] -> softmax over the keys j <= i of every row i."""
    T = s.shape[-1]
    ok = torch.ones(T, T, dtype=torch.bool).tril()
    return torch.softmax(s.masked_fill(~ok, float("-inf")), -1)


def mingru(h, W, p):
    """Gated recurrence whose gates read only the current token; the state starts at zero."""
    z = torch.sigmoid(h @ W[p + "z"].T + W[p + "z.b"])
    u = h @ W[p + "x"].T + W[p + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros_like(z[0])
    rows = []
    for t in range(h.shape[0]):
        S = (1.0 - z[t]) * S + z[t] * cand[t]
        rows.append(S)
    g = h @ W[p + "g"].T
    return (torch.stack(rows) * g * torch.sigmoid(g)) @ W[p + "o"].T


def talking_attention(h, W, p, m):
    """Grouped-query softmax attention whose scaled scores are mixed over the heads before the softmax; rotate-half
    positions on the first rot.dims dimensions; sigmoid output gate."""
    T = h.shape[0]
    H, G, D, Dv = (int(m[k]) for k in ("heads", "kv_heads", "dim", "vdim"))
    q = (h @ W[p + "q"].T).view(T, H, D)
    k = (h @ W[p + "k"].T).view(T, G, D)
    v = (h @ W[p + "v"].T).view(T, G, Dv)
    rot = m.get("rot")
    if rot:
        q = rotate_halves(q, int(rot["dims"]), rot["base"])
        k = rotate_halves(k, int(rot["dims"]), rot["base"])
    rep = H // G
    kh = k.repeat_interleave(rep, 1)
    vh = v.repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q, kh) * float(m["scale"])
    s = torch.einsum("hg,gij->hij", W[p + "talk"], s)
    o = torch.einsum("hij,jhv->ihv", causal_softmax(s), vh).reshape(T, H * Dv)
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def hgrn2(h, W, p, m, eps):
    """Linear attention whose forget gate (with a lower bound) also decides what is written: per head
    S <- diag(f) S + (1 - f) v^T, read-out S^T q, RMS norm per head."""
    T = h.shape[0]
    H, D, Dv = (int(m[k]) for k in ("heads", "dim", "vdim"))
    q = h @ W[p + "q"].T
    q = (q * torch.sigmoid(q)).view(T, H, D)
    v = (h @ W[p + "v"].T).view(T, H, Dv)
    low = W[p + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).view(T, H, D)
    S = torch.zeros(H, D, Dv, dtype=h.dtype)
    rows = []
    for t in range(T):
        S = f[t][:, :, None] * S + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
        rows.append(torch.einsum("hdv,hd->hv", S, q[t]))
    o = rms_norm(torch.stack(rows), W[p + "norm"], eps).reshape(T, H * Dv)
    return o @ W[p + "o"].T


def parallel(h, W, p, m, eps):
    left = talking_attention(h, W, p + "left.", m["left"])
    right = hgrn2(h, W, p + "right.", m["right"], eps)
    return float(m["left_scale"]) * left + float(m["right_scale"]) * right


def latent_attention(h, W, p, m, eps):
    """Queries through a normed latent; keys and values are per-head projections of one normed latent row per token,
    plus one rotated key part (pairs of neighbours) shared by all heads."""
    T = h.shape[0]
    H, D, rd, Dv, R = (int(m[k]) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank"))
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps)
    q = (cq @ W[p + "uq"].T).view(T, H, D + rd)
    ckv = h @ W[p + "dkv"].T
    c = rms_norm(ckv[:, :R], W[p + "dkv.norm"], eps)
    dims, base = int(m["rot"]["dims"]), m["rot"]["base"]
    kr = rotate_pairs(ckv[:, None, R:], dims, base)[:, 0]
    qr = rotate_pairs(q[..., D:], dims, base)
    k = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, Dv)
    s = (torch.einsum("ihd,jhd->hij", q[..., :D], k) + torch.einsum("ihd,jd->hij", qr, kr)) * float(m["scale"])
    o = torch.einsum("hij,jhv->ihv", causal_softmax(s), v).reshape(T, H * Dv)
    return o @ W[p + "o"].T


def dense_ff(h, W, p, mlp):
    lim = float(mlp["limit"])
    g = (h @ W[p + "gate"].T + W[p + "gate.b"]).clamp(max=lim)
    u = (h @ W[p + "up"].T + W[p + "up.b"]).clamp(min=-lim, max=lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T + W[p + "down.b"]


def mixer(h, W, p, L, eps):
    kind, m = L["type"], L["mixer"]
    if kind == "mingru":
        return mingru(h, W, p)
    if kind == "parallel":
        return parallel(h, W, p, m, eps)
    if kind == "latent_attention":
        return latent_attention(h, W, p, m, eps)
    raise ValueError(kind)


def forward(cfg: dict, W: dict, tokens, dtype=torch.float64, layers_out: list | None = None):
    """Logits [T, vocab] of one whole sequence. ``layers_out`` receives the residual (the sum of the streams) after
    every layer."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    S = int(cfg.get("streams") or 0)
    x0 = layer_norm(W["embed"][torch.as_tensor(tokens, dtype=torch.long)], W["embed.norm"], eps)
    xs = [x0.clone() for _ in range(max(S, 1))]
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % int(L.get("weights_of", i))
        subs = [(1, lambda h: mixer(h, W, p + "mix.", L, eps))]
        if L.get("mlp"):
            subs.append((2, lambda h: dense_ff(h, W, p + "mlp.", L["mlp"])))
        for q, fn in subs:
            nw = W[p + "norm%d" % q]
            if S:
                a, b, M = W[p + "hc%d.in" % q], W[p + "hc%d.out" % q], W[p + "hc%d.mix" % q]
                u = sum(a[s] * xs[s] for s in range(S))
                y = fn(layer_norm(u, nw, eps))
                xs = [sum(M[s, t] * xs[s] for s in range(S)) + mult * b[t] * y for t in range(S)]
            else:
                xs = [xs[0] + mult * fn(layer_norm(xs[0], nw, eps))]
        if layers_out is not None:
            layers_out.append(sum(xs))
    x = layer_norm(sum(xs), W["final.norm"], eps)
    return (x @ W["head"].T) * float(cfg.get("logit_scale", 1.0))
