"""Plain, slow Mozidra forward for the tests: one function per mechanism, whole sequences only, no cache, nothing
carried between calls, float64 by default. It shares nothing with the package: the engine's chunked, paged and batched
results are compared with what these functions give for the whole token list at once.

``cfg`` is the model's config.json as a dict, ``W`` maps tensor names to torch tensors.
"""
from __future__ import annotations

import math

import torch


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plus_one(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def visible(T, window):
    """[T, T] bool: row i sees column j when 0 <= i - j < window (window None: every earlier position)."""
    i = torch.arange(T)
    dist = i[:, None] - i[None, :]
    ok = dist >= 0
    if window is not None:
        ok = ok & (dist < int(window))
    return ok


def sink_softmax(scores, ok, sink):
    """scores [H, T, T]; softmax over the visible keys of each row whose denominator also holds exp(sink_h): a
    column of its own, without a value."""
    H, T, _ = scores.shape
    s = scores.masked_fill(~ok[None], float("-inf"))
    full = torch.cat([s, sink.to(s.dtype).view(H, 1, 1).expand(H, T, 1)], 2)
    return torch.softmax(full, 2)[:, :, :T]


def rotate_pairs(x, dims, base):
    """x [T, heads, D]: dimensions (2i, 2i + 1), i < dims / 2, of every head turn by position * base^(-2i/dims)."""
    T = x.shape[0]
    half = dims // 2
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    ang = torch.arange(T, dtype=torch.float64)[:, None] * f[None]
    c, s = torch.cos(ang).to(x.dtype)[:, None], torch.sin(ang).to(x.dtype)[:, None]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def attention_values(h, W, p):
    return h @ W[p + "v"].T + W[p + "v.b"]


def attention_inputs(q, k, qw, kw, m, eps):
    """q [T, H D], k [T, G D] as projected -> (q [T, H, D], k [T, G, D]): RMS norm over each whole projection with
    its plain weight, split into heads, pairwise rotation."""
    T = q.shape[0]
    H, G, D = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = (rms_unit(q, eps) * qw).view(T, H, D)
    k = (rms_unit(k, eps) * kw).view(T, G, D)
    rot = m.get("rot")
    if rot:
        q = rotate_pairs(q, int(rot["dims"]), float(rot["base"]))
        k = rotate_pairs(k, int(rot["dims"]), float(rot["base"]))
    return q, k


def windowed_attention(q, k, v, scale, window, sink):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] (query head h reads key/value head h // (H / G)) -> [T, H Dv]."""
    T, H = q.shape[0], q.shape[1]
    rep = H // k.shape[1]
    kh = k.repeat_interleave(rep, 1).permute(1, 0, 2)
    vh = v.repeat_interleave(rep, 1).permute(1, 0, 2)
    s = torch.einsum("thd,hjd->htj", q, kh) * float(scale)
    pw = sink_softmax(s, visible(T, window), sink)
    return torch.einsum("htj,hjv->thv", pw, vh).reshape(T, -1)


def attention(h, W, p, m, eps, v_first=None):
    """Grouped-query attention with whole-projection query / key norms, pairwise rotation, a sliding window and a
    sink. ``v_first``: the values of the first value-mixing layer when this is a later one."""
    T = h.shape[0]
    G, Dv = int(m["kv_heads"]), int(m["vdim"])
    q = h @ W[p + "q"].T + W[p + "q.b"]
    k = h @ W[p + "k"].T + W[p + "k.b"]
    v = attention_values(h, W, p)
    q, k = attention_inputs(q, k, W[p + "q.norm"], W[p + "k.norm"], m, eps)
    if v_first is not None:
        lam = W[p + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    win = (m.get("mask") or {}).get("size")
    o = windowed_attention(q, k, v.view(T, G, Dv), m["scale"], win, W[p + "sink"])
    return o @ W[p + "o"].T


def latent_attention(h, W, p, m, eps):
    """Attention over keys and values that are projections of one normed latent row per token; no positions."""
    T = h.shape[0]
    H, D, Dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T).view(T, H, D)
    c = rms_unit(h @ W[p + "dkv"].T, eps) * W[p + "dkv.norm"]
    k = (c @ W[p + "uk"].T).view(T, H, D)
    v = (c @ W[p + "uv"].T).view(T, H, Dv)
    win = (m.get("mask") or {}).get("size")
    o = windowed_attention(q, k, v, m["scale"], win, W[p + "sink"])
    return o @ W[p + "o"].T


def swish_clamp(g, u, limit, alpha=1.702):
    g = g.clamp(max=limit)
    u = u.clamp(min=-limit, max=limit)
    return g * torch.sigmoid(alpha * g) * (u + 1.0)


def expert(h, W, p, limit):
    """Clamped gated unit: gate capped from above, up clamped both ways, gate * sigmoid(1.702 gate) * (up + 1)."""
    return swish_clamp(h @ W[p + "gate"].T, h @ W[p + "up"].T, limit) @ W[p + "down"].T


def route_logits(z, correction, top, n_g, keep):
    """Router logits z [T, E] -> (weights [T, top], experts [T, top])."""
    T, E = z.shape
    s = torch.softmax(z, -1)
    choice = s + correction
    gs = choice.view(T, n_g, E // n_g).max(-1).values
    best = gs.topk(keep, -1).indices
    allowed = torch.zeros(T, n_g, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    allowed = allowed[:, :, None].expand(T, n_g, E // n_g).reshape(T, E)
    idx = choice.masked_fill(~allowed, float("-inf")).topk(top, -1).indices
    w = s.gather(1, idx)
    return w / (w.sum(-1, keepdim=True) + 1e-20), idx


def route(h, W, p, mlp):
    """(weights [T, top], experts [T, top]): softmax over all experts; the choice adds the correction and keeps only
    the best groups; the weights are the uncorrected scores of the chosen, normalised."""
    r = mlp["router"]
    gr = r.get("groups") or {}
    return route_logits(h @ W[p + "router"].T, W[p + "correction"], int(r["top"]), int(gr.get("count", 1)),
                        int(gr.get("keep", 1)))


def feed_forward(h, W, p, mlp):
    if mlp.get("kind", "moe") != "moe":
        raise ValueError("unknown feed-forward")
    w, idx = route(h, W, p, mlp)
    limit = float(mlp["expert"]["limit"])
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for j in range(idx.shape[1]):
            e = int(idx[t, j])
            out[t] += w[t, j] * expert(h[t:t + 1], W, f"{p}e{e}.", limit)[0]
    sh = mlp.get("shared")
    if sh:
        gate = torch.sigmoid(h @ W[p + "shared.sg"].T)
        out = out + gate * expert(h, W, p + "shared.", float(sh["limit"]))
    return out


def hyper_step(xs, W, p, sub, eps):
    """One sublayer on the streams xs [S, T, d]: read a weighted sum, run the sublayer on its norm, then mix all
    streams among themselves (matrix indexed [from, to]) and add the sublayer's output with per-stream weights."""
    u = torch.einsum("s,std->td", W[p + "in"], xs)
    y = sub(u)
    return torch.einsum("sr,std->rtd", W[p + "mix"], xs) + W[p + "out"][:, None, None] * y[None]


def forward(cfg: dict, W: dict, tokens, dtype=torch.float64, layers_out: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence. ``layers_out`` receives the sum of the streams after every layer."""
    W = {k: v.to(dtype) for k, v in W.items()}
    eps = float(cfg["norm"]["eps"])
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    S = cfg.get("streams")
    xs = x[None].repeat(int(S), 1, 1) if S else None
    v_first = None
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]

        def mixer(u):
            nonlocal v_first
            h = norm_plus_one(u, W[p + "norm1"], eps)
            if L["type"] == "attention":
                if m.get("v_mix"):
                    if v_first is None:
                        v_first = attention_values(h, W, p + "mix.")
                        return attention(h, W, p + "mix.", m, eps)
                    return attention(h, W, p + "mix.", m, eps, v_first)
                return attention(h, W, p + "mix.", m, eps)
            if L["type"] == "latent_attention":
                return latent_attention(h, W, p + "mix.", m, eps)
            raise ValueError(L["type"])

        def ff(u):
            return feed_forward(norm_plus_one(u, W[p + "norm2"], eps), W, p + "mlp.", L["mlp"])

        if xs is not None:
            xs = hyper_step(xs, W, p + "hc1.", mixer, eps)
            if L.get("mlp"):
                xs = hyper_step(xs, W, p + "hc2.", ff, eps)
            x = xs.sum(0)
        else:
            x = x + mixer(x)
            if L.get("mlp"):
                x = x + ff(x)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_plus_one(x, W["final.norm"], eps) @ W["head"].T
