"""fp32 PyTorch references of the hybrid-model ops in ``ops/hybrid.py`` (CPU tensors: unit tests, CPU-only runs).

Same signatures and in-place effects as the HIP kernels of ``csrc/hybrid.hip``. Every op works on a step's flat token
rows; ``seg`` int32 [R, 4] = (first row, rows, first position, state slot) names the step's segments (one per
sequence in the step) and ``tok_seg`` int32 [T] the segment of each row. A segment whose first position is 0 starts
from zero state whatever its slot holds.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z * z * z)))


def _ln(x, w, b, eps):
    x = x.float()
    m = x.mean(-1, keepdim=True)
    d = x - m
    return d * torch.rsqrt((d * d).mean(-1, keepdim=True) + eps) * w.float() + b.float()


def ln_shift(x, w, b, eps, out, mu=None, tok_seg=None, seg=None, state=None, last=None):
    h = _ln(x, w, b, eps)
    if mu is None:
        out.copy_(h)
        return
    prev = torch.zeros_like(h)
    prev[1:] = h[:-1]
    for s, (q0, n, p0, slot) in enumerate(seg.tolist()):
        prev[q0] = state[slot] if p0 > 0 else 0.0
        last[s] = h[q0 + n - 1]
    out.copy_(h + (prev - h) * mu.float())


def scatter_rows(dst, seg, src):
    dst[seg[:, 3].long()] = src[:seg.shape[0]].to(dst.dtype)


def add_ln(x, y, w, b, eps, out2=None, w2=None, b2=None):
    x += _ln(y, w, b, eps)
    if out2 is not None:
        out2.copy_(_ln(x, w2, b2, eps) if w2 is not None else x)


def gelu_mul(gu, out):
    Fh = out.shape[-1]
    g = gu.float()
    out.copy_(gelu_tanh(g[:, :Fh]) * g[:, Fh:])


def side_gate(sg, tokens, side_embed, col0, out):
    dim = out.shape[-1]
    e = side_embed[tokens.long(), col0:col0 + dim].float()
    out.copy_(gelu_tanh(sg.float()) * e)


def side_dwa(x, y, side_w, eps, stack, layer, dwa):
    if y is not None:
        yf = y.float()
        x += yf * torch.rsqrt((yf * yf).mean(-1, keepdim=True) + eps) * side_w.float()
    if stack is not None:
        stack[layer + 1].copy_(x)
        if dwa is not None:
            x.copy_((dwa.float()[:, None, None] * stack[:layer + 2]).sum(0))


def latent_prep(qgd, H, dim, rd, R, dkv_off, dkv_w, eps, positions, cos_sin, rot_dims, cache, slot_mapping, q_rot):
    """qgd [T, ...]: the fused projection's row: q heads ([dim | rd] each) first, the latent pair at ``dkv_off``
    (< 0: the layer borrows its cache). Writes [normed latent | rotated shared key] into ``cache`` rows and the
    rotated query parts into ``q_rot`` [T, H, rd]."""
    T = qgd.shape[0]
    half = rot_dims // 2
    cs = cos_sin[positions.long()] if cos_sin is not None else torch.zeros(T, 0)
    c, s = cs[:, :half], cs[:, half:]

    def rot(v):  # [T, ..., rd]
        shp = [T] + [1] * (v.dim() - 2) + [half]
        cc, ss = c.view(shp), s.view(shp)
        u, w = v[..., :half], v[..., half:rot_dims]
        return torch.cat([u * cc - w * ss, w * cc + u * ss, v[..., rot_dims:]], -1)

    q = qgd[:, :H * (dim + rd)].float().view(T, H, dim + rd)
    q_rot.copy_(rot(q[..., dim:]))
    if dkv_off >= 0:
        dkv = qgd[:, dkv_off:dkv_off + R + rd].float()
        lat = dkv[:, :R]
        lat = lat * torch.rsqrt((lat * lat).mean(-1, keepdim=True) + eps) * dkv_w.float()
        row = torch.cat([lat, rot(dkv[:, R:])], -1).to(cache.dtype)
        ok = slot_mapping >= 0
        cache.view(-1, R + rd)[slot_mapping[ok].long()] = row[ok]


def latent_attn(q_lat, q_rot, cache, block_tables, tok_seg, seg, positions, scale, out, window=0, sink=None):
    """q_lat [H, T, R], q_rot [T, H, rd], cache [pages, page, R + rd]; out [H, T, R] = softmax-weighted latents over
    the keys of the row's window (0: all earlier ones); ``sink`` [H] joins the denominator only."""
    H, T, R = q_lat.shape
    page = cache.shape[1]
    flat = cache.view(-1, cache.shape[-1]).float()
    for t in range(T):
        r = int(tok_seg[t])
        n = int(positions[t]) + 1
        pages = block_tables[r, :(n + page - 1) // page].long()
        idx = (pages[:, None] * page + torch.arange(page)[None]).reshape(-1)[:n]
        kv = flat[idx]
        if window:
            kv = kv[max(0, n - window):]
        s = (q_lat[:, t].float() @ kv[:, :R].T + q_rot[t].float() @ kv[:, R:].T) * scale
        if sink is not None:
            s = torch.cat([s, sink.float()[:, None]], 1)
        out[:, t] = (torch.softmax(s, -1)[:, :kv.shape[0]] @ kv[:, :R]).to(out.dtype)


def sigmoid_mul(a, g, out):
    """a [H, T, v] (head-major), g [T, H * v] -> out [T, H * v]."""
    H, T, v = a.shape
    out.copy_(a.float().permute(1, 0, 2).reshape(T, H * v) * torch.sigmoid(g.float()))


def conv_silu(proj, c0, w, b, tok_seg, seg, state, out):
    C, taps = w.shape
    u = proj[:, c0:c0 + C].float()
    for q0, n, p0, slot in seg.tolist():
        hist = state[slot].float() if p0 > 0 else torch.zeros(taps - 1, C)
        full = torch.cat([hist, u[q0:q0 + n]], 0)
        acc = b.float().expand(n, C).clone()
        for k in range(taps):
            acc = acc + full[k:k + n] * w[:, k].float()
        out[q0:q0 + n] = F.silu(acc).to(out.dtype)
        state[slot] = full[n:].to(state.dtype)


def ssm_scan(xbc, proj, dt_off, dt_bias, A_log, D, heads, P, N, G, tok_seg, seg, state, y):
    """xbc [T, heads * P + 2 G N] (after conv + silu), raw dt at proj[:, dt_off + h]; state f32 [slots, heads, N, P]."""
    inner = heads * P
    grp = torch.arange(heads) // (heads // G)
    A = -torch.exp(A_log.float())
    for q0, n, p0, slot in seg.tolist():
        S = state[slot].clone() if p0 > 0 else torch.zeros(heads, N, P)
        for t in range(q0, q0 + n):
            x = xbc[t, :inner].float().view(heads, P)
            B = xbc[t, inner:inner + G * N].float().view(G, N)[grp]
            C = xbc[t, inner + G * N:].float().view(G, N)[grp]
            dt = F.softplus(proj[t, dt_off:dt_off + heads].float() + dt_bias.float(), threshold=1e9)
            S = torch.exp(A * dt)[:, None, None] * S + (dt[:, None] * B)[:, :, None] * x[:, None, :]
            y[t] = (torch.einsum("hnp,hn->hp", S, C) + D.float()[:, None] * x).reshape(-1)
        state[slot] = S


def gated_norm(y, proj, w, groups, eps, out):
    T, inner = y.shape
    v = y.float() * F.silu(proj[:, :inner].float())
    v = v.view(T, groups, inner // groups)
    v = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps)
    out.copy_(v.reshape(T, inner) * w.float())


# ---- gated mixers: sigmoid attention, real-gated linear recurrence, matrix memory, routed experts --------------------
def rms_norm(x, w, eps, out):
    v = x.float()
    out.copy_(v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps) * w.float())


def short_conv(u, c0, w, b, tok_seg, seg, state, out, act="none", residual=False):
    """Causal per-channel convolution over columns [c0, c0 + C) of ``u``: out_t = act(b + sum_k w[:, k] u_(t - taps + 1
    + k)) (+ u_t with ``residual``); ``state`` [slots, taps - 1, C] holds each sequence's last inputs and is advanced."""
    C, taps = w.shape
    x = u[:, c0:c0 + C].float()
    for q0, n, p0, slot in seg.tolist():
        hist = state[slot].float() if p0 > 0 and taps > 1 else torch.zeros(taps - 1, C)
        full = torch.cat([hist, x[q0:q0 + n]], 0)
        acc = b.float().expand(n, C).clone() if b is not None else torch.zeros(n, C)
        for k in range(taps):
            acc = acc + full[k:k + n] * w[:, k].float()
        if act == "silu":
            acc = F.silu(acc)
        if residual:
            acc = acc + x[q0:q0 + n]
        out[q0:q0 + n] = acc.to(out.dtype)
        if taps > 1:
            state[slot] = full[n:].to(state.dtype)


def kv_store(src, k_off, v_off, k_cache, v_cache_t, slot_mapping):
    """Row t's key columns -> k_cache [pages, page, Ck] at its slot; its value columns -> v_cache_t [pages, Cv, page]
    (each page transposed: a channel's 16 tokens are consecutive)."""
    page, Ck = k_cache.shape[1], k_cache.shape[2]
    Cv = v_cache_t.shape[1]
    ok = slot_mapping >= 0
    sl = slot_mapping[ok].long()
    k_cache.view(-1, Ck)[sl] = src[ok][:, k_off:k_off + Ck].to(k_cache.dtype)
    v_cache_t[sl // page, :, sl % page] = src[ok][:, v_off:v_off + Cv].to(v_cache_t.dtype)


def sigmoid_attn(q, q_off, k_cache, v_cache_t, block_tables, tok_seg, positions, H, G, scale, softcap, t_coef,
                 t_every, r1, r2, pb, out):
    """q rows [T, >= q_off + H D]; out [T, H Dv] = sum over keys j <= position of
    sigmoid(cap(q . k_j scale temp) - r1 ln(1 + r2 (position - j)) + pb) v_j per head, not normalised."""
    T = q.shape[0]
    page, D = k_cache.shape[1], k_cache.shape[2] // G
    Dv = v_cache_t.shape[1] // G
    for t in range(T):
        r, p = int(tok_seg[t]), int(positions[t])
        n = p + 1
        pages = block_tables[r, :(n + page - 1) // page].long()
        k = k_cache[pages].reshape(-1, G, D)[:n].float()                       # [n, G, D]
        v = v_cache_t[pages].permute(0, 2, 1).reshape(-1, G, Dv)[:n].float()   # [n, G, Dv]
        temp = 1.0 + t_coef * math.log(math.floor((p + 1) / t_every) + 1.0) if t_coef else 1.0
        dist = (p - torch.arange(n)).float()
        qt = q[t, q_off:q_off + H * D].float().view(H, D)
        for h in range(H):
            g = h // (H // G)
            s = (k[:, g] @ qt[h]) * (scale * temp)
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            s = s - r1[h] * torch.log1p(r2[h] * dist) + pb[h]
            out[t, h * Dv:(h + 1) * Dv] = (torch.sigmoid(s) @ v[:, g]).to(out.dtype)


def rglru_scan(gates, proj, u, rate, tok_seg, seg, state, out):
    """gates fp32 [T, 2 W] = pre-activations of the recurrence gate | the input gate (biases included), proj [T, >= W]
    whose first W columns are the raw gelu branch, u [T, W] the convolved branch, rate fp32 [W] = -8 softplus(lam):
    a = exp(rate sigmoid(g_r)), S <- a S + sqrt(1 - a^2) sigmoid(g_i) u, out = S gelu(branch); state fp32 [slots, W]."""
    Wd = u.shape[1]
    la = rate.float() * torch.sigmoid(gates[:, :Wd].float())
    a = torch.exp(la)
    inp = torch.sqrt(-torch.expm1(2.0 * la)) * torch.sigmoid(gates[:, Wd:].float()) * u.float()
    y = gelu_tanh(proj[:, :Wd].float())
    for q0, n, p0, slot in seg.tolist():
        S = state[slot].clone() if p0 > 0 else torch.zeros(Wd)
        for t in range(q0, q0 + n):
            S = a[t] * S + inp[t]
            out[t] = (S * y[t]).to(out.dtype)
        state[slot] = S


def mlstm_scan(qkv, gates, H, D, Dv, cap, tok_seg, seg, S, nrm, mx, out):
    """qkv [T, >= H (2 D + Dv)] = q | k | v heads (q still unscaled), gates fp32 [T, 2 H] = raw input | forget gate
    (biases included). Per head, with i = cap tanh(g_i / cap), f = logsigmoid(cap tanh(g_f / cap)):
    m' = max(f + m, i), S <- e^(f + m - m') S + e^(i - m') k v^T, n likewise with k,
    out = S^T q' / (max(|n . q'|, e^(-m')) + 1e-6), q' = q D^(-1/2). State per slot: S [H, D, Dv], n [H, D], m [H],
    all fp32, zero (m too) before a sequence's first token. out fp32 [T, H Dv]."""
    for q0, n, p0, slot in seg.tolist():
        if p0 > 0:
            Ss, ns, ms = S[slot].clone(), nrm[slot].clone(), mx[slot].clone()
        else:
            Ss, ns, ms = torch.zeros(H, D, Dv), torch.zeros(H, D), torch.zeros(H)
        for t in range(q0, q0 + n):
            q = qkv[t, :H * D].float().view(H, D) * D ** -0.5
            k = qkv[t, H * D:2 * H * D].float().view(H, D)
            v = qkv[t, 2 * H * D:2 * H * D + H * Dv].float().view(H, Dv)
            ig = cap * torch.tanh(gates[t, :H].float() / cap)
            fg = F.logsigmoid(cap * torch.tanh(gates[t, H:].float() / cap))
            m_new = torch.maximum(fg + ms, ig)
            dec, gain = torch.exp(fg + ms - m_new), torch.exp(ig - m_new)
            Ss = dec[:, None, None] * Ss + gain[:, None, None] * k[:, :, None] * v[:, None, :]
            ns = dec[:, None] * ns + gain[:, None] * k
            ms = m_new
            num = torch.einsum("hdv,hd->hv", Ss, q)
            den = torch.maximum((ns * q).sum(-1).abs(), torch.exp(-ms)) + 1e-6
            out[t] = (num / den[:, None]).reshape(-1)
        S[slot], nrm[slot], mx[slot] = Ss, ns, ms


def head_norm_gate(o, w, g, g_off, H, eps, out, scale=1.0):
    """out = unit_rms_per_head(o) * w * sigmoid(g[:, g_off : g_off + H Dv]) * scale (o fp32 [T, H Dv]; no gate
    when ``g`` is None)."""
    T, n = o.shape
    v = o.float().view(T, H, n // H)
    v = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps)
    v = v.reshape(T, n) * w.float()
    if g is not None:
        v = v * torch.sigmoid(g[:, g_off:g_off + n].float())
    out.copy_((v * scale).to(out.dtype))


def moe_router(h, w, b, k, topk_w, topk_e):
    """fp32 logits h W^T + b; the k largest (ties: the lower index first) and a softmax over those k."""
    z = h.float() @ w.float().T + b.float()
    val, idx = torch.sort(z, dim=-1, descending=True, stable=True)
    topk_e.copy_(idx[:, :k])
    topk_w.copy_(torch.softmax(val[:, :k], -1))


def _glu(gu, Fh, limit, alpha):
    g, u = gu[:, :Fh], gu[:, Fh:]
    if limit > 0:
        g, u = g.clamp(max=limit), u.clamp(min=-limit, max=limit)
        return g * torch.sigmoid(alpha * g) * (u + 1.0)
    return F.silu(g) * u


def moe_rows(h, w_gu, w_down, topk_w, topk_e, out, limit=0.0, alpha=1.0):
    """out[t] = sum_j topk_w[t, j] W_down[e] act(W_gate[e] h_t, W_up[e] h_t), e = topk_e[t, j]; w_gu [E, 2 F, d]
    = gate rows then up rows, w_down [E, d, F]; act = silu(g) * u, or with a limit the clamped swish form."""
    T, k = topk_e.shape
    Fh = w_down.shape[2]
    hf = h.float()
    acc = torch.zeros(T, w_down.shape[1])
    for j in range(k):
        e = topk_e[:, j].long()
        gu = torch.einsum("tfd,td->tf", w_gu[e].float(), hf)
        a = _glu(gu, Fh, limit, alpha).to(h.dtype).float()
        acc += topk_w[:, j:j + 1].float() * torch.einsum("tdf,tf->td", w_down[e].float(), a)
    out.copy_(acc)


def add2(x, y1, y2=None):
    """x += y1 (+ y2), summed in fp32."""
    s = y1.float() if y2 is None else y1.float() + y2.float()
    x += s


def stream_step(xs, y, mix, write, read, norm_w, eps, out, y2, row_scale, total, center=False):
    """xs fp32 [S, T, d]: optional write (all streams from the old ones), optional normed read (RMS norm, or with
    ``center`` a layer norm without bias), optional sum."""
    if mix is not None:
        ys = y.float()
        if y2 is not None:
            ys = ys + row_scale.float()[:, None] * y2.float()
        new = torch.einsum("sr,std->rtd", mix.float(), xs) + write.float()[:, None, None] * ys[None]
        xs.copy_(new)
    if read is not None:
        u = torch.einsum("s,std->td", read.float(), xs)
        if center:
            u = u - u.mean(-1, keepdim=True)
        out.copy_((u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * norm_w.float()).to(out.dtype))
    if total is not None:
        total.copy_(xs.sum(0))


def swish_clamp_mul(gu, limit, alpha, out):
    out.copy_(_glu(gu.float(), gu.shape[1] // 2, limit, alpha).to(out.dtype))


def qk_norm_rope_store(qkv, H, G, D, Dv, q_w, k_w, eps, positions, cos_sin, rot_dims, v_first, v_first_off, lam,
                       k_cache, v_cache_t, slot_mapping, q_out):
    T = qkv.shape[0]
    Cq, Ck, Cv = H * D, G * D, G * Dv
    q, k, v = (t.float() for t in qkv[:, :Cq + Ck + Cv].split([Cq, Ck, Cv], 1))
    q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_w.float()
    k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_w.float()
    q, k = q.view(T, H, D).clone(), k.view(T, G, D).clone()
    if rot_dims:
        half = rot_dims // 2
        cs = cos_sin[positions.long()]
        c, s = cs[:, None, :half], cs[:, None, half:]
        for x in (q, k):
            a, b = x[..., 0:rot_dims:2].clone(), x[..., 1:rot_dims:2].clone()
            x[..., 0:rot_dims:2] = a * c - b * s
            x[..., 1:rot_dims:2] = b * c + a * s
    if v_first is not None:
        v = (1.0 - lam) * v + lam * v_first[:, v_first_off:v_first_off + Cv].float()
    q_out.copy_(q.reshape(T, Cq).to(q_out.dtype))
    kv_store(torch.cat([k.reshape(T, Ck), v], 1).to(k_cache.dtype), 0, Ck, k_cache, v_cache_t, slot_mapping)


def window_attn(q, k_cache, v_cache_t, block_tables, tok_seg, positions, H, G, scale, window, sink, out,
                shared_keys=False):
    """``shared_keys``: every query head is a row of the whole key row's size and meets all G key heads at once
    (queries that already hold a mix over the heads); values stay per key/value head."""
    T = q.shape[0]
    page, D = k_cache.shape[1], k_cache.shape[2] // G
    Dv = v_cache_t.shape[1] // G
    rep = H // G
    for t in range(T):
        r, n = int(tok_seg[t]), int(positions[t]) + 1
        pages = block_tables[r, :(n + page - 1) // page].long()
        lo = max(0, n - window) if window else 0
        k = k_cache[pages].reshape(-1, G, D)[lo:n].float()                       # [n, G, D]
        v = v_cache_t[pages].permute(0, 2, 1).reshape(-1, G, Dv)[lo:n].float()   # [n, G, Dv]
        if shared_keys:
            s = torch.einsum("hc,jc->hj", q[t].float().view(H, G * D), k.reshape(-1, G * D)) * scale
        else:
            s = torch.einsum("hd,jhd->hj", q[t].float().view(H, D), k.repeat_interleave(rep, 1)) * scale
        if sink is not None:
            s = torch.cat([s, sink.float()[:, None]], 1)
        pw = torch.softmax(s, -1)[:, :n - lo]
        out[t] = torch.einsum("hj,jhv->hv", pw, v.repeat_interleave(rep, 1)).reshape(H * Dv).to(out.dtype)


def moe_router_grouped(h, w, E, correction, k, groups, keep, eps, topk_w, topk_e, gate):
    z = h.float() @ w.float().T
    s = torch.softmax(z[:, :E], -1)
    choice = s + correction.float()
    T = h.shape[0]
    gsz = E // groups
    gs = choice.view(T, groups, gsz).max(-1).values
    gi = torch.sort(gs, dim=-1, descending=True, stable=True).indices[:, :keep]
    ok = torch.zeros(T, groups, dtype=torch.bool)
    ok.scatter_(1, gi, True)
    choice = choice.masked_fill(~ok[:, :, None].expand(T, groups, gsz).reshape(T, E), float("-inf"))
    idx = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :k]
    wv = s.gather(1, idx)
    topk_e.copy_(idx)
    topk_w.copy_(wv / (wv.sum(-1, keepdim=True) + eps))
    if gate is not None:
        gate.copy_(torch.sigmoid(z[:, E]))


# ---- gated recurrences beside attention: minGRU, HGRN2; rotation + head mix + paged store ---------------------------
def act_norm(x, c0, n, w, eps, out, center=False):
    """out = norm(x[:, c0 : c0 + n]) * w: RMS norm, or with ``center`` a layer norm without bias."""
    u = x[:, c0:c0 + n].float()
    if center:
        u = u - u.mean(-1, keepdim=True)
    out.copy_((u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * w.float()).to(out.dtype))


def gate_mul(a, g, g_off, scale, out):
    """out = a * sigmoid(g[:, g_off : g_off + n]) * scale."""
    n = a.shape[1]
    out.copy_((a.float() * torch.sigmoid(g[:, g_off:g_off + n].float()) * scale).to(out.dtype))


def mingru_scan(proj, bias, Wd, tok_seg, seg, state, out):
    """proj [T, >= 3 W] = pre-activations of the update gate | the candidate | the output gate, bias fp32 [2 W] for
    the first two: z = sigmoid(.), c = u + 1/2 where u >= 0 else sigmoid(u), S <- (1 - z) S + z c,
    out = S silu(g); state fp32 [slots, W]."""
    z = torch.sigmoid(proj[:, :Wd].float() + bias[:Wd].float())
    u = proj[:, Wd:2 * Wd].float() + bias[Wd:].float()
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = proj[:, 2 * Wd:3 * Wd].float()
    y = g * torch.sigmoid(g)
    for q0, n, p0, slot in seg.tolist():
        S = state[slot].clone() if p0 > 0 else torch.zeros(Wd)
        for t in range(q0, q0 + n):
            S = (1.0 - z[t]) * S + z[t] * c[t]
            out[t] = (S * y[t]).to(out.dtype)
        state[slot] = S


def hgrn2_scan(proj, q_off, f_off, v_off, f_bias, lower, H, D, Dv, tok_seg, seg, S, out):
    """Per head: f = lower + (1 - lower) sigmoid(raw f + bias) per key channel, S <- diag(f) S + (1 - f) v^T,
    out = S^T silu(raw q). proj [T, ...] holds raw q (H D) at q_off, raw f (H D) at f_off, v (H Dv) at v_off;
    S fp32 [slots, H, D, Dv]; out fp32 [T, H Dv]."""
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * D].float()
    q = (q * torch.sigmoid(q)).view(T, H, D)
    lo = lower.float()
    f = (lo + (1.0 - lo) * torch.sigmoid(proj[:, f_off:f_off + H * D].float() + f_bias.float())).view(T, H, D)
    v = proj[:, v_off:v_off + H * Dv].float().view(T, H, Dv)
    for q0, n, p0, slot in seg.tolist():
        St = S[slot].clone() if p0 > 0 else torch.zeros(H, D, Dv)
        for t in range(q0, q0 + n):
            St = f[t][:, :, None] * St + (1.0 - f[t])[:, :, None] * v[t][:, None, :]
            out[t] = torch.einsum("hdv,hd->hv", St, q[t]).reshape(-1)
        S[slot] = St


def rope_kv_store(qkv, H, G, D, Dv, positions, cos_sin, rot_dims, pairs, talk, k_cache, v_cache_t, slot_mapping,
                  q_out):
    """Fused projection row [q (H D) | k (G D) | v (G Dv)]: rotation of the first rot_dims dimensions of every q and
    k head (partners i, i + rot_dims / 2, or with ``pairs`` 2i, 2i + 1), keys and values into their pages. With
    ``talk`` fp32 [H, H] the queries leave as q'[h] = [sum over the heads g of key head c of talk[h, g] q[g]] for
    c = 0 .. G - 1 (row size G D): q'[h] . (whole key row) is the head-mixed score."""
    T = qkv.shape[0]
    Cq, Ck, Cv = H * D, G * D, G * Dv
    q, k, v = (t.float() for t in qkv[:, :Cq + Ck + Cv].split([Cq, Ck, Cv], 1))
    q, k = q.view(T, H, D).clone(), k.view(T, G, D).clone()
    if rot_dims:
        half = rot_dims // 2
        cs = cos_sin[positions.long()]
        c, s = cs[:, None, :half], cs[:, None, half:]
        for x in (q, k):
            if pairs:
                a, b = x[..., 0:rot_dims:2].clone(), x[..., 1:rot_dims:2].clone()
                x[..., 0:rot_dims:2] = a * c - b * s
                x[..., 1:rot_dims:2] = b * c + a * s
            else:
                a, b = x[..., :half].clone(), x[..., half:rot_dims].clone()
                x[..., :half] = a * c - b * s
                x[..., half:rot_dims] = b * c + a * s
    if talk is not None:
        rep = H // G
        q = torch.einsum("hcr,tcrd->thcd", talk.float().view(H, G, rep), q.view(T, G, rep, D)).reshape(T, H * Ck)
    q_out.copy_(q.reshape(T, -1).to(q_out.dtype))
    kv_store(torch.cat([k.reshape(T, Ck), v], 1).to(k_cache.dtype), 0, Ck, k_cache, v_cache_t, slot_mapping)
