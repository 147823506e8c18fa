"""Mozidra in the serving engine against the plain whole-sequence implementation of tests/mozidra_plain.py.

Small configurations of odd sizes (nothing a multiple of 64, head sizes that differ between keys and values and
between layers, windows that end inside pages, a layer without feed-forward, a model without streams) with random
weights made here. Each test runs on the CPU reference ops and, marked ``gpu``, on the HIP kernels.
"""
import copy
import math

import pytest
import torch

import mozidra_plain as plain
from kafka_llm_service_amd.engine.engine import EngineConfig, LLMEngine
from kafka_llm_service_amd.engine.sequence import SamplingParams
from kafka_llm_service_amd.models import mozidra as mz
from kafka_llm_service_amd.ops import hybrid as hops

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def _attn(heads=6, kv_heads=2, dim=24, vdim=20, window=21, rot=10, base=9000.0, v_mix=False, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = {"base": base, "dims": rot}
    if v_mix:
        m["v_mix"] = True
    return m


def _lat(heads=5, dim=12, vdim=18, rank=40, window=10, scale=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale or dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    return m


def _moe(experts=6, top=2, ff=28, groups=(3, 2), shared=36, limit=0.9):
    r = {"experts": experts, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}
    if shared:
        m["shared"] = {"ff": shared, "limit": 1.3 * limit}
    return m


def cfg_a(scale=None):
    return {"architecture": "Mozidra", "vocab": 211, "width": 88, "norm": {"eps": 2e-5}, "streams": 3,
            "layers": [{"type": "latent_attention", "mixer": _lat(scale=scale), "mlp": _moe()},
                       {"type": "attention", "mixer": _attn(v_mix=True, scale=scale), "mlp": _moe(8, 3, 20, (4, 2), 0)},
                       {"type": "attention", "mixer": _attn(4, 4, 10, 7, window=0, rot=0, scale=scale), "mlp": None},
                       {"type": "latent_attention", "mixer": _lat(3, 20, 9, 33, window=37, scale=scale),
                        "mlp": _moe(5, 2, 36, None, 12)},
                       {"type": "attention", "mixer": _attn(8, 2, 16, 20, window=16, rot=16, base=100.0, v_mix=True,
                                                            scale=scale), "mlp": _moe(4, 1, 24, (4, 1))}]}


def cfg_b():
    """Ones and equal values: no streams, one head, as many key/value heads as query heads, one expert of one, one
    group, no shared expert, a window of one token (a row sees itself only), a full rotation, key and value sizes
    equal."""
    return {"architecture": "Mozidra", "vocab": 97, "width": 48, "norm": {"eps": 1e-6},
            "layers": [{"type": "attention", "mixer": _attn(1, 1, 16, 16, window=1, rot=16, v_mix=True),
                        "mlp": _moe(1, 1, 40, None, 0)},
                       {"type": "latent_attention", "mixer": _lat(1, 16, 16, 16, window=1000),
                        "mlp": _moe(2, 2, 8, (1, 1), 8)},
                       {"type": "attention", "mixer": _attn(3, 1, 8, 16, window=2, rot=2, v_mix=True), "mlp": None},
                       {"type": "latent_attention", "mixer": _lat(2, 8, 8, 8, window=0),
                        "mlp": _moe(4, 1, 8, (2, 2), 8)}]}


def cfg_s1():
    """One stream given as such (the stream tensors exist, with one entry each)."""
    c = cfg_b()
    c["streams"] = 1
    return c


class Bench:
    """A config, its random weights and engines over them."""

    def __init__(self, cfg: dict, seed=0, sharpen=1.0, static_routes=False):
        self.cfg = cfg
        self.mc = mz.MozidraConfig.from_dict(cfg, name="test")
        self.W = mz.random_tensors(self.mc, seed)
        for k in self.W:
            if sharpen != 1.0 and (k.endswith("mix.q.norm") or (k.endswith("mix.q") and k[:-5] + "mix.dkv" in self.W)):
                # scores far from zero: single keys carry the result
                self.W[k] = (self.W[k].float() * sharpen).to(torch.bfloat16)
            if static_routes and k.endswith("correction"):
                # corrections far apart: the choice of experts (and of groups) rarely follows the input, and never
                # hangs on a bf16 rounding (the fp32 benches keep input-driven routes)
                self.W[k] = (torch.arange(self.W[k].numel()).float() * 3.0).roll(seed + len(k)).to(torch.bfloat16)
        self._oracle = {}

    def engine(self, device, dtype="float32", blocks=64, seqs=4, **kw):
        model = mz.MozidraLM(self.mc, device, dtype=getattr(torch, dtype), max_positions=1024).load_tensors(self.W)
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
    return Bench(cfg_a(scale=0.9), seed=3, sharpen=3.0)


# ---- mechanisms alone ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S,d", [(3, 70), (1, 33), (4, 4500), (8, 2300), (13, 1100)])
def test_stream_step(device, S, d):
    """Write, read + norm and sum of the streams, each alone and together, against the plain stream step; rows wider
    than the kernel keeps in registers; bf16 and fp32 sublayer outputs; a second output with a row gate."""
    g = torch.Generator().manual_seed(S * 1000 + d)
    T = 5
    xs0 = torch.randn(S, T, d, generator=g)
    Wt = {"in": torch.randn(S, generator=g), "mix": torch.eye(S) + 0.3 * torch.randn(S, S, generator=g),
          "out": torch.randn(S, generator=g)}
    y, y2 = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g).to(torch.bfloat16)
    gate = torch.rand(T, generator=g)
    nw = 0.2 * torch.randn(d, generator=g)
    eps = 1e-4
    W64 = {k: v.double() for k, v in Wt.items()}
    ysum = y.double() + gate.double()[:, None] * y2.double()
    want_xs = plain.hyper_step(xs0.double(), W64, "", lambda u: ysum, eps)
    want_h = plain.norm_plus_one(torch.einsum("s,std->td", W64["in"], want_xs), nw.double(), eps)
    dv = lambda t: t.to(device)  # noqa: E731
    for out_dt in (torch.float32, torch.bfloat16):
        xs = dv(xs0.clone())
        h = torch.empty(T, d, dtype=out_dt, device=device)
        total = torch.empty(T, d, device=device)
        hops.stream_step(xs, dv(y), dv(Wt["mix"]), dv(Wt["out"]), dv(Wt["in"]), dv(1.0 + nw), eps, h, y2=dv(y2),
                         row_scale=dv(gate), total=total)
        assert (xs.cpu().double() - want_xs).abs().max() < 1e-5 * want_xs.abs().max()
        assert (total.cpu().double() - want_xs.sum(0)).abs().max() < 1e-5 * want_xs.abs().max()
        tol = 1e-5 if out_dt == torch.float32 else 1e-2
        assert (h.float().cpu().double() - want_h).abs().max() < tol * want_h.abs().max()
    # the parts alone: a read of untouched streams; a write without a read
    xs = dv(xs0.clone())
    h = torch.empty(T, d, device=device)
    hops.stream_step(xs, read=dv(Wt["in"]), norm_w=dv(1.0 + nw), eps=eps, out=h)
    assert torch.equal(xs.cpu(), xs0)
    want = plain.norm_plus_one(torch.einsum("s,std->td", W64["in"], xs0.double()), nw.double(), eps)
    assert (h.cpu().double() - want).abs().max() < 1e-5 * want.abs().max()
    hops.stream_step(xs, dv(y.to(torch.bfloat16)), dv(Wt["mix"]), dv(Wt["out"]))
    want = plain.hyper_step(xs0.double(), W64, "", lambda u: y.to(torch.bfloat16).double(), eps)
    assert (xs.cpu().double() - want).abs().max() < 1e-5 * want.abs().max()
    with pytest.raises(ValueError):
        hops.stream_step(xs, read=dv(Wt["in"]))


@pytest.mark.parametrize("device", DEVICES)
def test_swish_clamp(device):
    g = torch.Generator().manual_seed(5)
    gu = 3.0 * torch.randn(9, 2 * 37, generator=g)
    for limit, alpha in ((1.0, 1.702), (2.5, 1.0), (100.0, 0.5)):
        out = torch.empty(9, 37, device=device)
        hops.swish_clamp_mul(gu.to(device), limit, alpha, out)
        want = plain.swish_clamp(gu[:, :37].double(), gu[:, 37:].double(), limit, alpha)
        assert (out.cpu().double() - want).abs().max() < 1e-5
    with pytest.raises(ValueError):
        hops.swish_clamp_mul(gu.to(device), 0.0, 1.0, torch.empty(9, 37, device=device))


class Paged:
    """Scattered pages for sequences of given lengths, fed in given portions: the step tensors the kernels take."""

    def __init__(self, device, lengths, n_pages=None, seed=0):
        self.device = device
        need = sum(-(-n // 16) for n in lengths)
        self.n_pages = n_pages or need + 3
        perm = torch.randperm(self.n_pages, generator=torch.Generator().manual_seed(seed)).tolist()
        self.tables, at = [], 0
        for n in lengths:
            k = -(-n // 16)
            self.tables.append(perm[at:at + k])
            at += k

    def step(self, runs):
        """runs: (sequence, first position, rows) -> block tables, tok_seg, positions, slot mapping"""
        W = max(len(t) for t in self.tables)
        bt = torch.zeros(len(runs), W, dtype=torch.int32)
        ts, pos, sl = [], [], []
        for j, (s, p0, n) in enumerate(runs):
            bt[j, :len(self.tables[s])] = torch.tensor(self.tables[s], dtype=torch.int32)
            for p in range(p0, p0 + n):
                ts.append(j)
                pos.append(p)
                sl.append(self.tables[s][p // 16] * 16 + p % 16)
        d = self.device
        return (bt.to(d), torch.tensor(ts, dtype=torch.int32, device=d), torch.tensor(pos, dtype=torch.long, device=d),
                torch.tensor(sl, dtype=torch.long, device=d))


def _loud(q, k, at, key, head, kv_head, gain):
    """Make row ``at``'s query of ``head`` point at key ``key`` of ``kv_head``: one score stands out."""
    k[key, kv_head] = k[key, kv_head] / k[key, kv_head].norm() * gain
    q[at, head] = k[key, kv_head] / gain * gain


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv,window,rot", [(6, 2, 24, 20, 21, 10), (4, 4, 7, 70, 16, 0), (3, 1, 100, 9, 0, 100),
                                                 (2, 1, 8, 8, 1, 8), (8, 1, 16, 130, 33, 6)])
def test_windowed_attention_single_keys(device, H, G, D, Dv, window, rot):
    """The attention inputs (whole-projection norms, pair rotation, value mix, paged store) and the windowed softmax
    with a sink, through scattered pages, in portions, two sequences side by side. Loud keys sit at the first
    position, on both sides of page borders, at the row's own position, on the window's last visible position and one
    before it (which must not count), and far behind the window."""
    g = torch.Generator().manual_seed(H * 100 + D)
    n0, n1 = 150, 23
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv}
    if rot:
        m["rot"] = {"dims": rot, "base": 777.0}
    eps, lam, scale = 1e-5, 0.3, 1.0
    qw, kw = 1.0 + 0.2 * torch.randn(H * D, generator=g), 1.0 + 0.2 * torch.randn(G * D, generator=g)
    sink = torch.randn(H, generator=g)
    seqs = []
    for n in (n0, n1):
        q, k = torch.randn(n, H * D, generator=g), torch.randn(n, G * D, generator=g)
        v, vf = torch.randn(n, G * Dv, generator=g), torch.randn(n, G * Dv, generator=g)
        seqs.append((q, k, v, vf))
    # loud keys for rows of sequence 0: the rotation moves q and k alike only for equal positions, so the loudness is
    # planted after norm and rotation, by solving for the raw rows: simplest with weights 1 and no rotation; with
    # rotation the gain is spread but stays far above the rest
    q, k, v, vf = seqs[0]
    qh, kh = q.view(n0, H, D), k.view(n0, G, D)
    w = window or 10 ** 6
    # (row 97 is fed alone, as a decoded token: its window's last visible key and the one just outside it)
    spots = [(149, 0), (149, 149), (140, 127), (140, 128), (100, 15), (100, 16), (120, max(0, 120 - w + 1)),
             (121, max(0, 121 - w)), (149, 3), (97, max(0, 97 - w + 1)), (97, max(0, 97 - w))]
    for i, (at, key) in enumerate(spots):
        h = i % H
        kh[key, h // (H // G)] = torch.randn(D, generator=g) * 3.0
        qh[at, h] = kh[key, h // (H // G)] * 2.0
    want = []
    for q, k, v, vf in seqs:
        n = q.shape[0]
        qq, kk = plain.attention_inputs(q.double(), k.double(), qw.double(), kw.double(), m, eps)
        vv = ((1.0 - lam) * v.double() + lam * vf.double()).view(n, G, Dv)
        want.append(plain.windowed_attention(qq, kk, vv, scale, window or None, sink.double()))
    pg = Paged(device, [n0, n1], seed=H)
    kc = torch.zeros(pg.n_pages, 16, G * D, device=device)
    vt = torch.zeros(pg.n_pages, G * Dv, 16, device=device)
    cs = None
    if rot:
        from kafka_llm_service_amd.models.budurax import rotary_table
        cs = rotary_table(256, m["rot"], device)
    got = [torch.empty(n0, H * Dv), torch.empty(n1, H * Dv)]
    at = [0, 0]
    for portions in ([(0, 97), (1, 2)], [(1, 20), (0, 1)], [(0, 2)], [(0, 31), (1, 1)], [(0, 19)]):
        runs = [(s, at[s], n) for s, n in portions]
        bt, ts, pos, sl = pg.step(runs)
        rows = torch.cat([torch.cat([seqs[s][0][a:a + n], seqs[s][1][a:a + n], seqs[s][2][a:a + n]], 1)
                          for s, a, n in runs]).to(device)
        vfr = torch.cat([torch.cat([torch.zeros(n, 5), seqs[s][3][a:a + n]], 1) for s, a, n in runs]).to(device)
        qo = torch.empty(rows.shape[0], H * D, device=device)
        hops.qk_norm_rope_store(rows, H, G, D, Dv, qw.to(device), kw.to(device), eps, pos, cs, rot, vfr, 5, lam, kc, vt,
                                sl, qo)
        out = torch.empty(rows.shape[0], H * Dv, device=device)
        hops.window_attn(qo, kc, vt, bt, ts, pos, H, G, scale, window, sink.to(device), out)
        r = 0
        for s, a, n in runs:
            got[s][a:a + n] = out[r:r + n].cpu()
            r += n
            at[s] += n
    assert at == [n0, n1]
    for s in (0, 1):
        assert (got[s].double() - want[s]).abs().max() < 2e-4 * want[s].abs().max(), s


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,window,n", [(8, 2, 32, 48, 40, 300), (4, 4, 16, 20, 129, 700),
                                               (32, 1, 64, 96, 0, 200),
                                               (6, 3, 96, 96, 1, 150), (8, 2, 128, 256, 1000, 1500),
                                               (8, 1, 64, 80, 150, 520)])
def test_windowed_attention_matrix_cores(H, G, D, Dv, window, n):
    """The matrix-core windowed attention (bf16) against the plain function and the vector kernel: prompt portions and
    decode rows, whole key ranges and split ones, loud keys on the window's edges and one outside them."""
    dev = "cuda:0"
    g = torch.Generator().manual_seed(H * D + n)
    w = window or 10 ** 6
    q = torch.randn(n, H, D, generator=g) * 0.5
    k = torch.randn(n, G, D, generator=g)
    v = torch.randn(n, G, Dv, generator=g)
    spots = [(n - 1, 0), (n - 1, n - 1), (140, 127), (140, 128), (100, 15), (120, max(0, 120 - w + 1)),
             (121, max(0, 121 - w)), (n - 1, max(0, n - w)), (n - 2, max(0, n - 2 - w)), (n - 1, max(0, n - 1 - w))]
    for i, (at, key) in enumerate(spots):
        h = i % H
        k[key, h // (H // G)] = torch.randn(D, generator=g) * 2.0
        q[at, h] = k[key, h // (H // G)] * 1.5
    sink = torch.randn(H, generator=g)
    qb, kb, vb = q.to(torch.bfloat16), k.to(torch.bfloat16), v.to(torch.bfloat16)
    scale = D ** -0.5
    want = plain.windowed_attention(qb.double(), kb.double(), vb.double(), scale, window or None, sink.double())
    pg = Paged(dev, [n], seed=5)
    kc = torch.zeros(pg.n_pages, 16, G * D, dtype=torch.bfloat16, device=dev)
    vt = torch.zeros(pg.n_pages, G * Dv, 16, dtype=torch.bfloat16, device=dev)
    tt = hops.sig_tile_tokens(H, G)
    got = torch.empty(n, H * Dv)
    at = 0
    for rows in (n - 40, 1, 38, 1):
        bt, ts, pos, sl = pg.step([(0, at, rows)])
        src = torch.cat([kb[at:at + rows].reshape(rows, -1), vb[at:at + rows].reshape(rows, -1)], 1).to(dev)
        hops.kv_store(src, 0, G * D, kc, vt, sl)
        tiles = torch.tensor([(a, min(tt, rows - a), 0, 0) for a in range(0, rows, tt)], dtype=torch.int32, device=dev)
        qq = qb[at:at + rows].reshape(rows, H * D).contiguous().to(dev)
        assert hops.window_attn_mfma_ok(qq, kc, vt, H, G)
        outs = []
        for max_keys in (0, at + rows):   # unsplit; split key ranges where the launch has few tiles
            out = torch.empty(rows, H * Dv, dtype=torch.bfloat16, device=dev)
            hops.window_attn(qq, kc, vt, bt, ts, pos, H, G, scale, window, sink.to(dev), out, tiles, max_keys)
            outs.append(out.float().cpu())
        vec = torch.empty(rows, H * Dv, dtype=torch.bfloat16, device=dev)
        hops.window_attn(qq, kc, vt, bt, ts, pos, H, G, scale, window, sink.to(dev), vec)
        for o in outs:
            assert (o - vec.float().cpu()).abs().max() < 0.03 * want.abs().max()
        got[at:at + rows] = outs[1]
        at += rows
    assert at == n
    assert (got.double() - want).abs().max() < 0.03 * want.abs().max()
    # without a sink
    out = torch.empty(1, H * Dv, dtype=torch.bfloat16, device=dev)
    hops.window_attn(qq, kc, vt, bt, ts, pos, H, G, scale, window, None, out, tiles, n)
    want0 = plain.windowed_attention(qb.double(), kb.double(), vb.double(), scale, window or None,
                                     torch.full((H,), -1e30).double())
    assert (out.float().cpu().double() - want0[n - 1:]).abs().max() < 0.03 * want0.abs().max()


@pytest.mark.parametrize("device", DEVICES)
def test_attention_without_sink_mix_and_rotation(device):
    """The optional parts switched off: no sink, no earlier values, no rotation, no window."""
    g = torch.Generator().manual_seed(2)
    n, H, G, D, Dv = 40, 4, 2, 12, 9
    q, k = torch.randn(n, H * D, generator=g), torch.randn(n, G * D, generator=g)
    v = torch.randn(n, G * Dv, generator=g)
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv}
    one_q, one_k = torch.ones(H * D), torch.ones(G * D)
    qq, kk = plain.attention_inputs(q.double(), k.double(), one_q.double(), one_k.double(), m, 1e-6)
    # the plain softmax: a sink at minus infinity adds nothing
    want = plain.windowed_attention(qq, kk, v.double().view(n, G, Dv), 0.5, None, torch.full((H,), -1e30).double())
    pg = Paged(device, [n])
    kc, vt = torch.zeros(pg.n_pages, 16, G * D, device=device), torch.zeros(pg.n_pages, G * Dv, 16, device=device)
    bt, ts, pos, sl = pg.step([(0, 0, n)])
    qo = torch.empty(n, H * D, device=device)
    hops.qk_norm_rope_store(torch.cat([q, k, v], 1).to(device), H, G, D, Dv, one_q.to(device), one_k.to(device), 1e-6,
                            pos, None, 0, None, 0, 0.0, kc, vt, sl, qo)
    out = torch.empty(n, H * Dv, device=device)
    hops.window_attn(qo, kc, vt, bt, ts, pos, H, G, 0.5, 0, None, out)
    assert (out.cpu().double() - want).abs().max() < 2e-4 * want.abs().max()


def _latent_case(g, n, H, R, window, spots):
    """Random latent rows and latent-space queries with loud (row, key) pairs; the plain result [H, n, R]."""
    c = torch.randn(n, R, generator=g)
    ql = 0.3 * torch.randn(H, n, R, generator=g)
    for i, (at, key) in enumerate(spots):
        c[key] = torch.randn(R, generator=g) * 2.0
        ql[i % H, at] = c[key] * 1.5
    sink = torch.randn(H, generator=g)
    # keys and values of every head are the latent row itself (identity up-projections)
    kk = c.double()[:, None, :].expand(n, H, R)
    want = plain.windowed_attention(ql.double().permute(1, 0, 2), kk, kk, 1.0, window or None, sink.double())
    return c, ql, sink, want.view(n, H, R).permute(1, 0, 2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,R,window", [(5, 40, 10), (3, 33, 37), (1, 16, 1), (9, 200, 0), (2, 600, 129)])
def test_latent_attention_window_and_sink(device, H, R, window):
    """The latent kernel with a window and a sink, no rotated part, through scattered pages and in portions: loud keys
    at the first position, at page borders, on the window's edge and one outside it."""
    g = torch.Generator().manual_seed(H + R)
    n = 150
    w = window or 10 ** 6
    # (row 97 is fed alone, as a decoded token: its window's last visible key and the one just outside it)
    spots = [(149, 0), (149, 149), (140, 127), (140, 128), (100, 15), (100, 16), (120, max(0, 120 - w + 1)),
             (121, max(0, 121 - w)), (97, max(0, 97 - w + 1)), (97, max(0, 97 - w))]
    c, ql, sink, want = _latent_case(g, n, H, R, window, spots)
    pg = Paged(device, [n], seed=R)
    cache = torch.zeros(pg.n_pages, 16, R, device=device)
    got = torch.empty(H, n, R)
    at = 0
    for rows in (97, 1, 2, 31, 19):
        bt, ts, pos, sl = pg.step([(0, at, rows)])
        qd = torch.cat([torch.zeros(rows, H * 4), c[at:at + rows]], 1).to(device)   # [q heads (unused) | raw latent]
        hops.latent_prep(qd, H, 4, 0, R, H * 4, torch.ones(R, device=device), 0.0, pos, None, 0, cache, sl,
                         torch.empty(rows, H, 0, device=device))
        out = torch.empty(H, rows, R, device=device)
        hops.latent_attn(ql[:, at:at + rows].contiguous().to(device), torch.empty(rows, H, 0, device=device), cache, bt,
                         ts, None, pos, 1.0, out, window=window, sink=sink.to(device))
        got[:, at:at + rows] = out.cpu()
        at += rows
    # (the cache holds unit-RMS rows: compare with the plain result on the normed rows)
    cn = c.double() / c.double().pow(2).mean(-1, keepdim=True).sqrt()
    kk = cn[:, None, :].expand(n, H, R)
    want = plain.windowed_attention(ql.double().permute(1, 0, 2), kk, kk, 1.0, window or None, sink.double())
    want = want.view(n, H, R).permute(1, 0, 2)
    assert (got.double() - want).abs().max() < 2e-4 * want.abs().max()


@pytest.mark.gpu
@pytest.mark.parametrize("H,R,window,n", [(8, 64, 40, 300), (32, 128, 129, 700), (5, 512, 0, 200), (16, 96, 1, 150),
                                          (4, 32, 1000, 1500)])
def test_latent_attention_matrix_cores_window_and_sink(H, R, window, n):
    """The matrix-core latent kernel (bf16) with a window, a sink and no rotated part against the plain function and
    the vector kernel, whole and with split key ranges, decode rows included."""
    dev = "cuda:0"
    g = torch.Generator().manual_seed(H * R)
    w = window or 10 ** 6
    spots = [(n - 1, 0), (n - 1, n - 1), (140, 127), (140, 128), (100, 15), (120, max(0, 120 - w + 1)),
             (121, max(0, 121 - w)), (n - 1, max(0, n - w)), (n - 2, max(0, n - 2 - w)), (n - 1, max(0, n - 1 - w))]
    c, ql, sink, _ = _latent_case(g, n, H, R, window, spots)
    c = c / c.pow(2).mean(-1, keepdim=True).sqrt()
    cb, qb = c.to(torch.bfloat16), ql.to(torch.bfloat16)
    kk = cb.double()[:, None, :].expand(n, H, R)
    want = plain.windowed_attention(qb.double().permute(1, 0, 2), kk, kk, 1.0, window or None, sink.double())
    want = want.view(n, H, R).permute(1, 0, 2)
    pg = Paged(dev, [n], seed=3)
    cache = torch.zeros(pg.n_pages, 16, R, dtype=torch.bfloat16, device=dev)
    cache_t = torch.zeros(pg.n_pages, R, 16, dtype=torch.bfloat16, device=dev)
    assert hops.latent_mfma_ok(cache, R, 0)
    tt = hops.tile_tokens(H)
    got = torch.empty(H, n, R)
    at = 0
    for rows in (n - 40, 1, 38, 1):
        bt, ts, pos, sl = pg.step([(0, at, rows)])
        qd = torch.cat([torch.zeros(rows, H * 8), c[at:at + rows]], 1).to(dev).to(torch.bfloat16)
        hops.latent_prep(qd, H, 8, 0, R, H * 8, torch.ones(R, dtype=torch.bfloat16, device=dev), 0.0, pos, None, 0,
                         cache, sl, torch.empty(rows, H, 0, dtype=torch.bfloat16, device=dev), cache_t)
        tiles = torch.tensor([(a, min(tt, rows - a), 0, 0) for a in range(0, rows, tt)], dtype=torch.int32, device=dev)
        q = qb[:, at:at + rows].contiguous().to(dev)
        qr = torch.empty(rows, H, 0, dtype=torch.bfloat16, device=dev)
        outs = []
        for max_keys in (0, at + rows):   # unsplit; split key ranges where the launch has few tiles
            out = torch.empty(H, rows, R, dtype=torch.bfloat16, device=dev)
            hops.latent_attn(q, qr, cache, bt, ts, None, pos, 1.0, out, cache_t, tiles, max_keys, window=window,
                             sink=sink.to(dev))
            outs.append(out.float().cpu())
        vec = torch.empty(H, rows, R, dtype=torch.bfloat16, device=dev)
        hops.latent_attn(q, qr, cache, bt, ts, None, pos, 1.0, vec, window=window, sink=sink.to(dev))
        for o in outs:
            assert (o - vec.float().cpu()).abs().max() < 0.03 * want.abs().max()
        got[:, at:at + rows] = outs[1]
        at += rows
    assert at == n
    assert (got.double() - want).abs().max() < 0.03 * want.abs().max()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,k,groups,keep,d", [(10, 3, 2, 1, 40), (6, 2, 3, 2, 33), (1, 1, 1, 1, 16), (64, 6, 8, 3, 70),
                                               (300, 12, 1, 1, 33), (16, 4, 16, 4, 20), (70, 5, 7, 7, 9)])
def test_grouped_router(device, E, k, groups, keep, d):
    """Softmax over all experts, choice by corrected score within the best groups, weights from the uncorrected
    scores; with a shared expert's gate row appended. Corrections include large negative ones, so that a masked
    group's score must count as minus infinity and not as zero."""
    g = torch.Generator().manual_seed(E * 10 + k)
    T = 37
    h = torch.randn(T, d, generator=g)
    w = torch.randn(E + 1, d, generator=g) * 2.0 / math.sqrt(d)
    corr = 0.05 * torch.randn(E, generator=g)
    corr[::3] -= 2.0
    tw, te, gate = hops.moe_router_grouped(h.to(device), w.to(device), corr.to(device), k, groups, keep, 1e-20,
                                           extra_gate=True)
    z = h.double() @ w.double().T
    ww, wi = plain.route_logits(z[:, :E], corr.double(), k, groups, keep)
    assert torch.equal(te.cpu().long().sort(-1).values, wi.sort(-1).values)
    order = te.cpu().long().argsort(-1)
    assert (tw.cpu().double().gather(1, order) - ww.gather(1, wi.argsort(-1))).abs().max() < 1e-5
    assert (gate.cpu().double() - torch.sigmoid(z[:, E])).abs().max() < 1e-5
    # without a gate row
    tw2, te2, none = hops.moe_router_grouped(h.to(device), w[:E].to(device), corr.to(device), k, groups, keep, 1e-20)
    assert none is None and torch.equal(te2.cpu(), te.cpu()) and torch.allclose(tw2.cpu(), tw.cpu(), atol=1e-6)


@pytest.mark.parametrize("device", DEVICES)
def test_grouped_router_ties_and_masked_groups(device):
    """Equal scores go to the lower index, for groups and for experts; with all-negative corrected scores an expert
    of a dropped group is never chosen although its score is larger than zero would be."""
    T, E = 3, 8
    h = torch.ones(T, 4)
    w = torch.zeros(E, 4)
    corr = torch.full((E,), -5.0)
    tw, te, _ = hops.moe_router_grouped(h.to(device), w.to(device), corr.to(device), 3, 4, 2)
    assert te.cpu().tolist() == [[0, 1, 2]] * T            # groups 0 and 1 kept, experts in index order
    assert torch.allclose(tw.cpu(), torch.full((T, 3), 1 / 3), atol=1e-6)
    corr[6] = -4.0                                          # group 3 is best; group 0 second by the tie rule
    tw, te, _ = hops.moe_router_grouped(h.to(device), w.to(device), corr.to(device), 3, 4, 2)
    assert te.cpu().tolist() == [[6, 0, 1]] * T
    with pytest.raises(ValueError):
        hops.moe_router_grouped(h.to(device), w.to(device), corr.to(device), 3, 4, 1)   # 3 of a group of 2
    with pytest.raises(ValueError):
        hops.moe_router_grouped(h.to(device), w.to(device), corr.to(device), 2, 3, 1)   # 8 experts in 3 groups


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,k,d,ff", [(5, 2, 40, 28), (1, 1, 16, 8), (12, 4, 130, 70)])
def test_clamped_experts(device, E, k, d, ff):
    g = torch.Generator().manual_seed(E + d)
    T, limit = 11, 0.8
    h = torch.randn(T, d, generator=g)
    W = {}
    for e in range(E):
        W[f"e{e}.gate"], W[f"e{e}.up"] = torch.randn(ff, d, generator=g) / 3, torch.randn(ff, d, generator=g) / 3
        W[f"e{e}.down"] = torch.randn(d, ff, generator=g) / 3
    te = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    tw = torch.rand(T, k, generator=g)
    want = torch.zeros(T, d, dtype=torch.float64)
    W64 = {n: t.double() for n, t in W.items()}
    for t in range(T):
        for j in range(k):
            want[t] += tw[t, j].double() * plain.expert(h[t:t + 1].double(), W64, f"e{int(te[t, j])}.", limit)[0]
    w_gu = torch.stack([torch.cat([W[f"e{e}.gate"], W[f"e{e}.up"]], 0) for e in range(E)]).to(device)
    w_dn = torch.stack([W[f"e{e}.down"] for e in range(E)]).to(device)
    out = torch.empty(T, d, device=device)
    hops.moe_experts(h.to(device), w_gu, w_dn, tw.to(device), te.to(device), out, act="swish_clamp", limit=limit,
                     alpha=mz.SWISH_ALPHA)
    assert (out.cpu().double() - want).abs().max() < 2e-5 * max(1.0, want.abs().max())
    with pytest.raises(ValueError):
        hops.moe_experts(h.to(device), w_gu, w_dn, tw.to(device), te.to(device), out, act="relu")


@pytest.mark.gpu
def test_clamped_experts_on_the_matrix_cores():
    """bf16 sizes the expert-sorted kernels take, with the clamped activation between the two grouped products."""
    dev = "cuda:0"
    g = torch.Generator().manual_seed(9)
    T, E, k, d, ff, limit = 300, 8, 2, 128, 64, 0.7
    h = torch.randn(T, d, generator=g).to(torch.bfloat16)
    w_gu = (torch.randn(E, 2 * ff, d, generator=g) / 8).to(torch.bfloat16)
    w_dn = (torch.randn(E, d, ff, generator=g) / 8).to(torch.bfloat16)
    te = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    tw = torch.rand(T, k, generator=g)
    assert hops.moe_grouped_ok(h.to(dev), w_gu.to(dev), w_dn.to(dev))
    out = torch.empty(T, d, device=dev)
    hops.moe_experts(h.to(dev), w_gu.to(dev), w_dn.to(dev), tw.to(dev), te.to(dev), out, act="swish_clamp", limit=limit,
                     alpha=mz.SWISH_ALPHA)
    ref = torch.empty(T, d)
    hops.moe_experts(h, w_gu, w_dn, tw, te, ref, act="swish_clamp", limit=limit, alpha=mz.SWISH_ALPHA)
    assert (out.cpu() - ref).abs().max() < 0.03 * ref.abs().max()


@pytest.mark.gpu
@pytest.mark.parametrize("T", [1, 70, 300])
def test_clamped_experts_on_the_streaming_kernel(T):
    """Tiled expert weights: steps of few rows run the grouped weight-streaming kernel with the clamped activation in
    its epilogue."""
    from kafka_llm_service_amd import ops

    dev = "cuda:0"
    g = torch.Generator().manual_seed(T)
    E, k, d, ff, limit = 8, 2, 256, 256, 0.6
    h = torch.randn(T, d, generator=g).to(torch.bfloat16)
    w_gu = (torch.randn(E, 2 * ff, d, generator=g) / 8).to(torch.bfloat16)
    w_dn = (torch.randn(E, d, ff, generator=g) / 8).to(torch.bfloat16)
    te = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    tw = torch.rand(T, k, generator=g)
    assert ops.stream_moe_supported(2 * ff, d) and ops.stream_moe_supported(d, ff)
    gu_t, dn_t = ops.tile_experts(w_gu.to(dev), glu=True), ops.tile_experts(w_dn.to(dev))
    out = torch.empty(T, d, device=dev)
    hops.moe_experts(h.to(dev), w_gu.to(dev), w_dn.to(dev), tw.to(dev), te.to(dev), out, gu_t, dn_t, act="swish_clamp",
                     limit=limit, alpha=mz.SWISH_ALPHA)
    ref = torch.empty(T, d)
    hops.moe_experts(h, w_gu, w_dn, tw, te, ref, act="swish_clamp", limit=limit, alpha=mz.SWISH_ALPHA)
    assert (out.cpu() - ref).abs().max() < 0.03 * ref.abs().max()


# ---- the model in the engine ---------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompt_and_layers(bench_a, device, dtype):
    t = toks(75, 211, 1)
    eng = bench_a.engine(device, dtype)
    lo = []
    got = eng.feed([("a", t, list(range(75)))], ["a"], layers_out=lo)
    if dtype == "float32":
        want_l = []
        plain.forward(bench_a.cfg, bench_a.W, t, layers_out=want_l)
        assert len(lo) == len(want_l) == 5
        for i, (a, b) in enumerate(zip(lo, want_l)):
            assert (a.cpu().double() - b).abs().max() < 1e-4 * b.abs().max(), i
        assert rel_err(got, bench_a.oracle(t)) < TOL[dtype]
    else:
        assert mean_err(got, bench_a.oracle(t)) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("make", [cfg_b, cfg_s1])
def test_other_sizes_and_ones(device, make):
    b = Bench(make(), seed=5)
    t = toks(41, 97, 2)
    eng = b.engine(device)
    assert rel_err(feed_all(eng, "a", t, [41]), b.oracle(t)) < TOL["float32"]
    assert rel_err(feed_all(eng, "b", t, [7, 1, 2]), b.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_models_of_one_layer_kind(device):
    for layer in (cfg_a()["layers"][0], cfg_a()["layers"][1]):
        c = cfg_a()
        c["layers"] = [copy.deepcopy(layer), copy.deepcopy(layer)]
        b = Bench(c, seed=6)
        t = toks(50, 211, 3)
        assert rel_err(feed_all(b.engine(device), "a", t, [30, 1, 19]), b.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2], [16], [17, 15, 1, 2], [31, 1, 1, 1, 33], [64, 2]])
def test_portions_and_decoding(bench_sharp, device, cuts):
    """Prompts cut into portions of every size down to two tokens and single decoded tokens, with a peaky softmax
    (single keys carry the result): every cut lands inside pages and windows somewhere along 90 tokens."""
    t = toks(90, 211, 7)
    eng = bench_sharp.engine(device)
    assert rel_err(feed_all(eng, "a", t, cuts), bench_sharp.oracle(t)) < TOL["float32"]
    assert eng.kvm.num_free() == eng.num_blocks


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_and_reuse(bench_a, bench_sharp, device, dtype):
    """Four unequal requests through two slots and ten pages: portions beside single tokens, a request left out of a
    step, pages and slots freed and used again by later requests; every request against itself alone."""
    b = bench_sharp if dtype == "float32" else bench_a
    eng = b.engine(device, dtype, blocks=10, seqs=2)
    A, B, C, D = toks(70, 211, 11), toks(33, 211, 12), toks(50, 211, 13), toks(17, 211, 14)
    got = {k: [] for k in "ABCD"}

    def step(entries, end=()):
        out = eng.feed([(k, tk, list(range(len(tk)))) for k, tk in entries], list(end))
        r = 0
        for k, tk in entries:
            got[k].append(out[r:r + len(tk)])
            r += len(tk)

    step([("A", A[:30]), ("B", B[:2])])
    step([("B", B[2:3]), ("A", A[30:47])])
    step([("A", A[47:48])])
    step([("A", A[48:49]), ("B", B[3:33])], end=["B"])
    step([("C", C[:40]), ("A", A[49:50])])          # C takes B's slot and pages
    step([("A", A[50:70]), ("C", C[40:41])], end=["A"])
    step([("D", D[:16]), ("C", C[41:50])], end=["C"])
    step([("D", D[16:])], end=["D"])
    assert eng.kvm.num_free() == 10 and eng.slots.num_free() == 2
    for k, tk in (("A", A), ("B", B), ("C", C), ("D", D)):
        g = torch.cat(got[k])
        if dtype == "float32":
            assert rel_err(g, b.oracle(tk)) < TOL["float32"], k
        else:
            assert mean_err(g, b.oracle(tk)) < TOL["bfloat16"], k
            alone = feed_all(b.engine(device, dtype), "x", tk, [len(tk)])
            assert rel_err(g, alone.cpu()) < 0.05, k


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_over_window_edges(bench_sharp, device):
    """A 40-token prompt and 150 single tokens: every window (10, 16, 21, 37) passes over decoded tokens, and the
    first tokens fall out of them one by one."""
    t = toks(190, 211, 21)
    eng = bench_sharp.engine(device)
    assert rel_err(feed_all(eng, "a", t, [40, 1]), bench_sharp.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_long_prompt(bench_sharp, device):
    """300 tokens: keys 18 pages back (the layer without a window sees them all), whole and in portions."""
    t = toks(300, 211, 22)
    eng = bench_sharp.engine(device)
    assert rel_err(feed_all(eng, "a", t, [300]), bench_sharp.oracle(t)) < TOL["float32"]
    assert rel_err(feed_all(eng, "b", t, [129, 2, 100, 1]), bench_sharp.oracle(t)) < TOL["float32"]


@pytest.mark.gpu
def test_preset_sizes_matrix_cores_and_streamed_projections():
    """The smallest preset in bf16 (128-wide heads, latent layers on the matrix-core kernel with their transposed
    latent copy, tiled projections on the weight-streaming kernel for steps of few rows, the expert-sorted kernels):
    single tokens and short portions against the whole prompt, the whole prompt against the oracle on average."""
    from kafka_llm_service_amd.models.config import MOZIDRA_PRESETS

    cfg = copy.deepcopy(MOZIDRA_PRESETS["mozidra-tiny"])
    cfg["vocab"] = 1000
    b = Bench(cfg, seed=2, static_routes=True)
    t = toks(200, 1000, 4)
    eng = b.engine("cuda:0", "bfloat16")
    eng.model.enable_stream_weights()
    assert eng.model.stream and eng.model.attn_tile_tokens and eng.model.pages_t[0] is not None
    assert hasattr(eng.model.layers[0], "w_gu_t")
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

    b = Bench(cfg_a(), seed=8)
    mz.save_checkpoint(b.mc, b.W, tmp_path / "m")
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "mozidra" and mc.num_layers == 5 and mc.vocab_size == 211 and mc.streams == 3
    eng = LLMEngine(EngineConfig(model=str(tmp_path / "m"), weights=str(tmp_path / "m"), device="cpu",
                                 num_kv_blocks=8, max_num_seqs=2, max_model_len=128, dtype="float32"))
    t = toks(20, 211, 9)
    assert rel_err(feed_all(eng, "x", t, [20]), b.oracle(t)) < TOL["float32"]
    bad = copy.deepcopy(b.W)
    bad["l0.mix.q"] = bad["l0.mix.q"][:-1]
    with pytest.raises(ValueError):
        mz.MozidraLM(b.mc, "cpu").load_tensors(bad)
    del bad["l0.mix.q"]
    with pytest.raises(KeyError):
        mz.MozidraLM(b.mc, "cpu").load_tensors(bad)
    for spoil in (lambda c: c["layers"][0]["mlp"]["router"].update(top=5),          # 5 of 2 groups of 2
                  lambda c: c["layers"][1]["mixer"].update(kv_heads=4),            # 6 heads over 4
                  lambda c: c["layers"][1]["mixer"]["rot"].update(dims=26),        # beyond the head
                  lambda c: c["layers"][0].update(type="mamba2")):
        c = cfg_a()
        spoil(c)
        with pytest.raises((ValueError, KeyError)):
            mc2 = mz.MozidraConfig.from_dict(c)
            mz.MozidraLM(mc2, "cpu").load_tensors(mz.random_tensors(mc2))
    tiny = get_config("mozidra-tiny")
    assert tiny.arch == "mozidra" and math.isclose(tiny.norm_eps, 1e-6) and tiny.streams == 4


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
    mz.save_checkpoint(b.mc, b.W, tmp_path / "m")
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
