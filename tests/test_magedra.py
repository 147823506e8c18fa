"""Magedra in the serving engine against the plain whole-sequence implementation of tests/magedra_plain.py.

Small configurations of odd sizes (nothing a multiple of 64, head sizes that differ between keys and values and
between layers, a layer without feed-forward, layers that run another layer's tensors, a model without streams) with
random weights made here. Each test runs on the CPU reference ops and, marked ``gpu``, on the HIP kernels.
"""
import copy
import math

import pytest
import torch

import magedra_plain as plain
from kafka_llm_service_amd.engine.engine import EngineConfig, LLMEngine
from kafka_llm_service_amd.engine.sequence import SamplingParams
from kafka_llm_service_amd.models import magedra as mg
from kafka_llm_service_amd.models.budurax import rotary_table
from kafka_llm_service_amd.ops import hybrid as hops

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def _lat(heads=5, dim=12, rot_dim=6, vdim=18, rank=40, q_rank=28, base=9000.0, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "q_rank": q_rank,
            "rot": {"base": base, "dims": rot_dim}, "scale": scale or (dim + rot_dim) ** -0.5}


def _par(heads=6, kv_heads=2, dim=24, vdim=20, rot=10, base=50000.0, rh=3, rd=10, rv=14, ls=0.7, rs=0.6, scale=None):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale or dim ** -0.5}
    if rot:
        left["rot"] = {"base": base, "dims": rot}
    return {"left": left, "right": {"heads": rh, "dim": rd, "vdim": rv}, "left_scale": ls, "right_scale": rs}


def _ff(ff=52, limit=0.9):
    return {"kind": "dense", "ff": ff, "limit": limit}


def cfg_a(scale=None):
    layers = [{"type": "mingru", "mixer": {"width": 70}, "mlp": _ff()},
              {"type": "parallel", "mixer": _par(scale=scale), "mlp": _ff(36, 2.0)},
              {"type": "latent_attention", "mixer": _lat(scale=scale), "mlp": None},
              {"type": "parallel", "mixer": _par(4, 4, 10, 7, rot=0, rh=1, rd=33, rv=70, ls=1.2, rs=0.3, scale=scale),
               "mlp": _ff(20, 5.0)},
              {"type": "latent_attention", "mixer": _lat(3, 20, 16, 9, 33, 50, base=100.0, scale=scale), "mlp": _ff()}]
    layers += [dict(copy.deepcopy(layers[1]), weights_of=1), dict(copy.deepcopy(layers[0]), weights_of=0),
               dict(copy.deepcopy(layers[4]), weights_of=4)]
    return {"architecture": "Magedra", "vocab": 211, "width": 88, "norm": {"eps": 2e-5}, "streams": 3,
            "residual_mult": 0.4, "logit_scale": 0.3, "layers": layers}


def cfg_b():
    """Ones and equal values: no streams, no residual multiplier and no logit scale in the file, one head, as many
    key/value heads as query heads, a full rotation, key and value sizes equal, a recurrence as wide as the model, a
    rotated part of two dimensions."""
    return {"architecture": "Magedra", "vocab": 97, "width": 48, "norm": {"eps": 1e-6},
            "layers": [{"type": "parallel", "mixer": _par(1, 1, 16, 16, rot=16, rh=1, rd=16, rv=16, ls=1.0, rs=1.0),
                        "mlp": _ff(48, 1.0)},
                       {"type": "mingru", "mixer": {"width": 48}, "mlp": None},
                       {"type": "latent_attention", "mixer": _lat(1, 16, 2, 16, 16, 16), "mlp": _ff(8, 100.0)},
                       {"type": "parallel", "mixer": _par(3, 3, 8, 8, rot=2, rh=2, rd=8, rv=8), "mlp": None}]}


def cfg_s1():
    """One stream given as such (the stream tensors exist, with one entry each)."""
    c = cfg_b()
    c["streams"] = 1
    c["residual_mult"] = 1.5
    return c


class Bench:
    """A config, its random weights and engines over them."""

    def __init__(self, cfg: dict, seed=0, sharpen=1.0):
        self.cfg = cfg
        self.mc = mg.MagedraConfig.from_dict(cfg, name="test")
        self.W = mg.random_tensors(self.mc, seed)
        for k in self.W:
            if sharpen != 1.0 and (k.endswith("left.q") or k.endswith("mix.uq")):
                # scores far from zero: single keys carry the result
                self.W[k] = (self.W[k].float() * sharpen).to(torch.bfloat16)
        self._oracle = {}

    def engine(self, device, dtype="float32", blocks=64, seqs=4, **kw):
        model = mg.MagedraLM(self.mc, device, dtype=getattr(torch, dtype), max_positions=1024).load_tensors(self.W)
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


def poison_state(eng):
    """NaN in every state slot: a sequence's first portion must not read its slot."""
    for st in eng.runner.v_caches.layers:
        for t in st.values():
            t.fill_(float("nan"))


@pytest.fixture(scope="module")
def bench_a():
    return Bench(cfg_a())


@pytest.fixture(scope="module")
def bench_sharp():
    return Bench(cfg_a(scale=0.9), seed=3, sharpen=3.0)


def close(got, want, tol):
    return (got.double().cpu() - want.double()).abs().max().item() < tol * want.abs().max().item()


def seg_tensors(device, runs):
    """runs: (first row, rows, first position, slot) -> (tok_seg, seg)"""
    ts = [j for j, r in enumerate(runs) for _ in range(r[1])]
    return (torch.tensor(ts, dtype=torch.int32, device=device), torch.tensor(runs, dtype=torch.int32, device=device))


# ---- mechanisms alone ------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("S,d", [(3, 70), (1, 33), (4, 4500), (8, 2300)])
def test_stream_step_with_layer_norm(device, S, d):
    """The stream step whose read goes through a layer norm (weight, no bias): a mean far from zero, rows wider than
    the kernel keeps in registers, with and without a write in the same pass."""
    g = torch.Generator().manual_seed(S * 1000 + d)
    T, eps = 5, 1e-4
    xs0 = torch.randn(S, T, d, generator=g) + 3.0
    a, M, b = torch.randn(S, generator=g), torch.eye(S) + 0.3 * torch.randn(S, S, generator=g), torch.randn(S, generator=g)
    y, nw = torch.randn(T, d, generator=g), 1.0 + 0.2 * torch.randn(d, generator=g)
    dv = lambda t: t.to(device)  # noqa: E731
    want = plain.layer_norm(torch.einsum("s,std->td", a.double(), xs0.double()), nw.double(), eps)
    h = torch.empty(T, d, device=device)
    xs = dv(xs0.clone())
    hops.stream_step(xs, read=dv(a), norm_w=dv(nw), eps=eps, out=h, center=True)
    assert torch.equal(xs.cpu(), xs0) and close(h, want, 2e-5)
    new = torch.einsum("sr,std->rtd", M.double(), xs0.double()) + b.double()[:, None, None] * y.double()[None]
    want = plain.layer_norm(torch.einsum("s,std->td", a.double(), new), nw.double(), eps)
    for out_dt, tol in ((torch.float32, 2e-5), (torch.bfloat16, 1e-2)):
        xs, h = dv(xs0.clone()), torch.empty(T, d, dtype=out_dt, device=device)
        total = torch.empty(T, d, device=device)
        hops.stream_step(xs, dv(y), dv(M), dv(b), dv(a), dv(nw), eps, h, total=total, center=True)
        assert close(xs, new, 1e-5) and close(total, new.sum(0), 1e-5) and close(h.float(), want, tol)


@pytest.mark.parametrize("device", DEVICES)
def test_row_ops(device):
    """Norm over a column range of activation rows (both kinds), the scaled sigmoid gate into a column slice, the
    per-head norm without a gate and with a scale."""
    g = torch.Generator().manual_seed(4)
    T = 7
    x, w = torch.randn(T, 150, generator=g) + 1.0, 1.0 + 0.2 * torch.randn(93, generator=g)
    for center, fn in ((False, plain.rms_norm), (True, plain.layer_norm)):
        out = torch.empty(T, 93, device=device)
        hops.act_norm(x.to(device), 11, 93, w.to(device), 1e-5, out, center)
        assert close(out, fn(x[:, 11:104].double(), w.double(), 1e-5), 1e-5)
    a, gate = torch.randn(T, 40, generator=g), torch.randn(T, 90, generator=g)
    both = torch.zeros(T, 100, device=device)
    hops.gate_mul(a.to(device), gate.to(device), 13, 0.7, both[:, :40])
    assert close(both[:, :40], a.double() * torch.sigmoid(gate[:, 13:53].double()) * 0.7, 1e-5)
    assert float(both[:, 40:].abs().max()) == 0.0
    o, hw = torch.randn(T, 3 * 20, generator=g), 1.0 + 0.1 * torch.randn(20, generator=g)
    hops.head_norm_gate(o.to(device), hw.repeat(3).to(device), None, 0, 3, 1e-5, both[:, 40:], 0.3)
    want = plain.rms_norm(o.double().view(T, 3, 20), hw.double(), 1e-5).reshape(T, 60) * 0.3
    assert close(both[:, 40:], want, 1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("n,off", [(64, 16), (4096, 8), (40, 13), (72, 0)])
def test_row_ops_bf16_vectors(n, off):
    """The bf16 forms of the gate and of the clamped activation: sizes and offsets that take 8-element vectors and
    ones that do not, outputs into column slices."""
    dev = "cuda:0"
    g = torch.Generator().manual_seed(n)
    T = 9
    a = torch.randn(T, n, generator=g).to(torch.bfloat16)
    gate = torch.randn(T, off + n + 8, generator=g).to(torch.bfloat16)
    both = torch.zeros(T, n + 16, dtype=torch.bfloat16, device=dev)
    hops.gate_mul(a.to(dev), gate.to(dev), off, 0.7, both[:, :n])
    want = a.double() * torch.sigmoid(gate[:, off:off + n].double()) * 0.7
    assert close(both[:, :n].float(), want, 1e-2) and float(both[:, n:].abs().max()) == 0.0
    gu = (2.0 * torch.randn(T, 2 * n, generator=g)).to(torch.bfloat16)
    hops.swish_clamp_mul(gu.to(dev), 1.3, 1.702, both[:, 8:8 + n])
    gg, uu = gu[:, :n].double().clamp(max=1.3), gu[:, n:].double().clamp(-1.3, 1.3)
    assert close(both[:, 8:8 + n].float(), gg * torch.sigmoid(1.702 * gg) * (uu + 1.0), 1e-2)


PORTIONS = [[(0, 9), (1, 2)], [(1, 1), (0, 1)], [(0, 2), (1, 3)], [(1, 7)], [(0, 130), (1, 65)], [(0, 1)], [(1, 201), (0, 3)]]


def _run_portions(device, lengths, fn):
    """Two sequences through PORTIONS; fn(runs of (sequence, first position, rows), tok_seg, seg) -> rows."""
    at, got = [0, 0], [[], []]
    for portions in PORTIONS:
        runs, r0 = [], 0
        for s, n in portions:
            n = min(n, lengths[s] - at[s])
            runs.append((s, at[s], n, r0))
            r0 += n
        ts, seg = seg_tensors(device, [(r0_, n, p0, 2 - s) for s, p0, n, r0_ in runs])   # slots 2 and 1 of 3
        out = fn([(s, p0, n) for s, p0, n, _ in runs], ts, seg)
        for s, p0, n, r0_ in runs:
            got[s].append(out[r0_:r0_ + n].cpu())
            at[s] += n
    assert at == lengths
    return [torch.cat(x) for x in got]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("Wd", [70, 1, 300])
def test_mingru_scan(device, Wd):
    """The recurrence through portions of 1, 2, 3, 7, 9 rows and long ones (the chunked form on the GPU) from NaN
    slots, two sequences side by side; candidates on both sides of zero; an update gate close to 0 keeps a far token."""
    g = torch.Generator().manual_seed(Wd)
    d, lengths = 20, [146, 279]
    W = {"z": torch.randn(Wd, d, generator=g), "z.b": torch.randn(Wd, generator=g) - 2.0,
         "x": torch.randn(Wd, d, generator=g), "x.b": torch.randn(Wd, generator=g),
         "g": torch.randn(Wd, d, generator=g), "o": torch.eye(Wd)}
    hs = [torch.randn(n, d, generator=g) for n in lengths]
    hs[0][3] *= 10.0     # a loud early token whose trace must survive a hundred gated steps
    want = [plain.mingru(h.double(), {k: v.double() for k, v in W.items()}, "") for h in hs]
    w_in = torch.cat([W["z"], W["x"], W["g"]], 0)
    bias = torch.cat([W["z.b"], W["x.b"]]).to(device)
    state = torch.full((3, Wd), float("nan"), device=device)

    def step(runs, ts, seg):
        proj = torch.cat([hs[s][p0:p0 + n] for s, p0, n in runs]).double() @ w_in.double().T
        proj = torch.cat([proj.float(), torch.zeros(proj.shape[0], 5)], 1).to(device)[:, :3 * Wd + 5]
        out = torch.empty(proj.shape[0], Wd, device=device)
        hops.mingru_scan(proj, bias, Wd, ts, seg, state, out, max(n for _, _, n in runs))
        return out

    got = _run_portions(device, lengths, step)
    for s in (0, 1):
        assert close(got[s], want[s], 2e-5), s
    assert not torch.isnan(state[1:]).any() and torch.isnan(state[0]).all()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,D,Dv", [(3, 10, 14), (1, 64, 64), (2, 100, 130), (4, 48, 65), (1, 1, 1), (2, 200, 8)])
def test_hgrn2_scan_and_head_norm(device, H, D, Dv):
    """The matrix recurrence through portions from NaN slots, then the per-head RMS norm with one weight vector for
    all heads; lower bounds near one keep what a far token wrote."""
    g = torch.Generator().manual_seed(H * 100 + D)
    d, lengths, eps = 24, [146, 279], 1e-5
    W = {"q": torch.randn(H * D, d, generator=g) / 3, "f": torch.randn(H * D, d, generator=g) / 3,
         "f.b": torch.randn(H * D, generator=g), "lower": torch.rand(H * D, generator=g) * 0.98,
         "v": torch.randn(H * Dv, d, generator=g) / 3, "norm": 1.0 + 0.2 * torch.randn(Dv, generator=g),
         "o": torch.eye(H * Dv)}
    hs = [torch.randn(n, d, generator=g) for n in lengths]
    hs[1][5] *= 8.0
    m = {"heads": H, "dim": D, "vdim": Dv}
    want = [plain.hgrn2(h.double(), {k: v.double() for k, v in W.items()}, "", m, eps) for h in hs]
    w_in = torch.cat([W["v"], W["q"], W["f"]], 0)    # (columns in another order than the model's)
    S = torch.full((3, H, D, Dv), float("nan"), device=device)

    def step(runs, ts, seg):
        proj = (torch.cat([hs[s][p0:p0 + n] for s, p0, n in runs]).double() @ w_in.double().T).float().to(device)
        o = torch.empty(proj.shape[0], H * Dv, device=device)
        hops.hgrn2_scan(proj, H * Dv, H * Dv + H * D, 0, W["f.b"].to(device), W["lower"].to(device), H, D, Dv, ts, seg,
                        S, o)
        out = torch.empty_like(o)
        hops.head_norm_gate(o, W["norm"].repeat(H).to(device), None, 0, H, eps, out)
        return out

    got = _run_portions(device, lengths, step)
    for s in (0, 1):
        assert close(got[s], want[s], 5e-5), s


@pytest.mark.gpu
@pytest.mark.parametrize("H,D,Dv", [(3, 10, 14), (2, 64, 128), (1, 200, 70)])
def test_hgrn2_scan_in_chunks(H, D, Dv):
    """The chunk-parallel form (every chunk from zero, entry states carried in order, every chunk again) against the
    token-by-token kernel and the plain function: two long segments, one of them continuing from a state."""
    import numpy as np

    dev = "cuda:0"
    g = torch.Generator().manual_seed(D)
    d, eps, n0, n1 = 24, 1e-5, 700, 513
    W = {"q": torch.randn(H * D, d, generator=g) / 3, "f": torch.randn(H * D, d, generator=g) / 3,
         "f.b": torch.randn(H * D, generator=g) + 2.0, "lower": torch.rand(H * D, generator=g) * 0.98,
         "v": torch.randn(H * Dv, d, generator=g) / 3, "norm": torch.ones(Dv), "o": torch.eye(H * Dv)}
    hs = [torch.randn(n0 + 40, d, generator=g), torch.randn(n1, d, generator=g)]
    m = {"heads": H, "dim": D, "vdim": Dv}
    want = [plain.hgrn2(h.double(), {k: v.double() for k, v in W.items()}, "", m, eps) for h in hs]
    w_in = torch.cat([W["q"], W["f"], W["v"]], 0)
    outs = []
    for chunked in (False, True):
        S = torch.full((2, H, D, Dv), float("nan"), device=dev)
        got = [[], []]
        for runs in ([(0, 0, 40)], [(0, 40, n0), (1, 0, n1)]):
            rows = [(r0, n, p0, s) for (s, p0, n), r0 in zip(runs, np.cumsum([0] + [r[2] for r in runs])[:-1].tolist())]
            ts, seg = seg_tensors(dev, rows)
            proj = (torch.cat([hs[s][p0:p0 + n] for s, p0, n in runs]).double() @ w_in.double().T).float().to(dev)
            o = torch.empty(proj.shape[0], H * Dv, device=dev)
            args = (proj, 0, H * D, 2 * H * D, W["f.b"].to(dev), W["lower"].to(dev), H, D, Dv)
            plan = hops.scan_chunks(np.asarray(rows, dtype=np.int32), H) if chunked else None
            if plan is not None:
                plan = tuple(torch.from_numpy(x).to(dev) for x in plan[:3]) + (plan[3],)
                hops.hgrn2_scan_chunked(*args, plan, S, o)
            else:
                assert not chunked or len(runs) == 1
                hops.hgrn2_scan(*args, ts, seg, S, o)
            out = torch.empty_like(o)
            hops.head_norm_gate(o, W["norm"].repeat(H).to(dev), None, 0, H, eps, out)
            for (s, p0, n), (r0, _, _, _) in zip(runs, rows):
                got[s].append(out[r0:r0 + n].cpu())
        outs.append(([torch.cat(x) for x in got], S.cpu()))
    for s in (0, 1):
        assert close(outs[1][0][s], want[s], 5e-5), s
        assert close(outs[1][0][s], outs[0][0][s], 5e-5), s
    assert close(outs[1][1], outs[0][1], 5e-5)


class Paged:
    """Scattered pages for sequences of given lengths, fed in given portions: the step tensors the kernels take."""

    def __init__(self, device, lengths, seed=0):
        self.device = device
        self.n_pages = sum(-(-n // 16) for n in lengths) + 3
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


def _talk_case(g, n, H, G, D, Dv, rot, spots, gain=3.0):
    """Rows [q | k | v | gate] of a sequence with loud (row, key) pairs, the head mix, and the plain result (the
    projections are selections of the row's columns, the output projection is the identity)."""
    C = H * D + G * D + G * Dv + H * Dv
    h = torch.randn(n, C, generator=g)
    h[:, :H * D] *= 0.5
    talk = torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)
    for i, (at, key) in enumerate(spots):
        hd = i % H
        kk = torch.randn(D, generator=g) * gain
        c = H * D + (hd // (H // G)) * D
        h[key, c:c + D] = kk
        h[at, hd * D:(hd + 1) * D] = kk * 1.5
    eye = torch.eye(C, dtype=torch.float64)
    a, b, c = H * D, H * D + G * D, H * D + G * D + G * Dv
    W = {"q": eye[:a], "k": eye[a:b], "v": eye[b:c], "g": eye[c:], "talk": talk.double(), "o": torch.eye(H * Dv).double()}
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": D ** -0.5}
    if rot:
        m["rot"] = {"dims": rot, "base": 777.0}
    return h, talk, m, W


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv,rot", [(6, 2, 24, 20, 10), (4, 4, 8, 70, 0), (3, 1, 100, 9, 100), (1, 1, 8, 8, 8),
                                          (8, 2, 16, 130, 6)])
def test_head_mixed_attention_single_keys(device, H, G, D, Dv, rot):
    """Rotation (halves layout, part of a head), the head mix folded into the queries, the paged store, the softmax
    over all earlier keys and the scaled output gate, through scattered pages, in portions, two sequences side by
    side. Loud keys sit at the first positions, on both sides of page borders, at the row's own position and hundreds
    of tokens back, for rows of a portion and for rows fed alone."""
    g = torch.Generator().manual_seed(H * 100 + D)
    n0, n1 = 330, 23
    spots = [(329, 0), (329, 329), (140, 127), (140, 128), (100, 15), (100, 16), (297, 1), (297, 2), (298, 40), (5, 0),
             (1, 1), (328, 31)]
    cases = [_talk_case(g, n0, H, G, D, Dv, rot, spots), _talk_case(g, n1, H, G, D, Dv, rot, [(22, 0), (20, 16)])]
    talk = cases[0][1]
    want = []
    for h, _, m, W in cases:
        W = dict(W, talk=talk.double())
        want.append(plain.talking_attention(h.double(), W, "", m) * 0.8)
    pg = Paged(device, [n0, n1], seed=H)
    kc = torch.zeros(pg.n_pages, 16, G * D, device=device)
    vt = torch.zeros(pg.n_pages, G * Dv, 16, device=device)
    cs = rotary_table(512, {"dims": rot, "base": 777.0}, device) if rot else None
    got = [torch.empty(n0, H * Dv), torch.empty(n1, H * Dv)]
    at = [0, 0]
    for portions in ([(0, 97), (1, 2)], [(1, 20), (0, 1)], [(0, 2)], [(0, 197), (1, 1)], [(0, 1)], [(0, 1)], [(0, 31)]):
        runs = [(s, at[s], n) for s, n in portions]
        bt, ts, pos, sl = pg.step(runs)
        rows = torch.cat([cases[s][0][a:a + n] for s, a, n in runs]).to(device)
        qo = torch.empty(rows.shape[0], H * G * D, device=device)
        hops.rope_kv_store(rows, H, G, D, Dv, pos, cs, rot, False, talk.to(device), kc, vt, sl, qo)
        ao = torch.empty(rows.shape[0], H * Dv, device=device)
        hops.window_attn(qo, kc, vt, bt, ts, pos, H, G, D ** -0.5, 0, None, ao, shared_keys=True)
        out = torch.empty_like(ao)
        hops.gate_mul(ao, rows, H * D + G * D + G * Dv, 0.8, out)
        r = 0
        for s, a, n in runs:
            got[s][a:a + n] = out[r:r + n].cpu()
            r += n
            at[s] += n
    assert at == [n0, n1]
    for s in (0, 1):
        assert close(got[s], want[s], 2e-4), s


@pytest.mark.parametrize("device", DEVICES)
def test_rotation_layouts_and_plain_queries(device):
    """rope_kv_store without a head mix: both pairings of the rotation against the plain functions, no rotation."""
    g = torch.Generator().manual_seed(9)
    n, H, G, D, Dv = 37, 4, 2, 12, 5
    rows = torch.randn(n, H * D + G * D + G * Dv + 3, generator=g)
    pg = Paged(device, [n])
    bt, ts, pos, sl = pg.step([(0, 0, n)])
    q = rows[:, :H * D].double().view(n, H, D)
    k = rows[:, H * D:H * D + G * D].double().view(n, G, D)
    for dims, pairs, fn in ((8, False, plain.rotate_halves), (8, True, plain.rotate_pairs), (12, True, plain.rotate_pairs),
                            (0, False, None)):
        kc, vt = torch.zeros(pg.n_pages, 16, G * D, device=device), torch.zeros(pg.n_pages, G * Dv, 16, device=device)
        cs = rotary_table(64, {"dims": dims, "base": 33.0}, device) if dims else None
        qo = torch.empty(n, H * D, device=device)
        hops.rope_kv_store(rows.to(device), H, G, D, Dv, pos, cs, dims, pairs, None, kc, vt, sl, qo)
        wq, wk = (fn(q, dims, 33.0), fn(k, dims, 33.0)) if dims else (q, k)
        assert close(qo, wq.reshape(n, -1), 1e-5)
        assert close(kc.view(-1, G * D)[sl.cpu() if device == "cpu" else sl], wk.reshape(n, -1), 1e-5)
        v = vt.permute(0, 2, 1).reshape(-1, G * Dv)[sl]
        assert close(v, rows[:, H * D + G * D:H * D + G * D + G * Dv], 1e-6)
    with pytest.raises((ValueError, RuntimeError)):
        hops.rope_kv_store(rows.to(device), H, 3, D, Dv, pos, None, 0, False, None, kc, vt, sl, qo)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,n", [(8, 2, 32, 48, 300), (4, 4, 64, 128, 700), (32, 1, 64, 96, 200),
                                        (6, 3, 80, 96, 150), (16, 2, 128, 128, 1500), (2, 1, 16, 256, 520)])
def test_head_mixed_attention_matrix_cores(H, G, D, Dv, n):
    """The matrix-core attention with shared keys (bf16) against the plain function and the vector kernel: prompt
    portions and decode rows, whole key ranges and split ones, loud keys far back and at page borders."""
    dev = "cuda:0"
    g = torch.Generator().manual_seed(H * D + n)
    spots = [(n - 1, 0), (n - 1, n - 1), (140, 127), (140, 128), (100, 15), (n - 2, 1), (n - 1, n - 41), (n - 40, 3)]
    h, talk, m, W = _talk_case(g, n, H, G, D, Dv, 0, spots, gain=2.0)
    hb = h.to(torch.bfloat16)
    want = plain.talking_attention(hb.double(), dict(W, g=torch.zeros_like(W["g"])), "", m) * 2.0   # sigmoid(0) = 1/2
    pg = Paged(dev, [n], seed=5)
    kc = torch.zeros(pg.n_pages, 16, G * D, dtype=torch.bfloat16, device=dev)
    vt = torch.zeros(pg.n_pages, G * Dv, 16, dtype=torch.bfloat16, device=dev)
    tt = hops.sig_tile_tokens(H, G)
    got = torch.empty(n, H * Dv)
    at = 0
    for rows in (n - 40, 1, 38, 1):
        bt, ts, pos, sl = pg.step([(0, at, rows)])
        qq = torch.empty(rows, H * G * D, dtype=torch.bfloat16, device=dev)
        hops.rope_kv_store(hb[at:at + rows].to(dev), H, G, D, Dv, pos, None, 0, False, talk.to(dev), kc, vt, sl, qq)
        tiles = torch.tensor([(a, min(tt, rows - a), 0, 0) for a in range(0, rows, tt)], dtype=torch.int32, device=dev)
        assert hops.window_attn_mfma_ok(qq, kc, vt, H, G, True)
        outs = []
        for max_keys in (0, at + rows):   # unsplit; split key ranges where the launch has few tiles
            out = torch.empty(rows, H * Dv, dtype=torch.bfloat16, device=dev)
            hops.window_attn(qq, kc, vt, bt, ts, pos, H, G, D ** -0.5, 0, None, out, tiles, max_keys, shared_keys=True)
            outs.append(out.float().cpu())
        vec = torch.empty(rows, H * Dv, dtype=torch.bfloat16, device=dev)
        hops.window_attn(qq, kc, vt, bt, ts, pos, H, G, D ** -0.5, 0, None, vec, shared_keys=True)
        for o in outs:
            assert (o - vec.float().cpu()).abs().max() < 0.03 * want.abs().max()
        got[at:at + rows] = outs[1]
        at += rows
    assert at == n
    assert (got.double() - want).abs().max() < 0.04 * want.abs().max()


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
        assert len(lo) == len(want_l) == 8
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
    for k in (0, 1, 2):
        c = cfg_a(scale=0.9)
        layer = c["layers"][k]
        c["layers"] = [copy.deepcopy(layer), dict(copy.deepcopy(layer), weights_of=0), copy.deepcopy(layer)]
        b = Bench(c, seed=6, sharpen=3.0)
        t = toks(50, 211, 3)
        assert rel_err(feed_all(b.engine(device), "a", t, [30, 1, 19]), b.oracle(t)) < TOL["float32"], k


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2], [16], [17, 15, 1, 2], [31, 1, 1, 1, 33], [64, 2]])
def test_portions_and_decoding(bench_sharp, device, cuts):
    """Prompts cut into portions of every size down to two tokens and single decoded tokens, with a peaky softmax
    (single keys carry the result), from NaN state slots: every cut lands inside pages somewhere along 90 tokens."""
    t = toks(90, 211, 7)
    eng = bench_sharp.engine(device)
    poison_state(eng)
    assert rel_err(feed_all(eng, "a", t, cuts), bench_sharp.oracle(t)) < TOL["float32"]
    assert eng.kvm.num_free() == eng.num_blocks


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_and_reuse(bench_a, bench_sharp, device, dtype):
    """Four unequal requests through two slots and ten pages: portions beside single tokens, a request left out of a
    step, pages and slots freed and used again by later requests; every request against itself alone."""
    b = bench_sharp if dtype == "float32" else bench_a
    eng = b.engine(device, dtype, blocks=10, seqs=2)
    poison_state(eng)
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
def test_long_decoding(bench_sharp, device):
    """A 40-token prompt and 150 single tokens from NaN state: the recurrent states are carried token by token and
    the prompt's keys stay visible."""
    t = toks(190, 211, 21)
    eng = bench_sharp.engine(device)
    poison_state(eng)
    assert rel_err(feed_all(eng, "a", t, [40, 1]), bench_sharp.oracle(t)) < TOL["float32"]


@pytest.mark.parametrize("device", DEVICES)
def test_long_prompt(bench_sharp, device):
    """300 tokens: keys 18 pages back, recurrences in their chunked form on the GPU; whole and in portions."""
    t = toks(300, 211, 22)
    eng = bench_sharp.engine(device)
    assert rel_err(feed_all(eng, "a", t, [300]), bench_sharp.oracle(t)) < TOL["float32"]
    assert rel_err(feed_all(eng, "b", t, [129, 2, 100, 1]), bench_sharp.oracle(t)) < TOL["float32"]


@pytest.mark.gpu
def test_chunked_scans_in_the_engine(bench_sharp):
    """A 700-token prompt beside a short one, then more of both: both recurrences take their chunked forms."""
    t, u = toks(760, 211, 23), toks(30, 211, 24)
    eng = bench_sharp.engine("cuda:0")
    poison_state(eng)
    a = eng.feed([("a", t[:20], list(range(20)))], [])
    b = eng.feed([("a", t[20:720], list(range(700))), ("u", u[:9], list(range(9)))], [])
    c = eng.feed([("u", u[9:], list(range(21))), ("a", t[720:], list(range(40)))], ["a", "u"])
    assert rel_err(torch.cat([a, b[:700], c[21:]]), bench_sharp.oracle(t)) < TOL["float32"]
    assert rel_err(torch.cat([b[700:], c[:21]]), bench_sharp.oracle(u)) < TOL["float32"]


@pytest.mark.gpu
def test_preset_sizes_matrix_cores_and_streamed_projections():
    """The smallest preset in bf16 (latent layers and the head-mixed attention on the matrix-core kernels, tiled
    projections on the weight-streaming kernel for steps of few rows): single tokens and short portions against the
    whole prompt, the whole prompt against the oracle on average."""
    from kafka_llm_service_amd.models.config import MAGEDRA_PRESETS

    cfg = copy.deepcopy(MAGEDRA_PRESETS["magedra-tiny"])
    cfg["vocab"] = 1000
    b = Bench(cfg, seed=2)
    t = toks(200, 1000, 4)
    eng = b.engine("cuda:0", "bfloat16")
    eng.model.enable_stream_weights()
    assert eng.model.stream and eng.model.attn_tile_tokens and eng.model.pages_t[0] is not None
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
    mg.save_checkpoint(b.mc, b.W, tmp_path / "m")
    assert not any(k.startswith("l5.") for k in b.W)            # a layer that runs another's tensors owns none
    mc = get_config(str(tmp_path / "m"))
    assert mc.arch == "magedra" and mc.num_layers == 8 and mc.vocab_size == 211 and mc.streams == 3
    assert math.isclose(mc.residual_mult, 0.4) and math.isclose(mc.logit_scale, 0.3)
    eng = LLMEngine(EngineConfig(model=str(tmp_path / "m"), weights=str(tmp_path / "m"), device="cpu",
                                 num_kv_blocks=8, max_num_seqs=2, max_model_len=128, dtype="float32"))
    t = toks(20, 211, 9)
    assert rel_err(feed_all(eng, "x", t, [20]), b.oracle(t)) < TOL["float32"]
    bad = copy.deepcopy(b.W)
    bad["l1.mix.left.talk"] = bad["l1.mix.left.talk"][:-1]
    with pytest.raises(ValueError):
        mg.MagedraLM(b.mc, "cpu").load_tensors(bad)
    del bad["l1.mix.left.talk"]
    with pytest.raises(KeyError):
        mg.MagedraLM(b.mc, "cpu").load_tensors(bad)
    for spoil in (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=4),          # 6 heads over 4
                  lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=26),      # beyond the head
                  lambda c: c["layers"][2]["mixer"]["rot"].update(dims=8),               # beyond the rotated part
                  lambda c: c["layers"][5].update(weights_of=6),                         # a layer that owns nothing
                  lambda c: c["layers"][6]["mixer"].update(width=71),                    # differs from its source
                  lambda c: c["layers"][0]["mlp"].update(kind="moe"),
                  lambda c: c["layers"][0].update(type="mamba2")):
        c = cfg_a()
        spoil(c)
        with pytest.raises((ValueError, KeyError)):
            mc2 = mg.MagedraConfig.from_dict(c)
            mg.MagedraLM(mc2, "cpu").load_tensors(mg.random_tensors(mc2))
    tiny = get_config("magedra-tiny")
    assert tiny.arch == "magedra" and math.isclose(tiny.norm_eps, 1e-6) and tiny.streams == 2


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
    b = Bench(cfg_s1(), seed=14)
    mg.save_checkpoint(b.mc, b.W, tmp_path / "m")
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
