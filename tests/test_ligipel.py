"""Ligipel through the engine against the plain implementation in
``ligipel_oracle.py``: each mechanism alone, prefill against token-by-token
decoding, portions, mixed batches, reuse of pages and state slots, window
edges and page borders, first tokens, long decoding, other sizes, and greedy
generation through ``submit`` / ``step``.

Every case runs on the CPU (the ops' fp32 forms, the same engine, cache manager
and scheduler) and, marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""
import json
import math

import pytest
import torch
import torch.nn.functional as F

import ligipel_oracle as O
from k8s_llm_rca_amd.engine.engine import EngineConfig, LLMEngine
from k8s_llm_rca_amd.models.ligipel import LigipelConfig, LigipelModel
from k8s_llm_rca_amd.ops import moe as M
from k8s_llm_rca_amd.ops import norm as N
from k8s_llm_rca_amd.ops import seq_ops as S

GPU = pytest.mark.gpu
BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=GPU),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=GPU)]
DT = torch.float64


def tol(dtype):
    return 3e-5 if dtype == torch.float32 else 4e-2


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)).max())


def row_errs(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)


def agrees(got, want, dtype, mult=1.0):
    """Logits rows against the oracle's.  fp32: every row.  bf16: rounding may flip a close router
    choice at a few positions, so a few rows may be off (never by much); the rest must be close."""
    e = row_errs(got, want)
    if dtype == torch.float32:
        return float(e.max()) < 3e-5 * mult
    return int((e > 4e-2 * mult).sum()) <= max(1, 0.03 * e.numel()) and float(e.max()) < 0.5 and float(e.median()) < 2e-2 * mult


def close(got, want, dtype, scale=1.0):
    """Element-wise check of an op's output against fp64."""
    got, want = got.double().cpu(), want.double().cpu()
    t = (2e-5 if dtype == torch.float32 else 2e-2) * scale
    err = float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))
    assert err < t, err


# ------------------------------------------------------------------ configurations and weights
def left(heads=4, kv_heads=2, dim=8, vdim=12, window=16, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
            "scale": 1.0 / math.sqrt(dim) if scale is None else scale}


def right(inner=40, state=6, dt_rank=5, conv=3):
    return {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}


def parallel(l=None, r=None):
    return {"type": "parallel", "mixer": {"left": l or left(), "right": r or right()}}


def ret(heads=3, dim=8, vdim=12, decay=None, rot_dims=None, base=10000.0):
    return {"type": "retention",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim,
                      "decay": decay or [1.0 - 2.0 ** (-2 - h) for h in range(heads)],
                      "rot": {"dims": dim if rot_dims is None else rot_dims, "base": base}}}


def moe(experts=5, top=2, ff=24, shared=16):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def config(layers, width=48, vocab=512, eps=1e-5, logit_scale=0.7, softcap=20.0):
    ls = [dict(mix, mlp=mlp) for mix, mlp in layers]
    return {"architecture": "Ligipel", "vocab": vocab, "width": width, "layers": ls, "norm": {"eps": eps},
            "logit_scale": logit_scale, "logit_softcap": softcap}


def default_config(**kw):
    return config([(parallel(), moe()), (ret(), moe(experts=3, top=1, shared=0)),
                   (parallel(left(heads=3, kv_heads=3, dim=4, vdim=4, window=7), right(24, 3, 2, 2)), None),
                   (ret(heads=2, dim=12, vdim=4, rot_dims=6), moe(4, 4, 8, 8))], **kw)


def weights(d, seed=0, big=1.0):
    """Random weights under the checkpoint's names, rounded to bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W = d["width"]

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    def lin(o, i, mul=1.0):
        return r(o, i, std=mul * i ** -0.5)

    t = {"embed": r(d["vocab"], W), "head": lin(d["vocab"], W)}

    def norm(name):
        t[name], t[name + ".b"] = r(W, std=0.2, mean=1.0), r(W, std=0.1)

    norm("embed.norm")
    norm("final.norm")
    for i, L in enumerate(d["layers"]):
        p = f"l{i}."
        norm(p + "norm1")
        norm(p + "norm1b")
        m = L["mixer"]
        if L["type"] == "parallel":
            a, b = m["left"], m["right"]
            q = p + "mix.left."
            t[q + "q"], t[q + "k"] = lin(a["heads"] * a["dim"], W, big), lin(a["kv_heads"] * a["dim"], W, big)
            t[q + "v"], t[q + "o"] = lin(a["kv_heads"] * a["vdim"], W), lin(W, a["heads"] * a["vdim"])
            t[q + "r1"], t[q + "r2"] = r(a["heads"], std=0.3, mean=0.5), r(a["heads"], std=0.2, mean=0.8).abs()
            t[q + "talk"] = (torch.eye(a["heads"]) + r(a["heads"], a["heads"], std=0.3)).to(torch.bfloat16).float()
            t[q + "out"] = r(W, std=0.2, mean=1.0)
            s = p + "mix.right."
            C, Ns, R = b["inner"], b["state"], b["dt_rank"]
            t[s + "in"] = lin(2 * C, W)
            t[s + "conv"], t[s + "conv.b"] = r(C, b["conv"], std=0.5), r(C, std=0.2)
            t[s + "x"] = lin(R + 2 * Ns, C)
            t[s + "dt"], t[s + "dt.b"] = lin(C, R), r(C, std=0.5, mean=-1.0)
            t[s + "A_log"] = r(C, Ns, std=0.5)
            t[s + "D"] = r(C, std=0.3, mean=1.0)
            t[s + "o"] = lin(W, C)
            t[s + "out"] = r(W, std=0.2, mean=1.0)
        else:
            s = p + "mix."
            H, D, V = m["heads"], m["dim"], m["vdim"]
            t[s + "q"], t[s + "k"] = lin(H * D, W), lin(H * D, W)
            t[s + "v"], t[s + "g"], t[s + "o"] = lin(H * V, W), lin(H * V, W), lin(W, H * V)
        f = L["mlp"]
        if f is not None:
            norm(p + "norm2")
            norm(p + "norm2b")
            E = f["router"]["experts"]
            t[p + "mlp.router"] = lin(E, W, 2.0)
            t[p + "mlp.correction"] = r(E, std=0.2)
            for e in [f"e{e}" for e in range(E)] + (["shared"] if f.get("shared") else []):
                ff = f["shared"]["ff"] if e == "shared" else f["expert"]["ff"]
                t[p + f"mlp.{e}.gate"], t[p + f"mlp.{e}.up"] = lin(ff, W), lin(ff, W)
                t[p + f"mlp.{e}.down"] = lin(W, ff)
        t[p + "dwa"] = r(i + 2, std=0.3, mean=0.4)
    return t


def engine(d, W, backend, num_blocks=24, block_size=32, slots=4, **kw):
    dev, dt = backend
    model = LigipelModel(LigipelConfig.from_json(d, "test"), dev, dt, init=False)
    model.load_tensors(W.__getitem__)
    cfg = dict(model="test", device=dev, dtype=dt, num_blocks=num_blocks, block_size=block_size, state_slots=slots,
               max_batch_tokens=1024, use_graphs=False, temperature=0.0)
    cfg.update(kw)
    eng = LLMEngine(EngineConfig(**cfg), model=model)
    for t in eng.states.t.values():       # a fresh slot must not be read: make a read loud
        t.fill_(float("nan"))
    for c in eng.kv.kc + eng.kv.vc + [t for t in eng.kv.vt if t is not None]:
        c.fill_(3e4)                      # stale pages hold finite garbage (a masked key multiplies it by 0)
    return eng


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def feed_all(eng, sid, tokens, cuts):
    """Feed ``tokens`` in portions ``cuts`` (the rest one by one); logits of every position."""
    out, at = [], 0
    for n in list(cuts) + [1] * len(tokens):
        if at >= len(tokens):
            break
        n = min(n, len(tokens) - at)
        out.append(eng.feed([(sid, tokens[at:at + n], list(range(n)))]))
        at += n
    return torch.cat(out)


def seg_meta(lens, pos0, slots, dev, block_tables=None):
    row0 = [0]
    for n in lens:
        row0.append(row0[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)  # noqa: E731
    row_seg = [s for s, n in enumerate(lens) for _ in range(n)]
    bt = i32(block_tables if block_tables is not None else [[0]] * len(lens))
    return S.SegMeta(len(lens), i32(row_seg), i32(row0), i32(pos0), i32(slots), bt, row0, list(pos0), list(slots),
                     n_single=0)


def rnd(*shape, seed=0, std=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=DT) * std


def in_portions(fn, total, cuts):
    """Call ``fn(a, e)`` on consecutive row ranges of sizes ``cuts`` (then the rest) and concatenate."""
    out, at = [], 0
    for n in list(cuts) + [total]:
        if at >= total:
            break
        e = min(total, at + n)
        out.append(fn(at, e))
        at = e
    return torch.cat(out)


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("W", [8, 48, 300, 1024])
def test_layer_norms_and_depth_sum(backend, W):
    dev, dt = backend
    T, eps = 7, 1e-5
    x, y, y2 = rnd(T, W, seed=1) + 3.0, rnd(T, W, seed=2, std=5.0), rnd(T, W, seed=3, std=0.1)
    w, b, nw, nb, wl, wr = (rnd(W, seed=4 + i) for i in range(6))
    f = lambda *ts: [t.float().to(dev) for t in ts]  # noqa: E731
    X, Y, Y2, Wt, B, NW, NB, WL, WR = f(x, y, y2, w, b, nw, nb, wl, wr)
    close(N.layernorm(X, Wt, B, eps, dt), O.layer_norm(x, w, b, eps), dt)
    for merge, u in (("rms", 0.5 * (O.rms(y, eps) * wl + O.rms(y2, eps) * wr)), ("sum", y + y2), (None, y)):
        dst = torch.empty_like(X)
        h = N.ln_residual(X, Y, Wt, B, eps, dst, y2=Y2 if merge else None, merge=merge, mw=(WL, WR), nw=NW, nb=NB,
                          out_dtype=dt)
        want = x + O.layer_norm(u, w, b, eps)
        close(dst, want, torch.float32)
        close(h, O.layer_norm(want, nw, nb, eps), dt)
    xin = X.clone()                                        # in place, no following norm
    assert N.ln_residual(xin, Y, Wt, B, eps, xin) is None
    close(xin, x + O.layer_norm(y, w, b, eps), torch.float32)
    st = rnd(4, T, W, seed=11)
    coef = rnd(4, seed=12)
    St, Cf = f(st, coef)
    a, h = N.depth_mix_ln(St, 3, Cf, Wt, B, eps, dt)
    want = sum(coef[j] * st[j] for j in range(3))
    close(a, want, torch.float32)
    close(h, O.layer_norm(want, w, b, eps), dt)
    rows = torch.tensor([5, 0, 5, 2], device=dev)
    a, h = N.depth_mix_ln(St, 4, Cf, Wt, B, eps, dt, rows=rows)
    want = sum(coef[j] * st[j] for j in range(4))[rows.cpu()]
    close(a, want, torch.float32)
    close(h, O.layer_norm(want, w, b, eps), dt)
    emb = rnd(20, W, seed=13).to(torch.bfloat16)
    ids = torch.tensor([3, 19, 0, 3], dtype=torch.int32, device=dev)
    x0 = torch.empty(4, W, device=dev)
    h = N.embed_layernorm(ids, emb.to(dev).to(dt), Wt, B, eps, x0, NW, NB, out_dtype=dt)
    want = O.layer_norm(emb.double()[ids.cpu().long()], w, b, eps)
    close(x0, want, torch.float32)
    close(h, O.layer_norm(want, nw, nb, eps), dt)
    z = rnd(3, 50, seed=14, std=30.0)
    close(N.softcap_(z.float().to(dev), 0.5, 15.0), 15.0 * torch.tanh(z * 0.5 / 15.0), torch.float32)
    close(N.softcap_(z.float().to(dev), 2.0, 0.0), z * 2.0, torch.float32)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_short_conv_portions_and_tail(backend, taps):
    dev, dt = backend
    C, T = 70, 23
    xw = rnd(T, 2 * C, seed=taps).to(torch.bfloat16).double()       # the convolution reads a column slice
    cw, cb = rnd(C, taps, seed=50), rnd(C, seed=51)
    want = O.causal_conv_silu(xw[:, :C], cw, cb)
    xd = xw.to(dev).to(dt)
    for cuts in [(T,), (1, 1, 1, 5, 2), (2, 3, 1, 9)]:
        tail = torch.full((3, taps - 1, C), float("nan"), device=dev)
        at = [0]

        def run(a, e):
            sg = seg_meta([e - a], [a], [1], dev)
            return S.short_conv(xd[a:e, :C], cw.float().to(dev), cb.float().to(dev), tail, sg)
        close(in_portions(run, T, cuts), want, dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_short_conv_two_sequences_in_one_step(backend):
    dev, dt = backend
    C, taps = 40, 4
    xa, xb = rnd(9, C, seed=1).to(torch.bfloat16).double(), rnd(6, C, seed=2).to(torch.bfloat16).double()
    cw, cb = rnd(C, taps, seed=3), rnd(C, seed=4)
    tail = torch.full((4, taps - 1, C), float("nan"), device=dev)
    f = lambda t: t.to(dev).to(dt)  # noqa: E731
    cwd, cbd = cw.float().to(dev), cb.float().to(dev)
    o1 = S.short_conv(f(torch.cat([xa[:5], xb[:1]])), cwd, cbd, tail, seg_meta([5, 1], [0, 0], [2, 0], dev))
    o2 = S.short_conv(f(torch.cat([xb[1:], xa[5:]])), cwd, cbd, tail, seg_meta([5, 4], [1, 5], [0, 2], dev))
    wa, wb = O.causal_conv_silu(xa, cw, cb), O.causal_conv_silu(xb, cw, cb)
    close(torch.cat([o1[:5], o2[5:]]), wa, dt)
    close(torch.cat([o1[5:], o2[:5]]), wb, dt)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("C,Ns,R", [(40, 6, 5), (130, 16, 8), (24, 24, 3), (16, 1, 1), (32, 40, 2)])
def test_selective_scan_across_portions(backend, C, Ns, R):
    dev, dt = backend
    T = 37
    xc = rnd(T, C, seed=1).to(torch.bfloat16).double()
    z = rnd(T, 2 * C, seed=2).to(torch.bfloat16).double()
    dtp, bias = rnd(T, C, seed=3), rnd(C, seed=4) - 1.0
    dbc = rnd(T, R + 2 * Ns, seed=5)
    A, D = -torch.exp(rnd(C, Ns, seed=6, std=0.5)), rnd(C, seed=7)
    want = O.selective_scan(xc, F.softplus(dtp + bias), A, dbc[:, R:R + Ns], dbc[:, R + Ns:], D) * F.silu(z[:, C:])
    f32 = lambda t: t.float().to(dev)  # noqa: E731
    xd, zd = xc.to(dev).to(dt), z.to(dev).to(dt)
    for cuts in [(T,), (1, 1, 2, 20), (5, 1, 1, 1, 13)]:
        state = torch.full((3, C, Ns), float("nan"), device=dev)

        def run(a, e):
            return S.selective_scan(xd[a:e].contiguous(), f32(dtp[a:e]), f32(bias), f32(dbc[a:e]), R, f32(A), f32(D),
                                    zd[a:e, C:], state, seg_meta([e - a], [a], [2], dev))
        close(in_portions(run, T, cuts), want, dt, scale=4.0)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,D,V,rot", [(3, 8, 12, 8), (2, 12, 4, 6), (1, 4, 4, 0), (4, 32, 64, 32), (2, 64, 128, 16),
                                       (2, 16, 100, 10), (1, 128, 256, 128)])
def test_retention_across_portions_and_slots(backend, H, D, V, rot):
    dev, dt = backend
    T, eps, base = 29, 1e-5, 500.0
    qkvg = rnd(T, 2 * H * (D + V), seed=H + D)
    decay = [1.0 - 2.0 ** (-1 - h) for h in range(H)]
    pos0 = 1000                                             # angles far from zero
    pos = torch.arange(pos0, pos0 + T)
    q = O.rotate(qkvg[:, :H * D].reshape(T, H, D), pos, rot, base, DT)
    k = O.rotate(qkvg[:, H * D:2 * H * D].reshape(T, H, D), pos, rot, base, DT) * D ** -0.5
    v = qkvg[:, 2 * H * D:2 * H * D + H * V].reshape(T, H, V)
    o = O.rms(O.retention_core(q, k, v, decay), eps).reshape(T, H * V) * F.silu(qkvg[:, 2 * H * D + H * V:])
    dec = torch.tensor(decay, dtype=torch.float32, device=dev)
    for cuts in [(T,), (1, 2, 1, 10), (7, 1, 1), (17, 2)]:
        qd = qkvg.float().to(dev)                           # the device kernels rotate q and k in place
        state = torch.full((3, H, D, V), float("nan"), device=dev)
        first = [True]

        def run(a, e):
            # the sequence starts at position pos0 of the rotation but at 0 of its state: a fresh slot is not read
            sg = seg_meta([e - a], [0 if a == 0 else pos0 + a], [1], dev)
            p = torch.arange(pos0 + a, pos0 + e, dtype=torch.int32, device=dev)
            return S.retention(qd[a:e], H, D, V, dec, rot, base, state, sg, p, eps, dt)
        close(in_portions(run, T, cuts), o, dt, scale=4.0)


@pytest.mark.parametrize("backend", BACKENDS)
def test_selective_scan_long_portions_parallel_over_time(backend):
    """Portions long enough for the chunk-parallel kernels, beside a short one in the same step, and a
    sequence that goes on from a long portion token by token."""
    dev, dt = backend
    T, C, Ns, R = 520, 48, 8, 4
    xc = rnd(T, C, seed=1).to(torch.bfloat16).double()
    z = rnd(T, 2 * C, seed=2).to(torch.bfloat16).double()
    dtp, bias = rnd(T, C, seed=3), rnd(C, seed=4) - 1.0
    dbc = rnd(T, R + 2 * Ns, seed=5)
    A, D = -torch.exp(rnd(C, Ns, seed=6, std=0.5)), rnd(C, seed=7)

    def plain(a, e):
        return (O.selective_scan(xc[a:e], F.softplus(dtp[a:e] + bias), A, dbc[a:e, R:R + Ns], dbc[a:e, R + Ns:], D)
                * F.silu(z[a:e, C:]))
    f32 = lambda t: t.float().to(dev)  # noqa: E731
    xd, zd = xc.to(dev).to(dt), z.to(dev).to(dt)
    state = torch.full((3, C, Ns), float("nan"), device=dev)

    def run(a, e, sg):
        return S.selective_scan(xd[a:e].contiguous(), f32(dtp[a:e]), f32(bias), f32(dbc[a:e]), R, f32(A), f32(D),
                                zd[a:e, C:], state, sg)
    # rows 0..299: sequence X; rows 300..519: sequence Y
    o1 = run(0, 200, seg_meta([200], [0], [0], dev))
    oy = run(300, 305, seg_meta([5], [0], [2], dev))
    got_x = torch.cat([o1, run(200, 201, seg_meta([1], [200], [0], dev)),
                       run(201, 300, seg_meta([99], [201], [0], dev))])
    close(got_x, plain(0, 300), dt, scale=4.0)
    # one step with two segments: Y goes on with 215 rows (chunked) beside the first 3 rows of another sequence
    xs = torch.cat([xd[305:520], xd[0:3]]).contiguous()
    both = S.selective_scan(xs, f32(torch.cat([dtp[305:520], dtp[0:3]])), f32(bias),
                            f32(torch.cat([dbc[305:520], dbc[0:3]])), R, f32(A), f32(D),
                            torch.cat([zd[305:520], zd[0:3]])[:, C:], state, seg_meta([215, 3], [5, 0], [2, 1], dev))
    close(torch.cat([oy, both[:215]]), plain(300, 520), dt, scale=4.0)
    close(both[215:], plain(0, 3), dt, scale=4.0)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,D,V", [(2, 8, 12), (3, 32, 64), (2, 64, 128)])
def test_retention_long_portions_parallel_over_time(backend, H, D, V):
    """Portions long enough for the chunk-parallel kernels, then on token by token, beside another sequence."""
    dev, dt = backend
    T, eps, base, rot = 330, 1e-5, 1e4, D
    qkvg = rnd(T, 2 * H * (D + V), seed=H + D)
    decay = [1.0 - 2.0 ** (-4 - h) for h in range(H)]
    pos = torch.arange(T)
    q = O.rotate(qkvg[:, :H * D].reshape(T, H, D), pos, rot, base, DT)
    k = O.rotate(qkvg[:, H * D:2 * H * D].reshape(T, H, D), pos, rot, base, DT) * D ** -0.5
    v = qkvg[:, 2 * H * D:2 * H * D + H * V].reshape(T, H, V)
    want = O.rms(O.retention_core(q, k, v, decay), eps).reshape(T, H * V) * F.silu(qkvg[:, 2 * H * D + H * V:])
    dec = torch.tensor(decay, dtype=torch.float32, device=dev)
    state = torch.full((3, H, D, V), float("nan"), device=dev)

    def run(rows, sg, p):
        return S.retention(qkvg[rows].float().to(dev), H, D, V, dec, rot, base, state, sg,
                           torch.tensor(p, dtype=torch.int32, device=dev), eps, dt)
    # one step: rows 0..199 of the sequence (slot 1) beside rows 0..2 of the same tokens as another one (slot 0)
    rows = list(range(200)) + [0, 1, 2]
    o1 = run(rows, seg_meta([200, 3], [0, 0], [1, 0], dev), list(range(200)) + [0, 1, 2])
    close(o1[200:], want[:3], dt, scale=4.0)
    o2 = run([200], seg_meta([1], [200], [1], dev), [200])
    o3 = run(list(range(201, 330)), seg_meta([129], [201], [1], dev), list(range(201, 330)))
    close(torch.cat([o1[:200], o2, o3]), want, dt, scale=4.0)


def paged(x, block_size, order, dev, dt):
    """Rows of ``x`` [n, w] laid into pages in ``order``; returns (pages [nb, BS, w], block table row)."""
    n, w = x.shape
    nb = max(order) + 1
    pages = torch.full((nb, block_size, w), float("nan"), dtype=dt, device=dev)
    for i in range(-(-n // block_size)):
        part = x[i * block_size:(i + 1) * block_size]
        pages[order[i], :part.shape[0]] = part.to(dev).to(dt)
    return pages, list(order[:-(-n // block_size)])


def run_window(backend, q, k, v, r1, r2, talk, win, scale, cuts, BS=32):
    dev, dt = backend
    T, H, D = q.shape
    G, V = k.shape[1], v.shape[2]
    order = [5, 2, 7, 0, 3, 6, 1, 4, 9, 8]
    kc, row = paged(k.reshape(T, G * D), BS, order, dev, dt)
    vc, _ = paged(v.reshape(T, G * V), BS, order, dev, dt)
    vt = None
    if S.window_mfma_ok(H, G, D, V, dt, dev):                 # the matrix-core kernel: values also transposed
        kc, vc = kc.nan_to_num(nan=3e4), vc.nan_to_num(nan=3e4)   # it reads whole 32-key blocks (masked, finite)
        vt = vc.transpose(1, 2).contiguous()
    f32 = lambda t: t.float().to(dev)  # noqa: E731
    qd = q.reshape(T, H * D).to(dev).to(dt)

    def run(a, e):
        sg = seg_meta([e - a], [a], [0], dev, [row])
        return S.window_attention(qd[a:e], H, G, D, V, kc, vc, f32(r1), f32(r2), f32(talk), win, scale, sg, vt)
    return in_portions(run, T, cuts).reshape(T, H, V)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,V,win", [(4, 2, 8, 12, 16), (3, 3, 4, 4, 7), (6, 1, 16, 8, 40), (1, 1, 8, 8, 1),
                                         (8, 2, 64, 64, 70), (5, 5, 24, 40, 300), (16, 2, 128, 128, 100),
                                         (5, 5, 64, 128, 33), (12, 4, 128, 64, 300), (1, 1, 64, 64, 20),
                                         (4, 4, 64, 64, 1), (9, 3, 64, 64, 32)])
def test_window_attention_paged(backend, H, G, D, V, win):
    T = 150
    b16 = lambda t: t.to(torch.bfloat16).double()  # noqa: E731
    q, k, v = b16(rnd(T, H, D, seed=1)), b16(rnd(T, G, D, seed=2)), b16(rnd(T, G, V, seed=3))
    r1, r2 = rnd(H, seed=4, std=0.3) + 0.5, rnd(H, seed=5).abs()
    talk = torch.eye(H, dtype=DT) + rnd(H, H, seed=6, std=0.3)
    want = O.window_attention_core(q, k, v, r1, r2, talk, win, 0.3)
    for cuts in [(T,), (3, 1, 1, 60, 2)]:
        close(run_window(backend, q, k, v, r1, r2, talk, win, 0.3, cuts), want, backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,G,D,V,win", [(16, 2, 128, 128, 200), (8, 1, 128, 64, 90), (8, 4, 64, 64, 50), (6, 2, 64, 128, 130)])
def test_window_attention_long_portion(backend, H, G, D, V, win):
    """A portion of many tiles (the kernels that do not split the keys over workgroups), then token by
    token (the ones that do)."""
    T = 540
    b16 = lambda t: t.to(torch.bfloat16).double()  # noqa: E731
    q, k, v = b16(rnd(T, H, D, seed=1)), b16(rnd(T, G, D, seed=2)), b16(rnd(T, G, V, seed=3))
    r1, r2 = rnd(H, seed=4, std=0.3) + 0.5, rnd(H, seed=5).abs()
    talk = torch.eye(H, dtype=DT) + rnd(H, H, seed=6, std=0.3)
    want = O.window_attention_core(q, k, v, r1, r2, talk, win, D ** -0.5)
    got = run_window(backend, q, k, v, r1, r2, talk, win, D ** -0.5, (530, 1, 1), BS=64)
    close(got, want, backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("aim", [0, 1], ids=["just-inside", "just-outside"])
@pytest.mark.parametrize("D,V", [(16, 8), (64, 64)])
def test_window_edge_one_key_stands_out(backend, aim, D, V):
    """Every query points at the key ``win - 1 + aim`` tokens back with a large score: it is the last key
    inside the window (and takes nearly all the weight) or the first one outside (and must not count).
    Rows run in a prompt portion, in portions that end and start at the edge, and one by one."""
    H, G, win, T = 2, 1, 33, 140
    k = F.normalize(rnd(T, G, D, seed=1), dim=-1)
    v = rnd(T, G, V, seed=2)
    q = rnd(T, H, D, seed=3, std=0.1)
    back = win - 1 + aim
    q[back:] += 12.0 * k[:T - back].expand(T - back, H, D)
    b16 = lambda t: t.to(torch.bfloat16).double()  # noqa: E731
    q, k, v = b16(q), b16(k), b16(v)
    r1, r2, talk = torch.full((H,), 0.25, dtype=DT), torch.full((H,), 0.5, dtype=DT), torch.eye(H, dtype=DT)
    want = O.window_attention_core(q, k, v, r1, r2, talk, win, 1.0)
    off_by_one = O.window_attention_core(q, k, v, r1, r2, talk, win - 1 + 2 * aim, 1.0)
    assert float((off_by_one - want).abs().max()) > 0.3       # a window one token off shows
    for cuts in [(T,), (win - 1, 1, 1, win, 2), (60,) + (1,) * 80]:
        close(run_window(backend, q, k, v, r1, r2, talk, win, 1.0, cuts), want, backend[1], scale=2.0)


@pytest.mark.parametrize("backend", BACKENDS)
def test_sink_takes_weight_and_heads_mix(backend):
    """All scores zero and all values one: a row with n keys in its window gives n / (n + 1), the sink
    takes the rest; a permutation as mixing matrix swaps the heads' weights."""
    H, G, D, V, T = 2, 2, 8, 8, 20
    q, k, v = rnd(T, H, D, seed=1), rnd(T, G, D, seed=2), rnd(T, G, V, seed=3)
    b16 = lambda t: t.to(torch.bfloat16).double()  # noqa: E731
    q, k, v = b16(q), b16(k), b16(v)
    zero, eye = torch.zeros(H, dtype=DT), torch.eye(H, dtype=DT)
    ones = run_window(backend, q, k, torch.ones_like(v), zero, zero, eye, 8, 0.0, (T,))
    n = torch.arange(1, T + 1).clamp(max=8).double()
    close(ones, (n / (n + 1))[:, None, None].expand(T, H, V), backend[1])
    swap = torch.tensor([[0.0, 1.0], [1.0, 0.0]], dtype=DT)
    want = O.window_attention_core(q, k, v, zero, zero, swap, 8, 0.3)
    plain = O.window_attention_core(q, k, v, zero, zero, eye, 8, 0.3)
    assert float((want - plain).abs().max()) > 1e-2
    close(run_window(backend, q, k, v, zero, zero, swap, 8, 0.3, (5, 1, 1)), want, backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("E,top,K", [(5, 2, 48), (3, 1, 48), (12, 3, 320), (4, 4, 40), (33, 6, 64)])
def test_router_chooses_with_correction_and_weighs_without(backend, E, top, K):
    dev, dt = backend
    T = 50
    h = rnd(T, K, seed=1).to(torch.bfloat16).double()
    wr = (rnd(E, K, seed=2) * 2.0 * K ** -0.5).to(torch.bfloat16).double()
    corr = rnd(E, seed=3, std=0.3)
    s, idx = O.route(h, wr, corr, top)
    plain = O.route(h, wr, torch.zeros(E, dtype=DT), top)[1]
    if top < E:
        assert not torch.equal(idx.sort(-1).values, plain.sort(-1).values)     # the correction changes the choice
    w, ids = M.route_direct(h.to(dev).to(dt), wr.to(dev).to(dt), top, scoring="softmax", renorm=True,
                            choice_bias=corr.float().to(dev), renorm_eps=1e-20)
    assert torch.equal(ids.cpu().long().sort(-1).values, idx.sort(-1).values)
    sel = torch.gather(s, 1, ids.cpu().long())
    close(w, sel / (sel.sum(-1, keepdim=True) + 1e-20), torch.float32, scale=1.0 if dt == torch.float32 else 300.0)


# ------------------------------------------------------------------ whole models through the engine
@pytest.mark.parametrize("backend", BACKENDS)
def test_layers_match_after_every_layer(backend):
    d = default_config()
    W = weights(d, 1)
    t = toks(30, d["vocab"], 2)
    want_layers = []
    want = O.forward(d, W, t, layers_out=want_layers)
    eng = engine(d, W, backend)
    sid = eng.new_sequence()
    s = eng.seqs[sid]
    s.tokens.extend(t)
    assert eng.kvm.ensure_blocks(s, len(t), {sid})
    header, flat = eng._pack_step([], [(s, len(t))], list(range(len(t))))
    flat_dev = torch.from_numpy(flat).to(eng.device)
    got_layers = []
    from k8s_llm_rca_amd.ops.seq_ops import SegMeta, SegStepInputs
    T = len(t)
    n, maxb = int(header[4]), int(header[5])
    o = [0]

    def take(k):
        a = o[0]
        o[0] += k
        return flat_dev[a:a + k], flat[a:a + k]
    ids, _ = take(T)
    pos, _ = take(T)
    slots, _ = take(T)
    sidx, _ = take(T)
    row_seg, _ = take(T)
    row0, row0_h = take(n + 1)
    pos0, pos0_h = take(n)
    slot, slot_h = take(n)
    bt, _ = take(n * maxb)
    seg = SegMeta(n, row_seg, row0, pos0, slot, bt.view(n, maxb), row0_h.tolist(), pos0_h.tolist(), slot_h.tolist())
    got = eng.model.forward(SegStepInputs(ids, pos, slots, seg, sidx.long()), *eng.kv.tensors(), eng.states.t,
                            layers_out=got_layers)
    assert len(got_layers) == len(want_layers)
    for i, (a, b) in enumerate(zip(got_layers, want_layers)):
        assert rel_err(a, b.float()) < tol(backend[1]), f"layer {i}"
    assert rel_err(got, want.float()) < tol(backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cuts", [(50,), (), (2, 2, 3, 9, 2, 17), (33, 2, 1, 1, 2), (16, 16, 2)],
                         ids=["whole", "decode", "small", "mid", "window"])
def test_prefill_decode_and_portions_agree_with_oracle(backend, cuts):
    d = default_config()
    W = weights(d, 2)
    t = toks(50, d["vocab"], 4)
    want = O.forward(d, W, t).float()
    eng = engine(d, W, backend)
    got = feed_all(eng, eng.new_sequence(), t, cuts)
    assert agrees(got, want, backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
def test_mixed_batches_equal_each_alone_and_reuse_pages_and_slots(backend):
    """Unequal requests side by side, more requests than slots and pages over time."""
    d = default_config()
    W = weights(d, 3)
    lens = [70, 5, 33, 1, 64, 20]
    T = [toks(n, d["vocab"], 10 + i) for i, n in enumerate(lens)]
    want = [O.forward(d, W, t).float() for t in T]
    eng = engine(d, W, backend, num_blocks=7, block_size=32, slots=3)   # 7 pages: not all requests at once
    got = [[] for _ in T]
    at = [0] * len(T)
    sid = {}
    live, waiting = [], list(range(len(T)))
    sizes = [3, 1, 30, 2, 1, 9, 1, 1, 40, 2]
    step = 0
    while live or waiting:
        while waiting and len(live) < 3:
            i = waiting[0]
            need = -(-lens[i] // 32)
            if need > eng.kv.free_blocks - sum(-(-lens[j] // 32) - len(eng.seqs[sid[j]].blocks) for j in live):
                break
            waiting.pop(0)
            sid[i] = eng.new_sequence()
            live.append(i)
        entries = []
        for k, i in enumerate(live):
            n = min(sizes[(step + 3 * k) % len(sizes)], lens[i] - at[i])
            entries.append((sid[i], T[i][at[i]:at[i] + n], list(range(n))))
        lg = eng.feed(entries)
        o = 0
        for (_, tk, _), i in zip(entries, list(live)):
            got[i].append(lg[o:o + len(tk)])
            o += len(tk)
            at[i] += len(tk)
            if at[i] == lens[i]:
                live.remove(i)
                eng.release_sequence(sid[i])
        step += 1
    assert eng.kv.free_blocks == 7 and eng.states.free_slots == 3
    for i in range(len(T)):
        assert agrees(torch.cat(got[i]), want[i], backend[1]), f"request {i}"


@pytest.mark.parametrize("backend", BACKENDS)
def test_window_edges_and_page_borders_sharp_softmax(backend):
    """Large query / key weights make every row attend to a few keys: a key missed, one too many at the
    window's edge or one read from a wrong page changes the logits.  The window (40) is longer than a
    page (32); rows run in portions and then one by one over several page borders."""
    d = config([(parallel(left(heads=2, kv_heads=1, dim=8, vdim=8, window=40, scale=1.0), right(16, 2, 2, 2)), None),
                (parallel(left(heads=2, kv_heads=2, dim=8, vdim=8, window=33, scale=1.0), right(16, 2, 2, 2)), moe())],
               width=32, vocab=128)
    W = weights(d, 4, big=3.0)
    n = 200
    t = toks(n, d["vocab"], 5)
    want = O.forward(d, W, t).float()
    eng = engine(d, W, backend, num_blocks=8, block_size=32)
    got = feed_all(eng, eng.new_sequence(), t, (31, 2, 31, 33, 30))      # then one by one over three borders
    if backend[1] == torch.float32:
        assert rel_err(got, want) < 1e-4
    else:
        e = (got.double().cpu() - want.double()).pow(2).mean(-1).sqrt() / want.double().pow(2).mean(-1).sqrt()
        assert float(e.median()) < 0.05 and float(e.max()) < 0.5


@pytest.mark.parametrize("backend", BACKENDS)
def test_first_tokens(backend):
    d = default_config()
    W = weights(d, 6)
    t = toks(9, d["vocab"], 7)
    want = O.forward(d, W, t).float()
    for cuts in [(1, 1, 1), (1, 3), (2, 1, 2), (4, 1), (9,)]:
        eng = engine(d, W, backend)
        assert agrees(feed_all(eng, eng.new_sequence(), t, cuts), want, backend[1]), cuts
    eng = engine(d, W, backend)
    one = eng.feed([(eng.new_sequence(), t[:1], [0])])
    assert rel_err(one, want[:1]) < tol(backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding_past_the_window(backend):
    d = config([(parallel(left(window=24), right(24, 4, 3, 4)), moe(experts=4, top=2, ff=16)), (ret(), None)],
               width=32, vocab=96)
    W = weights(d, 8)
    t = toks(170, d["vocab"], 9)
    want = O.forward(d, W, t).float()
    eng = engine(d, W, backend, num_blocks=6)
    got = feed_all(eng, eng.new_sequence(), t, (4,))
    assert agrees(got, want, backend[1], 2.0)


ODD = {
    "one-head-top1-conv1": config([(parallel(left(1, 1, 4, 6, 5), right(8, 1, 1, 1)), moe(2, 1, 8, 0))],
                                  width=16, vocab=40, logit_scale=1.0, softcap=5.0),
    "retention-first-no-ff": config([(ret(1, 4, 4, rot_dims=2), None), (ret(5, 6, 10, rot_dims=0), moe(7, 3, 12, 20)),
                                     (parallel(left(4, 4, 16, 4, 100), right(36, 10, 7, 5)), None)],
                                    width=24, vocab=64, eps=1e-3, logit_scale=2.0, softcap=50.0),
    "unaligned": config([(parallel(left(6, 3, 12, 20, 9), right(100, 17, 9, 3)), moe(6, 2, 36, 28)),
                         (ret(7, 6, 10, rot_dims=4, base=100.0), moe(3, 2, 20, 0)),
                         (parallel(left(7, 1, 6, 10, 2), right(60, 5, 4, 2)), moe(3, 3, 20, 4))],
                        width=100, vocab=333),
    "window-equals-page": config([(parallel(left(2, 2, 8, 8, 32), right(16, 4, 2, 3)), moe(4, 2, 130, 8))],
                                 width=136, vocab=30),
    "aligned": config([(parallel(left(8, 2, 64, 64, 48), right(256, 16, 16, 4)), moe(8, 2, 128, 128)),
                       (ret(8, 32, 64), moe(8, 2, 128, 128))], width=256, vocab=512),
}


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", sorted(ODD))
def test_other_sizes(backend, name):
    d = ODD[name]
    W = weights(d, 11)
    t = toks(45, d["vocab"], 12)
    want = O.forward(d, W, t).float()
    eng = engine(d, W, backend)
    got = feed_all(eng, eng.new_sequence(), t, (3, 11, 2, 20))
    assert agrees(got, want, backend[1], 4.0 if name == "retention-first-no-ff" else 1.0)


@pytest.mark.parametrize("backend", BACKENDS[:2])
def test_greedy_generation_through_submit_and_scheduler(backend):
    """``submit`` + ``step``: the scheduler's own batching (two prompts of unequal
    length, then decode rows) must produce the oracle's greedy continuation."""
    d = default_config(vocab=8192)
    W = weights(d, 13)
    eng = engine(d, W, backend, num_blocks=16)
    prompts = [toks(37, 2000, 14), toks(6, 2000, 15)]
    outs = {}
    for i, p in enumerate(prompts):
        eng.submit(eng.new_sequence(), p, None, 6, temperature=0.0, on_done=lambda g, st, i=i: outs.__setitem__(i, g))
    eng.run_until_idle()
    for i, p in enumerate(prompts):
        seq = list(p)
        for _ in range(6):
            seq.append(int(O.forward(d, W, seq)[-1, :eng.vocab].argmax()))
        assert outs[i][:6] == seq[len(p):], i


def test_thread_continues_and_restarts_when_history_diverges():
    d = default_config(vocab=8192)
    W = weights(d, 16)
    eng = engine(d, W, ("cpu", torch.float32), num_blocks=16)
    sid = eng.new_sequence()
    out = {}
    p1 = toks(20, 2000, 17)
    eng.submit(sid, p1, None, 3, temperature=0.0, on_done=lambda g, st: out.__setitem__(1, g))
    eng.run_until_idle()
    s = eng.seqs[sid]
    p2 = list(s.tokens) + toks(5, 2000, 18)
    eng.submit(sid, p2, None, 3, temperature=0.0, on_done=lambda g, st: out.__setitem__(2, g))
    eng.run_until_idle()
    assert eng.stats["recompute_tokens"] == 0
    seq = list(p2)
    for _ in range(3):
        seq.append(int(O.forward(d, W, seq)[-1, :eng.vocab].argmax()))
    assert out[2][:3] == seq[len(p2):]
    p3 = p1[:10] + toks(8, 2000, 19)              # diverges inside the cached tokens
    eng.submit(sid, p3, None, 3, temperature=0.0, on_done=lambda g, st: out.__setitem__(3, g))
    eng.run_until_idle()
    seq = list(p3)
    for _ in range(3):
        seq.append(int(O.forward(d, W, seq)[-1, :eng.vocab].argmax()))
    assert out[3][:3] == seq[len(p3):]


def test_config_round_trip_registry_and_replay(tmp_path):
    """config.json -> configuration -> config.json; a saved checkpoint is found by its architecture and
    replayed by the trace runner's engine with the oracle's logits."""
    from k8s_llm_rca_amd.engine import trace as TR
    from k8s_llm_rca_amd.models import registry as R
    from k8s_llm_rca_amd.models.ligipel import PRESETS, save_checkpoint
    d = default_config()
    cfg = LigipelConfig.from_json(d, "x")
    assert cfg.to_json() == json.loads(json.dumps(d))
    assert R.get_any_config("tiny-ligipel") is PRESETS["tiny-ligipel"]
    W = weights(d, 20)
    path = str(tmp_path / "ckpt")
    save_checkpoint(cfg, W, path)
    assert R.checkpoint_arch(path) == "ligipel"
    eng = TR.make_engine(path, torch.float32, 128, device="cpu")
    assert isinstance(eng.model, LigipelModel) and eng.kv.num_blocks == 2 and eng.states.slots == 4
    t = toks(40, d["vocab"], 21)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": t[:30], "want": [0, 29]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": t[30:31], "want": []},
                                     {"id": "b", "tokens": t[:3], "want": [2]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": t[31:], "want": [8]}], "end": ["a"]}]
    import io
    import numpy as np
    log = io.StringIO()
    out = str(tmp_path / "out")
    assert TR.replay(eng, io.StringIO("\n".join(json.dumps(s) for s in steps)), out, log) == 0
    assert log.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    want = O.forward(d, W, t).float()
    got = [np.fromfile(f"{out}/{i}.f32", dtype="<f4").reshape(-1, d["vocab"]) for i in (0, 1, 2)]
    assert rel_err(torch.from_numpy(got[0]), want[[0, 29]]) < 3e-5
    assert rel_err(torch.from_numpy(got[1]), want[[2]]) < 3e-5
    assert rel_err(torch.from_numpy(got[2]), want[[39]]) < 3e-5
    assert eng.kv.free_blocks == 2 and eng.states.free_slots == 4


def test_trace_run_command_line(tmp_path):
    """``bin/trace_run`` as a program: a checkpoint folder, steps on standard input, logits files out."""
    import os
    import subprocess
    import sys
    import numpy as np
    from k8s_llm_rca_amd.models.ligipel import save_checkpoint
    d = config([(ret(2, 4, 6, rot_dims=4), None), (parallel(left(2, 1, 4, 6, 5), right(12, 3, 2, 3)), moe(3, 2, 8, 0))],
               width=24, vocab=50)
    W = weights(d, 30)
    path = str(tmp_path / "ckpt")
    save_checkpoint(LigipelConfig.from_json(d, "x"), W, path)
    t = toks(12, d["vocab"], 31)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": t[:9], "want": [8]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": t[9:10], "want": [0]}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": t[10:], "want": [0, 1]}], "end": ["q"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = str(tmp_path / "out")
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                        "--out", out, "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    want = O.forward(d, W, t).float()
    got = torch.cat([torch.from_numpy(np.fromfile(f"{out}/{i}.f32", dtype="<f4").reshape(-1, d["vocab"]))
                     for i in range(3)])
    assert rel_err(got, want[[8, 9, 10, 11]]) < 3e-5
