"""Zasapel through the engine against the plain implementation in
``zasapel_oracle.py``: each mechanism alone, prefill against token-by-token
decoding, portions, mixed batches, reuse of pages and state slots, page
borders and far keys, first tokens, long decoding, odd sizes, and greedy
generation through ``submit`` / ``step``.

Every case runs on the CPU (the ops' fp32 forms, the same engine, cache manager
and scheduler) and, marked ``gpu``, on the HIP kernels in fp32 and bf16.
"""
import math

import pytest
import torch

import zasapel_oracle as O
from k8s_llm_rca_amd.engine.engine import EngineConfig, LLMEngine
from k8s_llm_rca_amd.models.zasapel import ZasapelConfig, ZasapelModel
from k8s_llm_rca_amd.ops import moe as M
from k8s_llm_rca_amd.ops import norm as N
from k8s_llm_rca_amd.ops import seq_ops as S

GPU = pytest.mark.gpu
BACKENDS = [pytest.param(("cpu", torch.float32), id="cpu-f32"),
            pytest.param(("cuda", torch.float32), id="gpu-f32", marks=GPU),
            pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=GPU)]


def tol(dtype):
    return 3e-5 if dtype == torch.float32 else 4e-2


def rel_err(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean(-1).sqrt().clamp_min(1e-30)).max())


# ------------------------------------------------------------------ configurations and weights
def attn(heads=2, dim=8, vdim=12, q_rank=20, kv_rank=24, scale=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": 1.0 / math.sqrt(dim) if scale is None else scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m}


def gru(width=40):
    return {"type": "mingru", "mixer": {"width": width}}


def dense(ff=56):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=24, limit=1.5):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top}}


def config(layers, width=48, vocab=512, taps=3, alpha=2.5, eps=1e-5):
    ls = [dict(mix, mlp=mlp) for mix, mlp in layers]
    return {"architecture": "Zasapel", "vocab": vocab, "width": width, "layers": ls, "norm": {"eps": eps},
            "postln_alpha": alpha, "canon": {"taps": taps}}


def default_config(**kw):
    return config([(attn(), dense()), (gru(), moe()), (attn(kv_from=0), moe(experts=3, top=1)),
                   (attn(heads=3, dim=4, vdim=4, q_rank=8, kv_rank=16), None)], **kw)


def weights(d, seed=0, big=1.0):
    """Random weights under the checkpoint's names, rounded to bfloat16."""
    g = torch.Generator().manual_seed(seed)
    W, taps = d["width"], d["canon"]["taps"]

    def r(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).to(torch.bfloat16).float()

    t = {"embed": r(d["vocab"], W), "final.norm": r(W, std=0.2), "head": r(d["vocab"], W, std=W ** -0.5)}
    for i, L in enumerate(d["layers"]):
        p = f"l{i}."
        t[p + "norm1"] = r(W, std=0.2)
        t[p + "canon1"] = r(W, taps, std=0.4)
        m = L["mixer"]
        if L["type"] == "mingru":
            C = m["width"]
            for n in "zxg":
                t[p + "mix." + n] = r(C, W, std=big * W ** -0.5)
            t[p + "mix.z.b"], t[p + "mix.x.b"] = r(C, std=0.7), r(C, std=0.7)
            t[p + "mix.o"] = r(W, C, std=C ** -0.5)
        else:
            H, D, V, QR, KR = m["heads"], m["dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            t[p + "mix.dq"] = r(QR, W, std=W ** -0.5)
            t[p + "mix.dq.norm"] = r(QR, std=0.2, mean=1.0)
            t[p + "mix.uq"] = r(H * D, QR, std=big * QR ** -0.5)
            if "kv_from" not in m:
                t[p + "mix.dkv"] = r(KR, W, std=W ** -0.5)
                t[p + "mix.dkv.norm"] = r(KR, std=0.2, mean=1.0)
            t[p + "mix.uk"] = r(H * D, KR, std=big * KR ** -0.5)
            t[p + "mix.uv"] = r(H * V, KR, std=KR ** -0.5)
            t[p + "mix.g"] = r(H, W, std=W ** -0.5)
            t[p + "mix.o"] = r(W, H * V, std=(H * V) ** -0.5)
        f = L["mlp"]
        if f is None:
            continue
        t[p + "norm2"] = r(W, std=0.2)
        t[p + "canon2"] = r(W, taps, std=0.4)
        if f["kind"] == "dense":
            t[p + "mlp.up"], t[p + "mlp.down"] = r(f["ff"], W, std=W ** -0.5), r(W, f["ff"], std=f["ff"] ** -0.5)
            t[p + "mlp.act"] = torch.tensor([0.75, -0.5, 0.25, 0.125])
        else:
            F = f["expert"]["ff"]
            t[p + "mlp.router"] = r(f["router"]["experts"], W, std=2 * W ** -0.5)
            for e in range(f["router"]["experts"]):
                q = p + f"mlp.e{e}."
                t[q + "gate"], t[q + "up"] = r(F, W, std=2 * W ** -0.5), r(F, W, std=2 * W ** -0.5)
                t[q + "down"] = r(W, F, std=F ** -0.5)
    return t


def engine(d, W, backend, num_blocks=24, block_size=32, slots=4, **kw):
    dev, dt = backend
    model = ZasapelModel(ZasapelConfig.from_json(d, "test"), dev, dt, init=False)
    model.load_tensors(W.__getitem__)
    cfg = dict(model="test", device=dev, dtype=dt, num_blocks=num_blocks, block_size=block_size, state_slots=slots,
               max_batch_tokens=1024, use_graphs=False, temperature=0.0)
    cfg.update(kw)
    eng = LLMEngine(EngineConfig(**cfg), model=model)
    for t in eng.states.t.values():       # a fresh slot must not be read: make a read loud
        t.fill_(float("nan"))
    for c in eng.kv.c + [t for t in eng.kv.ct if t is not None]:
        c.fill_(3e4)                      # stale pages hold finite garbage (masked keys multiply it by 0)
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


# ------------------------------------------------------------------ each mechanism alone
def seg_meta(lens, pos0, slots, dev, block_tables=None):
    row0 = [0]
    for n in lens:
        row0.append(row0[-1] + n)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)  # noqa: E731
    row_seg = [s for s, n in enumerate(lens) for _ in range(n)]
    bt = i32(block_tables if block_tables is not None else [[0]] * len(lens))
    return S.SegMeta(len(lens), i32(row_seg), i32(row0), i32(pos0), i32(slots), bt, row0, list(pos0), list(slots),
                     n_single=0)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_canon_conv_portions_and_tail(backend, taps):
    dev, dt = backend
    g = torch.Generator().manual_seed(taps)
    C, n = 70, 23
    x = torch.randn(n, C, generator=g)
    w = torch.randn(C, taps, generator=g).to(torch.bfloat16).float()
    want = x + O.causal_conv(x.double(), w.double()).float()
    tail = torch.full((3, taps - 1, C), float("nan"), device=dev)
    got = []
    at = 0
    for n_rows in (1, 1, 2, 1, 9, 3, 6):      # shorter and longer than the tail
        seg = seg_meta([n_rows], [at], [2], dev)
        got.append(S.canon_conv(x[at:at + n_rows].to(dev).contiguous(), w.to(dev, dt), tail, seg, dt))
        at += n_rows
    assert at == n
    assert rel_err(torch.cat(got).float(), want) < tol(dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_canon_conv_two_sequences_in_one_step(backend):
    dev, dt = backend
    g = torch.Generator().manual_seed(5)
    C, taps = 33, 4
    xa, xb = torch.randn(9, C, generator=g), torch.randn(6, C, generator=g)
    w = torch.randn(C, taps, generator=g).to(torch.bfloat16).float()
    wa = xa + O.causal_conv(xa.double(), w.double()).float()
    wb = xb + O.causal_conv(xb.double(), w.double()).float()
    tail = torch.full((2, taps - 1, C), float("nan"), device=dev)
    wd = w.to(dev, dt)
    # step 1: a[0:2] with b[0:5]; step 2: a[2:9] with b[5:6]
    s1 = S.canon_conv(torch.cat([xa[:2], xb[:5]]).to(dev), wd, tail, seg_meta([2, 5], [0, 0], [1, 0], dev), dt)
    s2 = S.canon_conv(torch.cat([xb[5:], xa[2:]]).to(dev), wd, tail, seg_meta([1, 7], [5, 2], [0, 1], dev), dt)
    got_a = torch.cat([s1[:2], s2[1:]]).float()
    got_b = torch.cat([s1[2:], s2[:1]]).float()
    assert rel_err(got_a, wa) < tol(dt) and rel_err(got_b, wb) < tol(dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_mingru_scan_matches_recurrence_across_portions(backend):
    dev, dt = backend
    g = torch.Generator().manual_seed(2)
    W, C, n = 24, 300, 40                      # more channels than one workgroup
    h = torch.randn(n, W, generator=g).to(torch.bfloat16).float()
    wt = {"z": torch.randn(C, W, generator=g) * 0.6, "x": torch.randn(C, W, generator=g) * 0.6,
          "g": torch.randn(C, W, generator=g) * 0.4, "z.b": torch.randn(C, generator=g),
          "x.b": torch.randn(C, generator=g), "o": torch.eye(C)}
    wt = {k: v.to(torch.bfloat16).float() for k, v in wt.items()}
    want = O.mingru(h.double(), {k: v.double() for k, v in wt.items()}, "").float()
    zug = (h @ torch.cat([wt["z"], wt["x"], wt["g"]]).T).to(dev).contiguous()
    state = torch.full((2, C), float("nan"), device=dev)
    got, at = [], 0
    for n_rows in (1, 2, 17, 1, 19):
        seg = seg_meta([n_rows], [at], [1], dev)
        got.append(S.mingru_scan(zug[at:at + n_rows].contiguous(), wt["z.b"].to(dev, dt), wt["x.b"].to(dev, dt), state,
                                 seg, dt))
        at += n_rows
    assert rel_err(torch.cat(got).float(), want) < tol(dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_mingru_long_portions_parallel_over_time(backend):
    """Portions much longer than a scan chunk, two sequences in a step, continued afterwards."""
    dev, dt = backend
    g = torch.Generator().manual_seed(3)
    C, na, nb = 70, 333, 200
    bz, bu = torch.randn(C, generator=g).to(torch.bfloat16).float(), torch.randn(C, generator=g).to(torch.bfloat16).float()
    za, zb = torch.randn(na, 3 * C, generator=g) * 1.5, torch.randn(nb, 3 * C, generator=g) * 1.5
    wt = {"z": torch.eye(C), "x": torch.eye(C), "g": torch.eye(C), "z.b": bz, "x.b": bu, "o": torch.eye(C)}

    def want(zug):
        h = zug.double()
        z = torch.sigmoid(h[:, :C] + bz.double())
        u = h[:, C:2 * C] + bu.double()
        cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        S, ys = torch.zeros(C, dtype=torch.float64), []
        for t in range(h.shape[0]):
            S = (1 - z[t]) * S + z[t] * cand[t]
            ys.append(S * torch.nn.functional.silu(h[t, 2 * C:]))
        return torch.stack(ys).float()

    state = torch.full((3, C), float("nan"), device=dev)
    b_, u_ = bz.to(dev, dt), bu.to(dev, dt)
    s1 = S.mingru_scan(torch.cat([za[:300], zb[:150]]).to(dev).contiguous(), b_, u_, state,
                       seg_meta([300, 150], [0, 0], [2, 0], dev), dt)
    s2 = S.mingru_scan(torch.cat([zb[150:], za[300:]]).to(dev).contiguous(), b_, u_, state,
                       seg_meta([50, 33], [150, 300], [0, 2], dev), dt)
    got_a = torch.cat([s1[:300], s2[50:]]).float()
    got_b = torch.cat([s1[300:], s2[:50]]).float()
    assert rel_err(got_a, want(za)) < tol(dt) and rel_err(got_b, want(zb)) < tol(dt)


def paged(c, block_size, order, dev, dt):
    """Latents [n, R] scattered over pages in ``order``; returns (cache, block table row)."""
    n, R = c.shape
    nb = -(-n // block_size)
    cache = torch.full((max(order) + 2, block_size, R), float("nan"), dtype=dt, device=dev)
    for j in range(n):
        cache[order[j // block_size], j % block_size] = c[j].to(dt)
    return cache, order[:nb]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("H,R", [(1, 8), (3, 24), (8, 64), (5, 80)])
def test_latent_attention_paged_causal(backend, H, R):
    dev, dt = backend
    g = torch.Generator().manual_seed(H * 100 + R)
    n, BS = 150, 32
    c = torch.randn(n, R, generator=g).to(torch.bfloat16).float()
    qa = torch.randn(n, H, R, generator=g) * 0.7
    gate = torch.randn(n, H + 3, generator=g)
    sc = torch.einsum("thr,jr->thj", qa.double(), c.double()) * 0.3
    sc = sc.masked_fill(torch.arange(n)[None, None, :] > torch.arange(n)[:, None, None], float("-inf"))
    want = torch.einsum("thj,jr->thr", torch.softmax(sc, -1), c.double()) * torch.sigmoid(gate[:, :H].double())[..., None]
    cache, bt = paged(c, BS, [4, 0, 3, 1, 5], dev, dt)
    # rows 0..99 as a prompt portion, 100..101 a two-token portion, the rest single tokens
    outs = []
    for a, b in [(0, 100), (100, 102)] + [(i, i + 1) for i in range(102, n)]:
        seg = seg_meta([b - a], [a], [0], dev, [bt])
        outs.append(S.latent_attention(qa[a:b].to(dev).contiguous(), cache, gate[a:b].to(dev), seg, 0.3, dt))
    assert rel_err(torch.cat(outs).float().flatten(1), want.float().flatten(1)) < tol(dt)


@pytest.mark.parametrize("backend", BACKENDS)
def test_latent_attention_finds_one_far_key(backend):
    """One key among hundreds carries the whole weight: at the first position, at page borders, far back."""
    dev, dt = backend
    n, R, BS, H = 420, 16, 32, 2
    for far in (0, 31, 32, 63, 64, 200, n - 2):
        c = torch.randn(n, R, generator=torch.Generator().manual_seed(far)).to(torch.bfloat16).float()
        c[far] = 0
        c[far, 0] = 8.0                           # the marked key
        qa = torch.zeros(2, H, R)
        qa[:, :, 0] = 6.0                         # every other key scores ~N(0, 6^2 / ...) below 6 * 8
        c[:, 0] = torch.where(torch.arange(n) == far, c[:, 0], -c[:, 0].abs())
        cache, bt = paged(c, BS, list(range(13, -1, -1)), dev, dt)
        gate = torch.full((2, H), 30.0)
        # the last row sees it; a row AT position far - 1 does not (when there is one)
        rows = [n - 1] + ([far - 1] if far > 0 else [])
        for r in rows:
            seg = seg_meta([1], [r], [0], dev, [bt])
            o = S.latent_attention(qa[:1].to(dev).contiguous(), cache, gate[:1].to(dev), seg, 1.0, dt).float().cpu()
            hit = torch.allclose(o[0, 0], c[far], atol=2e-2)
            assert hit == (r >= far), (far, r)


@GPU
@pytest.mark.parametrize("H,R", [(1, 32), (3, 64), (16, 96), (20, 256), (8, 512), (5, 128)])
def test_latent_attention_matrix_core_kernels(H, R):
    """The MFMA kernels: prompt portions (one and two tiles per wave, heads fewer and more than a
    tile), decode rows over several key partitions, pages in any order, stale pages behind the end."""
    dev, dt = "cuda", torch.bfloat16
    g = torch.Generator().manual_seed(H * 1000 + R)
    n, BS = 700, 64
    c = torch.randn(n, R, generator=g).to(dt).float()
    qa = (torch.randn(n, H, R, generator=g) * 0.5).to(dt).float()
    gate = torch.randn(n, H + 1, generator=g)
    scale = 2.0 / math.sqrt(R)
    sc = torch.einsum("thr,jr->thj", qa.double(), c.double()) * scale
    sc = sc.masked_fill(torch.arange(n)[None, None, :] > torch.arange(n)[:, None, None], float("-inf"))
    want = torch.einsum("thj,jr->thr", torch.softmax(sc, -1), c.double()) * torch.sigmoid(gate[:, :H].double())[..., None]
    order = [7, 2, 11, 0, 5, 9, 3, 1, 10, 4, 8]
    cache = torch.full((13, BS, R), 3e4, dtype=dt, device=dev)
    cache_t = torch.full((13, R, BS), 3e4, dtype=dt, device=dev)
    for j in range(n):
        cache[order[j // BS], j % BS] = c[j].to(dt)
        cache_t[order[j // BS], :, j % BS] = c[j].to(dt)
    pos = torch.arange(n, dtype=torch.int32, device=dev)
    outs = []
    # a long portion, a short one, then decode rows: three at once (one sequence's consecutive tokens), then single
    cuts = [(0, 300), (300, 303), (303, 650), (650, 653)] + [(i, i + 1) for i in range(653, n)]
    for a, b in cuts:
        seg = seg_meta([b - a], [a], [0], dev, [order])
        seg.n_single = (b - a) if b - a <= 3 and a >= 650 else 0
        outs.append(S.latent_attention_mfma(qa[a:b].to(dev, dt).contiguous(), cache, cache_t, gate[a:b].to(dev), seg,
                                            pos[a:b].contiguous(), scale))
    assert rel_err(torch.cat(outs).float().flatten(1), want.float().flatten(1)) < 2e-2


@GPU
def test_latent_attention_matrix_cores_find_one_far_key():
    dev, dt = "cuda", torch.bfloat16
    n, R, BS, H = 900, 64, 32, 4
    for far in (0, 31, 32, 255, 256, 257, 511, 512, 640, n - 2):
        c = torch.randn(n, R, generator=torch.Generator().manual_seed(far)).to(dt).float()
        c[:, 0] = -c[:, 0].abs()
        c[far] = 0
        c[far, 0] = 8.0
        qa = torch.zeros(1, H, R)
        qa[:, :, 0] = 6.0
        pages = list(range(29, -1, -1))
        cache = torch.full((31, BS, R), 3e4, dtype=dt, device=dev)
        cache_t = torch.full((31, R, BS), 3e4, dtype=dt, device=dev)
        for j in range(n):
            cache[pages[j // BS], j % BS] = c[j].to(dt)
            cache_t[pages[j // BS], :, j % BS] = c[j].to(dt)
        gate = torch.full((1, H), 30.0, device=dev)
        for r in [n - 1] + ([far - 1] if far > 0 else []):
            for single in (0, 1):                     # as a prompt row and as a decode row
                seg = seg_meta([1], [r], [0], dev, [pages])
                seg.n_single = single
                o = S.latent_attention_mfma(qa.to(dev, dt), cache, cache_t, gate, seg,
                                            torch.tensor([r], dtype=torch.int32, device=dev), 1.0).float().cpu()
                assert torch.allclose(o[0, 0], c[far], atol=3e-2) == (r >= far), (far, r, single)


@pytest.mark.parametrize("backend", BACKENDS)
def test_polynorm_postnorm_embed(backend):
    dev, dt = backend
    g = torch.Generator().manual_seed(9)
    z = torch.randn(5, 700, generator=g) * 3
    coef = torch.tensor([0.75, -0.5, 0.25, 0.125])
    got = N.polynorm(z.to(dev), coef.to(dev, dt), 1e-5, dt)
    assert rel_err(got.float(), O.polynorm(z.double(), coef, 1e-5).float()) < tol(dt)
    x, y, w = torch.randn(4, 300, generator=g), torch.randn(4, 300, generator=g), torch.randn(300, generator=g) * 0.2
    w = w.to(torch.bfloat16).float()
    xd = x.to(dev).clone()
    S.postnorm_(xd, y.to(dev), w.to(dev, dt), 2.5, 1e-5)
    assert rel_err(xd, O.norm_zero_centered(2.5 * x.double() + y.double(), w.double(), 1e-5).float()) < 3e-5
    emb = torch.randn(50, 36, generator=g).to(torch.bfloat16).float()
    ids, pos = torch.tensor([3, 7, 7, 49], dtype=torch.int32), torch.tensor([0, 1, 5000, 123456], dtype=torch.int32)
    e = S.embed_sinpos(ids.to(dev), pos.to(dev), emb.to(dev, dt))
    want = emb[ids.long()].double() + O.sin_positions(123457, 36, torch.float64)[pos.long()]
    assert float((e.cpu().double() - want).abs().max()) < 2e-6


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("E,top,K,F", [(5, 2, 48, 24), (3, 1, 48, 24), (16, 4, 64, 128), (4, 4, 40, 7)])
def test_sigmoid_router_and_clamped_experts(backend, E, top, K, F):
    """Scores are not renormalised and multiply the expert's INPUT; gate and up are clamped."""
    dev, dt = backend
    g = torch.Generator().manual_seed(E + top)
    T = 37
    h = (torch.randn(T, K, generator=g) * 2).to(torch.bfloat16).float()
    Wt = {"router": torch.randn(E, K, generator=g) * 0.3}
    for e in range(E):
        Wt[f"e{e}.gate"], Wt[f"e{e}.up"] = torch.randn(F, K, generator=g) * 0.4, torch.randn(F, K, generator=g) * 0.4
        Wt[f"e{e}.down"] = torch.randn(K, F, generator=g) * 0.3
    Wt = {k: v.to(torch.bfloat16).float() for k, v in Wt.items()}
    mlp = {"router": {"experts": E, "top": top}, "expert": {"ff": F, "limit": 1.5}}
    want = O.moe_ff(h.double(), {k: v.double() for k, v in Wt.items()}, "", mlp).float()
    hd = h.to(dev, dt)
    w, ids = M.route_direct(hd, Wt["router"].to(dev, dt), top, "sigmoid", False)
    s = torch.sigmoid(h.double() @ Wt["router"].double().T)
    assert torch.equal(ids.cpu().long(), torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top])
    order, inv, offsets = M.align(ids, E)
    xp = M.gather_rows(hd, order, top, w)
    w13 = torch.stack([torch.cat([Wt[f"e{e}.gate"], Wt[f"e{e}.up"]]) for e in range(E)]).to(dev, dt)
    w2 = torch.stack([Wt[f"e{e}.down"] for e in range(E)]).to(dev, dt)
    act = M.glu_clamp(M.grouped_gemm(xp, w13, offsets), 1.702, 1.5, 1.0)
    out = M.combine_f32(M.grouped_gemm(act, w2, offsets), inv, T, top)
    assert rel_err(out, want) < tol(dt)


# ------------------------------------------------------------------ the model through the engine
@pytest.mark.parametrize("backend", BACKENDS)
def test_layers_match_after_every_layer(backend):
    d = default_config()
    W = weights(d, 1)
    eng = engine(d, W, backend)
    t = toks(21, d["vocab"], 3)
    want_layers = []
    want = O.forward(d, W, t, layers_out=want_layers)
    from k8s_llm_rca_amd.models.zasapel import SegStepInputs
    sid = eng.new_sequence()
    s = eng.seqs[sid]
    s.tokens = list(t)
    assert eng.kvm.ensure_blocks(s, len(t), {sid})
    hdr, flat = eng._pack_step([], [(s, len(t))], list(range(len(t))))
    dev_flat = eng._to_dev([flat])[0]
    got_layers = []
    fwd = eng.model.forward
    eng.model.forward = lambda inp, *a: fwd(inp, *a, layers_out=got_layers)
    got = eng._exec_step(hdr, flat, dev_flat)
    for i, (a, b) in enumerate(zip(got_layers, want_layers)):
        assert rel_err(a, b.float()) < tol(backend[1]), f"layer {i}"
    assert rel_err(got, want.float()) < tol(backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("cuts", [(40,), (), (2, 2, 3, 9, 2, 17), (33, 2, 1, 1, 2)], ids=["whole", "decode", "small", "mid"])
def test_prefill_decode_and_portions_agree_with_oracle(backend, cuts):
    d = default_config()
    W = weights(d, 2)
    t = toks(40, d["vocab"], 4)
    want = O.forward(d, W, t).float()
    eng = engine(d, W, backend)
    got = feed_all(eng, eng.new_sequence(), t, cuts)
    assert rel_err(got, want) < tol(backend[1])


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
        assert rel_err(torch.cat(got[i]), want[i]) < tol(backend[1]), f"request {i}"


@pytest.mark.parametrize("backend", BACKENDS)
def test_page_borders_and_far_keys_sharp_softmax(backend):
    """A large score scale makes every row attend to a few keys: a key missed or
    read from a wrong page changes the logits.  Wanted rows sit around page
    borders, in the prompt and decoded one by one."""
    d = config([(attn(heads=2, dim=8, vdim=8, q_rank=16, kv_rank=16, scale=1.5), None),
                (attn(heads=1, dim=8, vdim=8, q_rank=16, kv_rank=16, scale=1.5, kv_from=0), dense(32))],
               width=32, vocab=128, taps=2)
    W = weights(d, 4, big=2.0)
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
def test_decode_past_the_key_partition_border(backend):
    """Decoded tokens whose keys span more than one split-KV partition (256 keys), rank 64 (matrix cores in bf16)."""
    d = config([(attn(heads=4, dim=16, vdim=8, q_rank=24, kv_rank=64), None),
                (attn(heads=2, dim=16, vdim=8, q_rank=24, kv_rank=64, kv_from=0), dense(32))],
               width=32, vocab=128, taps=2)
    W = weights(d, 22)
    t = toks(270, d["vocab"], 23)
    want = O.forward(d, W, t).float()
    eng = engine(d, W, backend, num_blocks=6, block_size=64)
    got = feed_all(eng, eng.new_sequence(), t, (250,))      # then 20 tokens one by one over key 256
    assert rel_err(got, want) < tol(backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
def test_first_tokens(backend):
    d = default_config(taps=5)
    W = weights(d, 6)
    t = toks(9, d["vocab"], 7)
    want = O.forward(d, W, t).float()
    for cuts in [(1, 1, 1), (1, 3), (2, 1, 2), (4, 1), (9,)]:
        eng = engine(d, W, backend)
        assert rel_err(feed_all(eng, eng.new_sequence(), t, cuts), want) < tol(backend[1]), cuts
    eng = engine(d, W, backend)
    one = eng.feed([(eng.new_sequence(), t[:1], [0])])
    assert rel_err(one, want[:1]) < tol(backend[1])


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding(backend):
    d = config([(gru(24), moe(experts=4, top=2, ff=16)), (attn(), None)], width=32, vocab=96, taps=4)
    W = weights(d, 8)
    t = toks(170, d["vocab"], 9)
    want = O.forward(d, W, t).float()
    eng = engine(d, W, backend, num_blocks=6)
    got = feed_all(eng, eng.new_sequence(), t, (4,))
    assert rel_err(got, want) < tol(backend[1]) * 2


ODD = {
    "one-head-top1-taps1": config([(attn(heads=1, dim=4, vdim=6, q_rank=4, kv_rank=8), moe(experts=2, top=1, ff=8))],
                                  width=16, vocab=40, taps=1, alpha=1.0),
    "gru-first-no-ff": config([(gru(16), None), (gru(72), dense(20)), (attn(heads=4, dim=16, vdim=4, q_rank=12,
                                                                              kv_rank=40), moe(7, 3, 12, 0.5))],
                              width=24, vocab=64, taps=2, alpha=4.0, eps=1e-3),
    "two-latent-groups": config([(attn(kv_rank=16), None), (attn(kv_rank=32, heads=5), dense(24)),
                                 (attn(kv_rank=16, kv_from=0, heads=1), None),
                                 (attn(kv_rank=32, kv_from=1, heads=2, vdim=5), moe())], width=40, vocab=50, taps=6),
    "unaligned": config([(attn(heads=3, dim=12, vdim=20, q_rank=36, kv_rank=40), dense(100)), (gru(60), moe(6, 2, 36, 1.0)),
                         (attn(heads=7, dim=6, vdim=10, q_rank=18, kv_rank=40, kv_from=0), moe(3, 2, 20, 3.0))],
                        width=100, vocab=333, taps=3),
    "top-equals-experts": config([(gru(32), moe(experts=3, top=3, ff=130, limit=0.25))], width=136, vocab=30),
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
    assert rel_err(got, want) < tol(backend[1]) * (4 if name == "gru-first-no-ff" else 1)


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
    """A second run on the same sequence keeps pages and state when the prompt
    extends the cached tokens, and starts over when it does not."""
    d = default_config(vocab=8192)
    W = weights(d, 16)
    eng = engine(d, W, ("cpu", torch.float32), num_blocks=16)
    sid = eng.new_sequence()
    out = {}
    p1 = toks(20, 2000, 17)
    eng.submit(sid, p1, None, 3, temperature=0.0, on_done=lambda g, st: out.__setitem__(1, g))
    eng.run_until_idle()
    s = eng.seqs[sid]
    kept = s.n_cached
    p2 = list(s.tokens) + toks(5, 2000, 18)
    eng.submit(sid, p2, None, 3, temperature=0.0, on_done=lambda g, st: out.__setitem__(2, g))
    eng.run_until_idle()
    assert eng.stats["recompute_tokens"] == 0 and kept > 0
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


@pytest.mark.parametrize("backend", BACKENDS)
def test_second_norm_without_feed_forward(backend):
    """A checkpoint that carries ``norm2`` for a layer without a feed-forward: the norm still applies."""
    d = config([(attn(), None), (gru(24), None)], width=32, vocab=64)
    W = weights(d, 24)
    W["l0.norm2"] = (torch.randn(32, generator=torch.Generator().manual_seed(1)) * 0.2).to(torch.bfloat16).float()
    t = toks(14, 64, 25)
    lo = []
    O.forward(d, W, t[:0] + t, layers_out=lo)
    # by hand: layer 0 with the extra norm, then layer 1 and the head from the oracle's pieces
    Wd = {k: v.double() for k, v in W.items()}
    x = Wd["embed"][torch.tensor(t)] + O.sin_positions(len(t), 32, torch.float64)
    h = x + O.causal_conv(x, Wd["l0.canon1"])
    c = O.latent_of(h, Wd, "l0.mix.", 1e-5)
    x = O.norm_zero_centered(2.5 * x + O.latent_attention(h, c, Wd, "l0.mix.", d["layers"][0]["mixer"], 1e-5), Wd["l0.norm1"], 1e-5)
    x = O.norm_zero_centered(2.5 * x, Wd["l0.norm2"], 1e-5)
    h = x + O.causal_conv(x, Wd["l1.canon1"])
    x = O.norm_zero_centered(2.5 * x + O.mingru(h, Wd, "l1.mix."), Wd["l1.norm1"], 1e-5)
    want = (O.norm_zero_centered(x, Wd["final.norm"], 1e-5) @ Wd["head"].T).float()
    dev, dt = backend
    model = ZasapelModel(ZasapelConfig.from_json(d, "test"), dev, dt, init=False)
    model.load_tensors(W.__getitem__, W.__contains__)
    eng = LLMEngine(EngineConfig(model="test", device=dev, dtype=dt, num_blocks=4, block_size=32, state_slots=2,
                                 use_graphs=False), model=model)
    got = feed_all(eng, eng.new_sequence(), t, (9,))
    assert rel_err(got, want) < tol(dt)


def test_config_round_trip_and_registry(tmp_path):
    from k8s_llm_rca_amd.models import registry
    from k8s_llm_rca_amd.models.zasapel import save_checkpoint
    d = ODD["two-latent-groups"]
    cfg = ZasapelConfig.from_json(d)
    assert cfg.to_json()["layers"][2]["mixer"]["kv_from"] == 0 and cfg.n_layers == 4
    W = weights(d, 20)
    save_checkpoint(cfg, W, str(tmp_path))
    assert registry.checkpoint_arch(str(tmp_path)) == "zasapel"
    eng = LLMEngine(EngineConfig(weights=str(tmp_path), device="cpu", dtype=torch.float32, num_blocks=8,
                                 block_size=32, state_slots=2))
    t = toks(12, d["vocab"], 21)
    got = eng.feed([(eng.new_sequence(), t, list(range(12)))])
    assert rel_err(got, O.forward(d, W, t).float()) < 3e-5
    assert registry.get_any_config("tiny-zasapel").arch == "zasapel"
