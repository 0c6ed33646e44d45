"""Zasapel decoder: post-norm layers over an fp32 residual, each sublayer behind a
short causal convolution; mixers are a minGRU recurrence or attention over a
shared latent cache; feed-forwards are dense (PolyNorm) or a sigmoid-routed
mixture of clamped gated experts.

Per layer, with ``x`` the fp32 residual and ``alpha`` = ``postln_alpha``::

    h = x + conv1(x)                               # canon_conv: per-channel, `taps` wide, causal
    x = unit_rms(alpha x + mixer(h)) * (1 + w1)    # postnorm_
    h = x + conv2(x)
    x = unit_rms(alpha x + ff(h)) * (1 + w2)       # when the layer has a feed-forward

``mingru``:            z, u, g = (W_z | W_x | W_g) h (+ biases on z, u); S <- (1 - z) S + z cand(u);
                       out = W_o (S * silu(g)).
``latent_attention``:  one GEMM (W_dq | W_dkv | W_g) h -> the query latent (normed) -> q = W_uq cq;
                       the key-value latent (normed) goes to the paged latent cache -- or is another
                       layer's (``kv_from``); q is moved into latent space with W_uk
                       (``qa[h] = W_uk[h]^T q[h]``), attention runs over the latents, W_uv and W_o follow.
``dense``:             W_down polynorm(W_up h).
``moe``:               scores = sigmoid(W_router h) in fp32, the `top` largest un-renormalised; an expert
                       reads ``score * h``: W_down (min(g, L) sigmoid(1.702 min(g, L)) (clamp(u, -L, L) + 1)).

What a sequence carries from step to step: latents in cache pages (per layer that projects its own),
and in its state slot the last ``taps - 1`` inputs of every convolution and the minGRU states (fp32).
Everything the design fixes is a constant here; every size comes from the configuration.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import torch

from ..ops import moe as M
from ..ops import norm as N
from ..ops import seq_ops as S
from ..ops.linear import linear, linear_f32out
from ..parallel.groups import ParallelContext, single

SIN_BASE = 10000.0      # sinusoidal positions
GLU_ALPHA = 1.702       # experts: g * sigmoid(GLU_ALPHA g)
GLU_UP_SHIFT = 1.0      # experts: (u + 1)


@dataclass(frozen=True)
class MixerSpec:
    kind: str                      # 'mingru' | 'latent_attention'
    width: int = 0                 # mingru: state size
    heads: int = 0
    dim: int = 0                   # query / key size per head
    vdim: int = 0                  # value size per head
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    kv_from: Optional[int] = None  # attend over that layer's latents


@dataclass(frozen=True)
class MlpSpec:
    kind: str                      # 'dense' | 'moe'
    ff: int = 0
    experts: int = 0
    top: int = 0
    limit: float = 0.0


@dataclass(frozen=True)
class ZasapelConfig:
    name: str
    vocab_size: int
    hidden: int
    layers: Tuple[Tuple[MixerSpec, Optional[MlpSpec]], ...]
    rms_eps: float = 1e-6
    postln_alpha: float = 1.0
    taps: int = 4
    max_position: int = 1 << 20    # no learned or tabulated positions: any length the cache holds
    init_std: float = 0.02
    arch: str = "zasapel"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_json(cls, d: dict, name: str = "zasapel") -> "ZasapelConfig":
        layers = []
        for L in d["layers"]:
            m = L.get("mixer") or {}
            if L["type"] == "mingru":
                mx = MixerSpec("mingru", width=int(m["width"]))
            elif L["type"] == "latent_attention":
                kvf = m.get("kv_from")
                mx = MixerSpec("latent_attention", heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                               q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                               kv_from=None if kvf is None else int(kvf))
            else:
                raise ValueError(f"unknown mixer type {L['type']!r}")
            f = L.get("mlp")
            if f is None:
                ff = None
            elif f["kind"] == "dense":
                ff = MlpSpec("dense", ff=int(f["ff"]))
            elif f["kind"] == "moe":
                ff = MlpSpec("moe", ff=int(f["expert"]["ff"]), limit=float(f["expert"]["limit"]),
                             experts=int(f["router"]["experts"]), top=int(f["router"]["top"]))
            else:
                raise ValueError(f"unknown feed-forward kind {f['kind']!r}")
            layers.append((mx, ff))
        return cls(name, int(d["vocab"]), int(d["width"]), tuple(layers), rms_eps=float(d["norm"]["eps"]),
                   postln_alpha=float(d["postln_alpha"]), taps=int(d["canon"]["taps"]))

    def to_json(self) -> dict:
        layers = []
        for mx, ff in self.layers:
            if mx.kind == "mingru":
                m = {"width": mx.width}
            else:
                m = {"heads": mx.heads, "dim": mx.dim, "vdim": mx.vdim, "q_rank": mx.q_rank, "kv_rank": mx.kv_rank,
                     "scale": mx.scale}
                if mx.kv_from is not None:
                    m["kv_from"] = mx.kv_from
            if ff is None:
                f = None
            elif ff.kind == "dense":
                f = {"kind": "dense", "ff": ff.ff}
            else:
                f = {"kind": "moe", "expert": {"ff": ff.ff, "limit": ff.limit},
                     "router": {"experts": ff.experts, "top": ff.top}}
            layers.append({"type": mx.kind, "mixer": m, "mlp": f})
        return {"architecture": "Zasapel", "vocab": self.vocab_size, "width": self.hidden, "layers": layers,
                "norm": {"eps": self.rms_eps}, "postln_alpha": self.postln_alpha, "canon": {"taps": self.taps}}


def _attn(heads, dim, vdim, q_rank, kv_rank, kv_from=None):
    return MixerSpec("latent_attention", heads=heads, dim=dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank,
                     scale=1.0 / math.sqrt(dim), kv_from=kv_from)


def _stack(n_groups: int, W: int, heads: int, dim: int, vdim: int, q_rank: int, kv_rank: int, ff: int,
           experts: int, top: int, eff: int):
    """Groups of (attention + dense, attention sharing latents + MoE, minGRU + MoE)."""
    out = []
    for g in range(n_groups):
        out.append((_attn(heads, dim, vdim, q_rank, kv_rank), MlpSpec("dense", ff=ff)))
        out.append((_attn(heads, dim, vdim, q_rank, kv_rank, kv_from=3 * g),
                    MlpSpec("moe", ff=eff, experts=experts, top=top, limit=7.0)))
        out.append((MixerSpec("mingru", width=W), MlpSpec("moe", ff=eff, experts=experts, top=top, limit=7.0)))
    return tuple(out)


PRESETS: Dict[str, ZasapelConfig] = {
    "tiny-zasapel": ZasapelConfig("tiny-zasapel", 8192, 256, _stack(1, 256, 4, 32, 32, 64, 64, 512, 4, 2, 128),
                                  postln_alpha=2.0),
    # sizes of a ~1B / ~8B-class decoder's layers (benchmarks; random weights)
    "zasapel-1b": ZasapelConfig("zasapel-1b", 32768, 2048, _stack(4, 2048, 16, 128, 128, 768, 256, 8192, 8, 2, 2048),
                                postln_alpha=2.0),
    "zasapel-8b": ZasapelConfig("zasapel-8b", 128256, 4096, _stack(8, 4096, 32, 128, 128, 1536, 512, 14336, 8, 2,
                                                                   4096), postln_alpha=2.0),
}


SegStepInputs = S.SegStepInputs   # the segment-layout step (its home is ops/seq_ops.py)


class ZasapelModel:
    stateful = True            # per-sequence state slots besides cache pages: no rewinding, no page sharing
    step_layout = "segments"   # the engine packs steps as segments (SegStepInputs)
    graph_capturable = False

    def __init__(self, cfg: ZasapelConfig, device, dtype=torch.bfloat16, pc: Optional[ParallelContext] = None,
                 seed: int = 0, init: bool = True):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Zasapel runs in bfloat16 or float32")
        self.dtype = dtype
        self.pc = pc or single()
        if self.pc.tp_size != 1:
            raise ValueError("Zasapel runs on one device per replica (no tensor-parallel sharding of its mixers)")
        self.logits_f32 = True
        self.layers: List[Dict[str, torch.Tensor]] = []
        # layer -> index of the latent cache it reads; conv index of each sublayer; minGRU state index
        self.cache_of: List[Optional[int]] = []
        self.cache_ranks: List[int] = []
        self.conv_of: List[Tuple[int, Optional[int]]] = []
        self.gru_of: List[Optional[int]] = []
        self.gru_widths: List[int] = []
        own: Dict[int, int] = {}
        n_conv = 0
        for i, (mx, ff) in enumerate(cfg.layers):
            if mx.kind == "latent_attention":
                if mx.kv_from is None:
                    own[i] = len(self.cache_ranks)
                    self.cache_ranks.append(mx.kv_rank)
                    self.cache_of.append(own[i])
                else:
                    if mx.kv_from not in own or cfg.layers[mx.kv_from][0].kv_rank != mx.kv_rank:
                        raise ValueError(f"layer {i}: kv_from must name an earlier layer with its own latents "
                                         f"of the same rank")
                    self.cache_of.append(own[mx.kv_from])
                self.gru_of.append(None)
            else:
                self.cache_of.append(None)
                self.gru_of.append(len(self.gru_widths))
                self.gru_widths.append(mx.width)
            self.conv_of.append((n_conv, n_conv + 1 if ff is not None else None))
            n_conv += 1 if ff is None else 2
        self.n_conv = n_conv
        if cfg.taps < 1 or cfg.taps > 16:
            raise ValueError("canon.taps must be 1..16")
        if init:
            self._random_init(seed)

    # ------------------------------------------------------- what the engine allocates for this model
    def cache_bytes_per_block(self, block_size: int) -> int:
        twice = [2 if S.mfma_tiles(r, self.dtype, self.device) else 1 for r in self.cache_ranks]
        return sum(r * t for r, t in zip(self.cache_ranks, twice)) * block_size * (2 if self.dtype == torch.bfloat16
                                                                                    else 4)

    def make_cache(self, num_blocks: int, block_size: int):
        from ..engine.kv_cache import LatentKVPool
        return LatentKVPool(self.cache_ranks, num_blocks, block_size, self.device, self.dtype)

    def state_spec(self) -> Dict[str, Tuple[int, ...]]:
        """Per-slot fp32 state tensors: name -> shape behind the slot dimension."""
        spec = {f"conv{j}": (self.cfg.taps - 1, self.cfg.hidden) for j in range(self.n_conv)}
        for j, c in enumerate(self.gru_widths):
            spec[f"gru{j}"] = (c,)
        return spec

    def workspace_bytes(self, tokens: int) -> int:
        w = self.cfg.hidden
        widest = max([w] + [max(mx.width * 3, mx.heads * max(mx.kv_rank, mx.dim, mx.vdim)) for mx, _ in self.cfg.layers]
                     + [ff.ff * (1 if ff.kind == "dense" else 2 * ff.top) for _, ff in self.cfg.layers if ff])
        return int(tokens * (w * 12 + widest * 12) + (2 << 30))

    # --------------------------------------------------------------- weights
    def _random_init(self, seed: int) -> None:
        t = random_tensors(self.cfg, seed, self.device)
        self.load_tensors(t.__getitem__)

    def load_tensors(self, get, has=None) -> None:
        """Build the fused device layout from checkpoint tensors (``get(name)`` -> tensor, names of the
        safetensors file: ``embed``, ``l<i>.norm1``, ``l<i>.mix.dq`` ...; ``has(name)`` tells what the
        file holds).  A layer without a feed-forward whose checkpoint still carries a second norm keeps
        that norm as an empty second sublayer."""
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def put(*names, dtype=dt):
            ts = [get(n) for n in names]
            t = ts[0] if len(ts) == 1 else torch.cat(ts, 0)
            return t.to(device=dev, dtype=dtype).contiguous()

        self.embed = put("embed")
        self.final_norm = put("final.norm")
        self.lm_head = put("head")
        self.layers = []
        for i, (mx, ff) in enumerate(cfg.layers):
            p = f"l{i}."
            L: Dict[str, torch.Tensor] = {"norm1": put(p + "norm1"), "canon1": put(p + "canon1")}
            if mx.kind == "mingru":
                L["w_zug"] = put(p + "mix.z", p + "mix.x", p + "mix.g")
                L["bz"], L["bu"] = put(p + "mix.z.b"), put(p + "mix.x.b")
                L["wo"] = put(p + "mix.o")
            else:
                H, D, V, KR = mx.heads, mx.dim, mx.vdim, mx.kv_rank
                if mx.kv_from is None:
                    L["w_in"] = put(p + "mix.dq", p + "mix.dkv", p + "mix.g")
                    L["dkv_norm"] = put(p + "mix.dkv.norm")
                else:
                    L["w_in"] = put(p + "mix.dq", p + "mix.g")
                L["dq_norm"] = put(p + "mix.dq.norm")
                L["w_uq"] = put(p + "mix.uq")
                # absorbed forms: per head [D, KR] (fp32: the query is moved into latent space exactly) and [KR, V]
                L["uk"] = put(p + "mix.uk", dtype=torch.float32).view(H, D, KR).contiguous()
                if S.mfma_tiles(KR, dt, dev):
                    L["uk16"] = put(p + "mix.uk").view(H, D, KR).contiguous()
                L["uv_t"] = put(p + "mix.uv").view(H, V, KR).transpose(1, 2).contiguous()
                L["wo"] = put(p + "mix.o")
            if ff is None and has is not None and has(p + "norm2"):
                L["norm2"] = put(p + "norm2")
            if ff is not None:
                L["norm2"], L["canon2"] = put(p + "norm2"), put(p + "canon2")
                if ff.kind == "dense":
                    L["w_up"], L["w_down"], L["act"] = put(p + "mlp.up"), put(p + "mlp.down"), put(p + "mlp.act")
                else:
                    L["router"] = put(p + "mlp.router")
                    L["w13"] = torch.stack([put(p + f"mlp.e{e}.gate", p + f"mlp.e{e}.up")
                                            for e in range(ff.experts)]).contiguous()
                    L["w2"] = torch.stack([put(p + f"mlp.e{e}.down") for e in range(ff.experts)]).contiguous()
            self.layers.append(L)

    def weight_bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for L in self.layers for t in L.values())
        return n + sum(t.numel() * t.element_size() for t in (self.embed, self.lm_head, self.final_norm))

    # -------------------------------------------------------------- forward
    def _lin32(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x @ w.T with an fp32 result (fp32 accumulation either way)."""
        return linear_f32out(x, w) if self.dtype == torch.bfloat16 else linear(x, w)

    def _mingru(self, li: int, h: torch.Tensor, seg: S.SegMeta, states) -> torch.Tensor:
        L = self.layers[li]
        zug = self._lin32(h, L["w_zug"])
        y = S.mingru_scan(zug, L["bz"], L["bu"], states[f"gru{self.gru_of[li]}"], seg, self.dtype)
        return self._lin32(y, L["wo"])

    def _latent_attention(self, li: int, h: torch.Tensor, inp: SegStepInputs, caches, caches_t) -> torch.Tensor:
        L = self.layers[li]
        mx = self.cfg.layers[li][0]
        H, D, V, QR, KR = mx.heads, mx.dim, mx.vdim, mx.q_rank, mx.kv_rank
        T = h.shape[0]
        cache, cache_t = caches[self.cache_of[li]], caches_t[self.cache_of[li]]
        own = mx.kv_from is None
        dn = self._lin32(h, L["w_in"])                       # [T, QR (+ KR) + H] fp32: latents and gate logits
        cq = S.latent_norm(dn, L["dq_norm"], L["dkv_norm"] if own else None, inp.slots, cache if own else None,
                           QR, KR, self.cfg.rms_eps, self.dtype, cache_t=cache_t)
        q = linear(cq, L["w_uq"]).view(T, H, D)
        gate = dn[:, QR + (KR if own else 0):]
        if cache_t is not None:
            # matrix cores: the query moves into latent space as a bf16 batched product (fp32 accumulation)
            qa = torch.bmm(q.transpose(0, 1), L["uk16"]).transpose(0, 1).contiguous()     # [T, H, KR] bf16
            o_lat = S.latent_attention_mfma(qa, cache, cache_t, gate, inp.seg, inp.positions, mx.scale)
        else:
            qa = torch.bmm(q.float().transpose(0, 1), L["uk"]).transpose(0, 1).contiguous()   # [T, H, KR] fp32
            o_lat = S.latent_attention(qa, cache, gate, inp.seg, mx.scale, self.dtype)    # [T, H, KR], gated
        o = torch.bmm(o_lat.transpose(0, 1), L["uv_t"]).transpose(0, 1).reshape(T, H * V)
        return self._lin32(o, L["wo"])

    def _dense(self, li: int, h: torch.Tensor) -> torch.Tensor:
        L = self.layers[li]
        a = N.polynorm(self._lin32(h, L["w_up"]), L["act"], self.cfg.rms_eps, self.dtype)
        return self._lin32(a, L["w_down"])

    def _moe(self, li: int, h: torch.Tensor) -> torch.Tensor:
        L = self.layers[li]
        ff = self.cfg.layers[li][1]
        T = h.shape[0]
        w, ids = M.route_direct(h, L["router"], ff.top, scoring="sigmoid", renorm=False)
        order, inv, offsets = M.align(ids, ff.experts)
        xp = M.gather_rows(h, order, ff.top, w)             # the weight multiplies the expert's input
        gu = M.grouped_auto(xp, L["w13"], offsets)
        act = M.glu_clamp(gu, GLU_ALPHA, ff.limit, GLU_UP_SHIFT)
        yp = M.grouped_auto(act, L["w2"], offsets)
        return M.combine_f32(yp, inv, T, ff.top)

    def forward(self, inp: SegStepInputs, caches: List[torch.Tensor], caches_t: List[Optional[torch.Tensor]],
                states: Dict[str, torch.Tensor], layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits [len(logits_idx), vocab] fp32.  ``caches``: one paged latent tensor per layer with its own
        key-value projection (``caches_t``: their transposed twins, or None); ``states``: the per-slot
        tensors of :meth:`state_spec`.  ``layers_out``
        (debugging): receives a copy of the residual after every layer."""
        cfg = self.cfg
        seg = inp.seg
        x = S.embed_sinpos(inp.input_ids, inp.positions, self.embed, SIN_BASE)
        for li, ((mx, ff), L) in enumerate(zip(cfg.layers, self.layers)):
            c1, c2 = self.conv_of[li]
            h = S.canon_conv(x, L["canon1"], states[f"conv{c1}"], seg, self.dtype)
            y = self._mingru(li, h, seg, states) if mx.kind == "mingru" else self._latent_attention(li, h, inp, caches,
                                                                                                      caches_t)
            S.postnorm_(x, y, L["norm1"], cfg.postln_alpha, cfg.rms_eps)
            if ff is not None:
                h = S.canon_conv(x, L["canon2"], states[f"conv{c2}"], seg, self.dtype)
                y = self._dense(li, h) if ff.kind == "dense" else self._moe(li, h)
                S.postnorm_(x, y, L["norm2"], cfg.postln_alpha, cfg.rms_eps)
            elif "norm2" in L:
                S.postnorm_(x, None, L["norm2"], cfg.postln_alpha, cfg.rms_eps)
            if layers_out is not None:
                layers_out.append(x.clone())
        sel = x.index_select(0, inp.logits_idx)   # wanted rows in the caller's order (any permutation)
        yn = S.unit_norm_out(sel.contiguous(), self.final_norm, cfg.rms_eps)
        return self._lin32(yn, self.lm_head)


def random_tensors(cfg: ZasapelConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Seeded random weights under the checkpoint's names, bfloat16 (so a bfloat16 and a float32 model
    built from them hold the same numbers)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W = cfg.hidden

    def rnd(*shape, std=cfg.init_std, mean=0.0):
        return torch.empty(*shape, dtype=torch.float32, device=dev).normal_(mean, std, generator=g).to(torch.bfloat16)

    t: Dict[str, torch.Tensor] = {"embed": rnd(cfg.vocab_size, W, std=1.0), "final.norm": rnd(W, std=0.1),
                                  "head": rnd(cfg.vocab_size, W, std=1.0 / math.sqrt(W))}
    for i, (mx, ff) in enumerate(cfg.layers):
        p = f"l{i}."
        t[p + "norm1"] = rnd(W, std=0.1)
        t[p + "canon1"] = rnd(W, cfg.taps, std=0.3)
        if mx.kind == "mingru":
            C = mx.width
            for n in ("z", "x", "g"):
                t[p + f"mix.{n}"] = rnd(C, W, std=1.0 / math.sqrt(W))
            t[p + "mix.z.b"] = rnd(C, std=0.5)
            t[p + "mix.x.b"] = rnd(C, std=0.5)
            t[p + "mix.o"] = rnd(W, C, std=1.0 / math.sqrt(C))
        else:
            H, D, V, QR, KR = mx.heads, mx.dim, mx.vdim, mx.q_rank, mx.kv_rank
            t[p + "mix.dq"] = rnd(QR, W, std=1.0 / math.sqrt(W))
            t[p + "mix.dq.norm"] = rnd(QR, std=0.1, mean=1.0)
            t[p + "mix.uq"] = rnd(H * D, QR, std=1.0 / math.sqrt(QR))
            if mx.kv_from is None:
                t[p + "mix.dkv"] = rnd(KR, W, std=1.0 / math.sqrt(W))
                t[p + "mix.dkv.norm"] = rnd(KR, std=0.1, mean=1.0)
            t[p + "mix.uk"] = rnd(H * D, KR, std=1.0 / math.sqrt(KR))
            t[p + "mix.uv"] = rnd(H * V, KR, std=1.0 / math.sqrt(KR))
            t[p + "mix.g"] = rnd(H, W, std=1.0 / math.sqrt(W))
            t[p + "mix.o"] = rnd(W, H * V, std=1.0 / math.sqrt(H * V))
        if ff is None:
            continue
        t[p + "norm2"] = rnd(W, std=0.1)
        t[p + "canon2"] = rnd(W, cfg.taps, std=0.3)
        if ff.kind == "dense":
            t[p + "mlp.up"] = rnd(ff.ff, W, std=1.0 / math.sqrt(W))
            t[p + "mlp.down"] = rnd(W, ff.ff, std=1.0 / math.sqrt(ff.ff))
            t[p + "mlp.act"] = torch.tensor([0.5, 0.3, 0.2, 0.1], device=dev).to(torch.bfloat16)
        else:
            t[p + "mlp.router"] = rnd(ff.experts, W, std=1.0 / math.sqrt(W))
            for e in range(ff.experts):
                t[p + f"mlp.e{e}.gate"] = rnd(ff.ff, W, std=1.0 / math.sqrt(W))
                t[p + f"mlp.e{e}.up"] = rnd(ff.ff, W, std=1.0 / math.sqrt(W))
                t[p + f"mlp.e{e}.down"] = rnd(W, ff.ff, std=1.0 / math.sqrt(ff.ff))
    return t


def load_checkpoint(path: str, device, dtype, pc=None) -> ZasapelModel:
    """A folder with config.json and model.safetensors (bfloat16 weights) -> the model on ``device``."""
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = ZasapelConfig.from_json(json.load(f), name=os.path.basename(os.path.normpath(path)) or "zasapel")
    model = ZasapelModel(cfg, device, dtype, pc, init=False)
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as h:
        model.load_tensors(h.get_tensor, set(h.keys()).__contains__)
    return model


def save_checkpoint(cfg: ZasapelConfig, tensors: Dict[str, torch.Tensor], path: str) -> None:
    """Write config.json + model.safetensors (bfloat16) in the layout :func:`load_checkpoint` reads."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
