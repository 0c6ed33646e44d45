"""Ligipel decoder: pre- and post-normed sublayers (layer norm with bias) over an
fp32 residual, a learned weighted sum over depth behind every layer, two kinds of
mixer and a mixture-of-experts feed-forward with a shared expert.

With ``X_0`` the normed embedding, ``a`` the layer's input and ``LN`` a layer norm::

    x       = a + LN1b(mixer(LN1(a)))
    X_(i+1) = x + LN2b(ff(LN2(x)))                      # when the layer has a feed-forward
    a'      = sum_{j <= i+1} dwa_i[j] X_j               # what the next layer (or the output) reads

``parallel``:   two mixers read the same input; the result is ``(unit_rms(left) w_l + unit_rms(right) w_r) / 2``.
                left  -- sliding-window attention without rotation: a logarithmic distance bias, a sink in
                         the softmax, the heads' weights mixed by a matrix, grouped key / value heads
                         (:func:`..ops.seq_ops.window_attention`);
                right -- a selective state-space layer: in-projection (x | z), short causal convolution +
                         SiLU, (dt | B | C) projection, softplus step size, diagonal recurrence, gate, out.
``retention``:  rotary q / k, ``S <- decay_h S + k v^T``, ``o = S^T q``, per-head unit norm, SiLU gate, out.
``moe``:        softmax router in fp32; experts are chosen by score + correction, weighted by their plain
                scores renormalised; gated SiLU experts; a shared expert runs for every token.
Output:         final layer norm, head, ``cap * tanh(scale * z / cap)``.

What a sequence carries from step to step: keys and values of the attention layers in cache pages,
and in its state slot the convolution tails, state-space states and retention states (fp32).
Every size and every constant that can differ between checkpoints comes from the configuration.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import torch

from ..ops import moe as M
from ..ops import norm as N
from ..ops import seq_ops as S
from ..ops.linear import linear, linear_f32out, swiglu_gemm
from ..parallel.groups import ParallelContext, single
from .moe import MoELayerSet

RENORM_EPS = 1e-20      # router: chosen scores are divided by their sum + RENORM_EPS


@dataclass(frozen=True)
class WindowAttnSpec:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    window: int
    scale: float


@dataclass(frozen=True)
class SsmSpec:
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclass(frozen=True)
class RetentionSpec:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class MoeSpec:
    experts: int
    top: int
    ff: int
    shared_ff: int = 0      # 0: no shared expert


@dataclass(frozen=True)
class LayerSpec:
    kind: str                              # 'parallel' | 'retention'
    left: Optional[WindowAttnSpec] = None
    right: Optional[SsmSpec] = None
    ret: Optional[RetentionSpec] = None
    mlp: Optional[MoeSpec] = None


@dataclass(frozen=True)
class LigipelConfig:
    name: str
    vocab_size: int
    hidden: int
    layers: Tuple[LayerSpec, ...]
    norm_eps: float = 1e-5
    logit_scale: float = 1.0
    logit_softcap: float = 0.0
    max_position: int = 1 << 20    # no tabulated positions: any length the cache holds
    init_std: float = 0.02
    arch: str = "ligipel"

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_json(cls, d: dict, name: str = "ligipel") -> "LigipelConfig":
        layers = []
        for L in d["layers"]:
            m = L.get("mixer") or {}
            f = L.get("mlp")
            mlp = None
            if f is not None:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
                sh = f.get("shared")
                mlp = MoeSpec(experts=int(f["router"]["experts"]), top=int(f["router"]["top"]),
                              ff=int(f["expert"]["ff"]), shared_ff=int(sh["ff"]) if sh else 0)
            if L["type"] == "parallel":
                a, b = m["left"], m["right"]
                layers.append(LayerSpec(
                    "parallel",
                    left=WindowAttnSpec(int(a["heads"]), int(a["kv_heads"]), int(a["dim"]), int(a["vdim"]),
                                        int(a["mask"]["size"]), float(a["scale"])),
                    right=SsmSpec(int(b["inner"]), int(b["state"]), int(b["dt_rank"]), int(b["conv"])), mlp=mlp))
            elif L["type"] == "retention":
                layers.append(LayerSpec(
                    "retention",
                    ret=RetentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]),
                                      tuple(float(v) for v in m["decay"]), int(m["rot"]["dims"]),
                                      float(m["rot"]["base"])), mlp=mlp))
            else:
                raise ValueError(f"unknown mixer type {L['type']!r}")
        return cls(name, int(d["vocab"]), int(d["width"]), tuple(layers), norm_eps=float(d["norm"]["eps"]),
                   logit_scale=float(d.get("logit_scale", 1.0)), logit_softcap=float(d.get("logit_softcap", 0.0)))

    def to_json(self) -> dict:
        layers = []
        for L in self.layers:
            if L.kind == "parallel":
                a, b = L.left, L.right
                m = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim,
                              "mask": {"size": a.window}, "scale": a.scale},
                     "right": {"inner": b.inner, "state": b.state, "dt_rank": b.dt_rank, "conv": b.conv}}
            else:
                r = L.ret
                m = {"heads": r.heads, "dim": r.dim, "vdim": r.vdim, "decay": list(r.decay),
                     "rot": {"dims": r.rot_dims, "base": r.rot_base}}
            f = None
            if L.mlp is not None:
                f = {"kind": "moe", "expert": {"ff": L.mlp.ff}, "router": {"experts": L.mlp.experts, "top": L.mlp.top}}
                if L.mlp.shared_ff:
                    f["shared"] = {"ff": L.mlp.shared_ff}
            layers.append({"type": L.kind, "mixer": m, "mlp": f})
        return {"architecture": "Ligipel", "vocab": self.vocab_size, "width": self.hidden, "layers": layers,
                "norm": {"eps": self.norm_eps}, "logit_scale": self.logit_scale, "logit_softcap": self.logit_softcap}


def _stack(n_groups: int, W: int, heads: int, kv_heads: int, dim: int, window: int, state: int, experts: int,
           top: int, eff: int):
    """Groups of (parallel, parallel, retention), every layer with experts and a shared expert."""
    par = LayerSpec("parallel",
                    left=WindowAttnSpec(heads, kv_heads, dim, dim, window, 1.0 / math.sqrt(dim)),
                    right=SsmSpec(inner=2 * W, state=state, dt_rank=max(1, W // 16), conv=4),
                    mlp=MoeSpec(experts, top, eff, eff))
    ret = LayerSpec("retention",
                    ret=RetentionSpec(heads, dim // 2, dim, tuple(1.0 - 2.0 ** (-5 - 3 * h / max(1, heads - 1))
                                                                  for h in range(heads)), dim // 2, 1e6),
                    mlp=MoeSpec(experts, top, eff, eff))
    return tuple([par, par, ret] * n_groups)


PRESETS: Dict[str, LigipelConfig] = {
    "tiny-ligipel": LigipelConfig("tiny-ligipel", 8192, 256, _stack(1, 256, 4, 2, 32, 48, 8, 4, 2, 128),
                                  logit_scale=0.5, logit_softcap=30.0),
    # sizes of a ~1B-class decoder's layers (benchmarks; random weights)
    "ligipel-1b": LigipelConfig("ligipel-1b", 32768, 2048, _stack(4, 2048, 16, 2, 128, 1024, 16, 8, 2, 2048),
                                logit_scale=1.0, logit_softcap=30.0),
}


class LigipelModel:
    stateful = True            # per-sequence state slots besides cache pages: no rewinding, no page sharing
    step_layout = "segments"   # the engine packs steps as segments (ops.seq_ops.SegStepInputs)
    graph_capturable = False

    def __init__(self, cfg: LigipelConfig, device, dtype=torch.bfloat16, pc: Optional[ParallelContext] = None,
                 seed: int = 0, init: bool = True):
        self.cfg = cfg
        self.device = torch.device(device)
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Ligipel runs in bfloat16 or float32")
        self.dtype = dtype
        self.pc = pc or single()
        if self.pc.tp_size != 1:
            raise ValueError("Ligipel runs on one device per replica (no tensor-parallel sharding of its mixers)")
        self.logits_f32 = True
        self.layers: List[Dict[str, torch.Tensor]] = []
        # layer -> index of its key / value pages, of its convolution tail / state-space state, of its
        # retention state
        self.cache_of: List[Optional[int]] = []
        self.cache_widths: List[Tuple[int, int]] = []
        self.ssm_of: List[Optional[int]] = []
        self.ret_of: List[Optional[int]] = []
        n_ssm = n_ret = 0
        for i, L in enumerate(cfg.layers):
            if L.kind == "parallel":
                a, b = L.left, L.right
                if a.heads % a.kv_heads:
                    raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
                if not 1 <= b.conv <= 16:
                    raise ValueError(f"layer {i}: conv must be 1..16")
                self.cache_of.append(len(self.cache_widths))
                self.cache_widths.append((a.kv_heads * a.dim, a.kv_heads * a.vdim))
                self.ssm_of.append(n_ssm)
                self.ret_of.append(None)
                n_ssm += 1
            else:
                r = L.ret
                if len(r.decay) != r.heads or r.rot_dims % 2 or r.rot_dims > r.dim:
                    raise ValueError(f"layer {i}: one decay per head, an even rot.dims <= dim")
                self.cache_of.append(None)
                self.ssm_of.append(None)
                self.ret_of.append(n_ret)
                n_ret += 1
            if L.mlp is not None and not 1 <= L.mlp.top <= L.mlp.experts:
                raise ValueError(f"layer {i}: top must be 1..experts")
        if init:
            self._random_init(seed)

    # ------------------------------------------------------- what the engine allocates for this model
    def cache_bytes_per_block(self, block_size: int) -> int:
        per = sum(a + (2 * b if tw else b) for (a, b), tw in zip(self.cache_widths, self._twins()))
        return max(1, per) * block_size * (2 if self.dtype == torch.bfloat16 else 4)

    def _twins(self) -> List[bool]:
        """Per attention layer: whether the matrix-core kernel runs it (then its values are also cached
        transposed)."""
        return [S.window_mfma_ok(L.left.heads, L.left.kv_heads, L.left.dim, L.left.vdim, self.dtype, self.device)
                for L in self.cfg.layers if L.kind == "parallel"]

    def make_cache(self, num_blocks: int, block_size: int):
        from ..engine.kv_cache import WindowKVPool
        return WindowKVPool(self.cache_widths, num_blocks, block_size, self.device, self.dtype, self._twins())

    def state_spec(self) -> Dict[str, Tuple[int, ...]]:
        """Per-slot fp32 state tensors: name -> shape behind the slot dimension."""
        spec: Dict[str, Tuple[int, ...]] = {}
        for i, L in enumerate(self.cfg.layers):
            if L.kind == "parallel":
                j, b = self.ssm_of[i], L.right
                spec[f"conv{j}"] = (b.conv - 1, b.inner)
                spec[f"ssm{j}"] = (b.inner, b.state)
            else:
                r = L.ret
                spec[f"ret{self.ret_of[i]}"] = (r.heads, r.dim, r.vdim)
        return spec

    def workspace_bytes(self, tokens: int) -> int:
        w = self.cfg.hidden
        widest = w
        for L in self.cfg.layers:
            if L.kind == "parallel":
                a, b = L.left, L.right
                widest = max(widest, a.heads * (a.dim + a.vdim) + a.kv_heads * (a.dim + a.vdim), 4 * b.inner)
            else:
                widest = max(widest, 2 * L.ret.heads * (L.ret.dim + L.ret.vdim))
            if L.mlp is not None:
                widest = max(widest, 3 * L.mlp.ff * L.mlp.top + w * L.mlp.top, 3 * L.mlp.shared_ff)
        # the stack of layer results (fp32) + the widest activations
        return int(tokens * ((self.cfg.n_layers + 4) * w * 4 + widest * 12) + (2 << 30))

    # --------------------------------------------------------------- weights
    def _random_init(self, seed: int) -> None:
        t = random_tensors(self.cfg, seed, self.device)
        self.load_tensors(t.__getitem__)

    def load_tensors(self, get, has=None) -> None:
        """Build the fused device layout from checkpoint tensors (``get(name)`` -> tensor; names of the
        safetensors file: ``embed``, ``l<i>.norm1``, ``l<i>.mix.left.q`` ...)."""
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def put(*names, dtype=dt):
            ts = [get(n) for n in names]
            t = ts[0] if len(ts) == 1 else torch.cat(ts, 0)
            return t.to(device=dev, dtype=dtype).contiguous()

        def f32(name):
            return put(name, dtype=torch.float32)

        def norm(name):
            return f32(name), f32(name + ".b")

        self.embed = put("embed")
        self.embed_norm = norm("embed.norm")
        self.final_norm = norm("final.norm")
        self.lm_head = put("head")
        self.layers = []
        for i, spec in enumerate(cfg.layers):
            p = f"l{i}."
            L: Dict[str, object] = {"norm1": norm(p + "norm1"), "norm1b": norm(p + "norm1b"), "dwa": f32(p + "dwa")}
            if spec.kind == "parallel":
                a, b = p + "mix.left.", p + "mix.right."
                L["w_qkv"] = put(a + "q", a + "k", a + "v")
                L["r1"], L["r2"], L["talk"] = f32(a + "r1"), f32(a + "r2"), f32(a + "talk")
                L["wo_l"] = put(a + "o")
                L["w_in"] = put(b + "in")
                L["conv_w"], L["conv_b"] = f32(b + "conv"), f32(b + "conv.b")
                L["w_x"], L["w_dt"], L["dt_b"] = put(b + "x"), put(b + "dt"), f32(b + "dt.b")
                L["A"] = (-torch.exp(f32(b + "A_log"))).contiguous()
                L["D"] = f32(b + "D")
                L["wo_r"] = put(b + "o")
                L["out_l"], L["out_r"] = f32(p + "mix.left.out"), f32(p + "mix.right.out")
            else:
                m = p + "mix."
                L["w_qkvg"] = put(m + "q", m + "k", m + "v", m + "g")
                L["wo"] = put(m + "o")
                L["decay"] = torch.tensor(spec.ret.decay, dtype=torch.float32, device=dev)
            f = spec.mlp
            if f is not None:
                L["norm2"], L["norm2b"] = norm(p + "norm2"), norm(p + "norm2b")
                L["router"] = put(p + "mlp.router")
                L["correction"] = f32(p + "mlp.correction")
                L["w13"] = torch.stack([put(p + f"mlp.e{e}.gate", p + f"mlp.e{e}.up")
                                        for e in range(f.experts)]).contiguous()
                L["w2"] = torch.stack([put(p + f"mlp.e{e}.down") for e in range(f.experts)]).contiguous()
                if f.shared_ff:
                    L["ws13"] = put(p + "mlp.shared.gate", p + "mlp.shared.up")
                    L["ws2"] = put(p + "mlp.shared.down")
            self.layers.append(L)

    def weight_bytes(self) -> int:
        def size(v):
            if isinstance(v, tuple):
                return sum(size(t) for t in v)
            return v.numel() * v.element_size()
        n = sum(size(t) for L in self.layers for t in L.values())
        return n + sum(size(t) for t in (self.embed, self.lm_head, self.embed_norm, self.final_norm))

    # -------------------------------------------------------------- forward
    def _lin32(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x @ w.T with an fp32 result (fp32 accumulation either way)."""
        return linear_f32out(x, w) if self.dtype == torch.bfloat16 else linear(x, w)

    def _window_attention(self, li: int, h: torch.Tensor, inp: S.SegStepInputs, kcs, vcs, vts) -> torch.Tensor:
        L, a = self.layers[li], self.cfg.layers[li].left
        ci = self.cache_of[li]
        kc, vc, vt = kcs[ci], vcs[ci], vts[ci]
        qkv = linear(h, L["w_qkv"])                                  # [T, H D + G D + G V]
        S.window_kv_write(qkv, a.heads * a.dim, kc, vc, inp.slots, vt)
        o = S.window_attention(qkv, a.heads, a.kv_heads, a.dim, a.vdim, kc, vc, L["r1"], L["r2"], L["talk"],
                               a.window, a.scale, inp.seg, vt)
        return self._lin32(o, L["wo_l"])

    def _ssm(self, li: int, h: torch.Tensor, seg: S.SegMeta, states) -> torch.Tensor:
        L, b = self.layers[li], self.cfg.layers[li].right
        j = self.ssm_of[li]
        C, R = b.inner, b.dt_rank
        xz = linear(h, L["w_in"])                                    # [T, 2C]: x | z
        xc = S.short_conv(xz[:, :C], L["conv_w"], L["conv_b"], states[f"conv{j}"], seg, act=True)
        dbc = self._lin32(xc, L["w_x"])                              # [T, R + 2N] fp32: dt | B | C
        dtp = self._lin32(dbc[:, :R].to(self.dtype).contiguous(), L["w_dt"])   # [T, C] fp32, before the bias
        y = S.selective_scan(xc, dtp, L["dt_b"], dbc, R, L["A"], L["D"], xz[:, C:], states[f"ssm{j}"], seg)
        return self._lin32(y, L["wo_r"])

    def _retention(self, li: int, h: torch.Tensor, inp: S.SegStepInputs, states) -> torch.Tensor:
        L, r = self.layers[li], self.cfg.layers[li].ret
        qkvg = self._lin32(h, L["w_qkvg"])                           # [T, 2 H D + 2 H V] fp32
        o = S.retention(qkvg, r.heads, r.dim, r.vdim, L["decay"], r.rot_dims, r.rot_base,
                        states[f"ret{self.ret_of[li]}"], inp.seg, inp.positions, self.cfg.norm_eps, self.dtype)
        return self._lin32(o, L["wo"])

    def _moe(self, li: int, h: torch.Tensor):
        """(routed experts' output, shared expert's output or None), both fp32 [T, W]."""
        L, f = self.layers[li], self.cfg.layers[li].mlp
        T = h.shape[0]
        w, ids = M.route_direct(h, L["router"], f.top, scoring="softmax", renorm=True, choice_bias=L["correction"],
                                renorm_eps=RENORM_EPS)
        order, inv, offsets = M.align(ids, f.experts)
        xp = M.gather_rows(h, order, f.top)
        rows, W = xp.shape
        if (xp.is_cuda and xp.dtype == torch.bfloat16 and rows > M.BIG_MIN_ROWS and M.grouped_big_ok(rows, f.ff, W, True)
                and M.grouped_big_ok(rows, W, f.ff, False)):
            # prefill sizes: the grouped MFMA GEMM with the gated unit in its epilogue (gate_up never written)
            act = M.grouped_big(xp, L["w13"], offsets, silu=True)
        elif xp.is_cuda and xp.dtype == torch.bfloat16 and rows <= MoELayerSet.GLDS_MAX_ROWS:
            # decode sizes: the weight-streaming kernels the Mixtral block runs there (LDS-DMA strips for
            # gate_up; the down projection below with its K split over workgroups)
            gu = M.grouped_gemm(xp, L["w13"], offsets, glds=MoELayerSet.GLDS_UP[0], splits=MoELayerSet.GLDS_UP[1])
            act = M.glu_clamp(gu, 1.0, math.inf, 0.0)
        else:
            act = M.glu_clamp(M.grouped_auto(xp, L["w13"], offsets), 1.0, math.inf, 0.0)  # silu(gate) * up
        if xp.is_cuda and xp.dtype == torch.bfloat16 and rows <= MoELayerSet.SPLIT_MAX_ROWS:
            yp = M.grouped_gemm(act, L["w2"], offsets, splits=MoELayerSet.DOWN_SPLITS)
        else:
            yp = M.grouped_auto(act, L["w2"], offsets)
        routed = M.combine_f32(yp, inv, T, f.top, w)
        shared = None
        if f.shared_ff:
            act = swiglu_gemm(h, L["ws13"])                       # one launch where a fused kernel takes the shape
            if act is None:
                act = M.glu_clamp(linear(h, L["ws13"]), 1.0, math.inf, 0.0)
            shared = self._lin32(act, L["ws2"])
        return routed, shared

    def forward(self, inp: S.SegStepInputs, kcs: List[torch.Tensor], vcs: List[torch.Tensor],
                vts: List[Optional[torch.Tensor]], states: Dict[str, torch.Tensor],
                layers_out: Optional[list] = None) -> torch.Tensor:
        """Logits [len(logits_idx), vocab] fp32.  ``kcs`` / ``vcs``: the paged keys and values of every
        attention layer (``vts``: the values' transposed twins, or None); ``states``: the per-slot tensors of :meth:`state_spec`.  ``layers_out``
        (debugging): receives a copy of the residual after every layer (behind its sum over depth)."""
        cfg, eps, dt = self.cfg, self.cfg.norm_eps, self.dtype
        T, W, nl = inp.input_ids.shape[0], cfg.hidden, cfg.n_layers
        X = torch.empty(nl + 1, T, W, dtype=torch.float32, device=self.device)   # X_0 and every layer's result
        a, A = X[0], torch.empty(T, W, dtype=torch.float32, device=self.device)
        first = self.layers[0]["norm1"] if nl else (None, None)
        h = N.embed_layernorm(inp.input_ids, self.embed, *self.embed_norm, eps, X[0], *first, out_dtype=dt)
        for li, (spec, L) in enumerate(zip(cfg.layers, self.layers)):
            nxt = L["norm2"] if spec.mlp is not None else (None, None)
            if spec.kind == "parallel":
                yl = self._window_attention(li, h, inp, kcs, vcs, vts)
                yr = self._ssm(li, h, inp.seg, states)
                h = N.ln_residual(a, yl, *L["norm1b"], eps, X[li + 1], y2=yr, merge="rms",
                                  mw=(L["out_l"], L["out_r"]), nw=nxt[0], nb=nxt[1], out_dtype=dt)
            else:
                y = self._retention(li, h, inp, states)
                h = N.ln_residual(a, y, *L["norm1b"], eps, X[li + 1], nw=nxt[0], nb=nxt[1], out_dtype=dt)
            if spec.mlp is not None:
                routed, shared = self._moe(li, h)
                N.ln_residual(X[li + 1], routed, *L["norm2b"], eps, X[li + 1], y2=shared, merge="sum")
            last = li == nl - 1
            if last and layers_out is None:
                _, h = N.depth_mix_ln(X, li + 2, L["dwa"], *self.final_norm, eps, dt, rows=inp.logits_idx)
            else:
                nn_ = self.final_norm if last else self.layers[li + 1]["norm1"]
                a, h = N.depth_mix_ln(X, li + 2, L["dwa"], *nn_, eps, dt, a_out=A)
                if layers_out is not None:
                    layers_out.append(a.clone())
                if last:
                    h = h.index_select(0, inp.logits_idx)
        if nl == 0:
            h = N.layernorm(X[0].index_select(0, inp.logits_idx).contiguous(), *self.final_norm, eps, dt)
        logits = self._lin32(h.contiguous(), self.lm_head)
        return N.softcap_(logits, cfg.logit_scale, cfg.logit_softcap)


def random_tensors(cfg: LigipelConfig, seed: int = 0, device="cpu") -> Dict[str, torch.Tensor]:
    """Seeded random weights under the checkpoint's names, bfloat16 (so a bfloat16 and a float32 model
    built from them hold the same numbers)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev)
    g.manual_seed(seed)
    W = cfg.hidden

    def rnd(*shape, std=cfg.init_std, mean=0.0):
        return torch.empty(*shape, dtype=torch.float32, device=dev).normal_(mean, std, generator=g).to(torch.bfloat16)

    def lin(n_out, n_in):
        return rnd(n_out, n_in, std=1.0 / math.sqrt(n_in))

    t: Dict[str, torch.Tensor] = {"embed": rnd(cfg.vocab_size, W, std=1.0), "head": lin(cfg.vocab_size, W)}

    def norm(name):
        t[name] = rnd(W, std=0.1, mean=1.0)
        t[name + ".b"] = rnd(W, std=0.05)

    norm("embed.norm")
    norm("final.norm")
    for i, L in enumerate(cfg.layers):
        p = f"l{i}."
        norm(p + "norm1")
        norm(p + "norm1b")
        if L.kind == "parallel":
            a, b = L.left, L.right
            q = p + "mix.left."
            t[q + "q"], t[q + "k"] = lin(a.heads * a.dim, W), lin(a.kv_heads * a.dim, W)
            t[q + "v"], t[q + "o"] = lin(a.kv_heads * a.vdim, W), lin(W, a.heads * a.vdim)
            t[q + "r1"] = rnd(a.heads, std=0.2, mean=0.5)
            t[q + "r2"] = rnd(a.heads, std=0.05, mean=0.5).abs()
            t[q + "talk"] = (torch.eye(a.heads, device=dev) + 0.1 * rnd(a.heads, a.heads, std=1.0).float()).to(
                torch.bfloat16)
            t[q + "out"] = rnd(W, std=0.1, mean=1.0)
            m = p + "mix.right."
            t[m + "in"] = lin(2 * b.inner, W)
            t[m + "conv"], t[m + "conv.b"] = rnd(b.inner, b.conv, std=0.4), rnd(b.inner, std=0.1)
            t[m + "x"] = lin(b.dt_rank + 2 * b.state, b.inner)
            t[m + "dt"], t[m + "dt.b"] = lin(b.inner, b.dt_rank), rnd(b.inner, std=0.5, mean=-2.0)
            t[m + "A_log"] = torch.log(torch.arange(1, b.state + 1, dtype=torch.float32, device=dev)).expand(
                b.inner, b.state).to(torch.bfloat16).contiguous()
            t[m + "D"] = rnd(b.inner, std=0.1, mean=1.0)
            t[m + "o"] = lin(W, b.inner)
            t[m + "out"] = rnd(W, std=0.1, mean=1.0)
        else:
            r = L.ret
            m = p + "mix."
            t[m + "q"], t[m + "k"] = lin(r.heads * r.dim, W), lin(r.heads * r.dim, W)
            t[m + "v"], t[m + "g"] = lin(r.heads * r.vdim, W), lin(r.heads * r.vdim, W)
            t[m + "o"] = lin(W, r.heads * r.vdim)
        f = L.mlp
        if f is not None:
            norm(p + "norm2")
            norm(p + "norm2b")
            t[p + "mlp.router"] = lin(f.experts, W)
            t[p + "mlp.correction"] = rnd(f.experts, std=0.02)
            for e in [f"e{e}" for e in range(f.experts)] + (["shared"] if f.shared_ff else []):
                ff = f.shared_ff if e == "shared" else f.ff
                t[p + f"mlp.{e}.gate"], t[p + f"mlp.{e}.up"] = lin(ff, W), lin(ff, W)
                t[p + f"mlp.{e}.down"] = lin(W, ff)
        d = torch.full((i + 2,), 0.1 / (i + 1), dtype=torch.float32, device=dev)
        d[-1] = 1.0
        t[p + "dwa"] = d.to(torch.bfloat16)
    return t


def load_checkpoint(path: str, device, dtype, pc=None) -> LigipelModel:
    """A folder with config.json and model.safetensors (bfloat16 weights) -> the model on ``device``."""
    from safetensors import safe_open
    with open(os.path.join(path, "config.json")) as f:
        cfg = LigipelConfig.from_json(json.load(f), name=os.path.basename(os.path.normpath(path)) or "ligipel")
    model = LigipelModel(cfg, device, dtype, pc, init=False)
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as h:
        model.load_tensors(h.get_tensor, set(h.keys()).__contains__)
    return model


def save_checkpoint(cfg: LigipelConfig, tensors: Dict[str, torch.Tensor], path: str) -> None:
    """Write config.json + model.safetensors (bfloat16) in the layout :func:`load_checkpoint` reads."""
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg.to_json(), f, indent=1)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in tensors.items()},
              os.path.join(path, "model.safetensors"))
