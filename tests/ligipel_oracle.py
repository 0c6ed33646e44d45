"""Plain, slow Ligipel: every mechanism as one function over a whole sequence,
straight from the design's equations.  Shares no code with the package; the
tests compare the engine against it.

``cfg`` is the config.json dictionary, ``w`` a name -> tensor mapping with the
checkpoint's names.  Everything runs in ``dt`` (float64 by default).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn.functional as F


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def window_attention_core(q, k, v, r1, r2, talk, win, scale):
    """q [T, H, D], k [T, G, D], v [T, G, V] of one sequence -> [T, H, V]."""
    T, H, _ = q.shape
    G, V = k.shape[1], v.shape[2]
    dt = q.dtype
    P = torch.zeros(H, T, T, dtype=dt)
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            lo = max(0, i - win + 1)
            j = torch.arange(lo, i + 1)
            s = (k[j, g] @ q[i, hh]) * scale - r1[hh] * torch.log1p(r2[hh] * (i - j).to(dt))
            e = torch.exp(s)
            P[hh, i, lo:i + 1] = e / (1.0 + e.sum())
    Pm = torch.einsum("hg,gij->hij", talk, P)
    out = torch.zeros(T, H, V, dtype=dt)
    for hh in range(H):
        out[:, hh] = Pm[hh] @ v[:, hh // (H // G)]
    return out


def window_attention(h, w, p, m, dt):
    """Sliding window, log-distance bias, softmax with a zero-score sink, heads' weights mixed."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].to(dt).T).view(T, H, D)
    k = (h @ w[p + "k"].to(dt).T).view(T, G, D)
    v = (h @ w[p + "v"].to(dt).T).view(T, G, V)
    out = window_attention_core(q, k, v, w[p + "r1"].to(dt), w[p + "r2"].to(dt), w[p + "talk"].to(dt),
                                m["mask"]["size"], m["scale"])
    return out.reshape(T, H * V) @ w[p + "o"].to(dt).T


def causal_conv_silu(x, cw, cb):
    """x [T, C], cw [C, taps] (last column: the current token), cb [C]."""
    T, C = x.shape
    taps = cw.shape[1]
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x])
    out = torch.zeros(T, C, dtype=x.dtype)
    for t in range(T):
        out[t] = (xp[t:t + taps] * cw.T).sum(0) + cb
    return F.silu(out)


def selective_scan(xc, dlt, A, B, Cm, D):
    """xc, dlt [T, C]; A [C, N]; B, Cm [T, N]; D [C] -> y [T, C] (before the gate)."""
    T, C = xc.shape
    S = torch.zeros(C, A.shape[1], dtype=xc.dtype)
    y = torch.zeros(T, C, dtype=xc.dtype)
    for t in range(T):
        S = torch.exp(dlt[t][:, None] * A) * S + (dlt[t] * xc[t])[:, None] * B[t][None, :]
        y[t] = S @ Cm[t] + D * xc[t]
    return y


def mamba(h, w, p, m, dt):
    C, N, R = m["inner"], m["state"], m["dt_rank"]
    xz = h @ w[p + "in"].to(dt).T
    x, z = xz[:, :C], xz[:, C:]
    xc = causal_conv_silu(x, w[p + "conv"].to(dt), w[p + "conv.b"].to(dt))
    dbc = xc @ w[p + "x"].to(dt).T
    dlt = F.softplus(dbc[:, :R] @ w[p + "dt"].to(dt).T + w[p + "dt.b"].to(dt))
    A = -torch.exp(w[p + "A_log"].to(dt))
    y = selective_scan(xc, dlt, A, dbc[:, R:R + N], dbc[:, R + N:R + 2 * N], w[p + "D"].to(dt))
    return (y * F.silu(z)) @ w[p + "o"].to(dt).T


def parallel_mixer(h, w, p, m, eps, dt):
    a = window_attention(h, w, p + "left.", m["left"], dt)
    b = mamba(h, w, p + "right.", m["right"], dt)
    return 0.5 * (rms(a, eps) * w[p + "left.out"].to(dt) + rms(b, eps) * w[p + "right.out"].to(dt))


def rotate(x, pos, dims, base, dt):
    """x [T, H, D]: the first ``dims`` entries of each head, entry i paired with i + dims/2."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    a = pos.double()[:, None] * f[None]
    c, s = a.cos().to(dt)[:, None, :], a.sin().to(dt)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], -1)


def retention_core(q, k, v, decay):
    """q, k [T, H, D] (rotated, k scaled), v [T, H, V] -> o [T, H, V]."""
    T, H, D = q.shape
    o = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for hh in range(H):
        S = torch.zeros(D, v.shape[2], dtype=q.dtype)
        for t in range(T):
            S = decay[hh] * S + k[t, hh][:, None] * v[t, hh][None, :]
            o[t, hh] = S.T @ q[t, hh]
    return o


def retention(h, w, p, m, eps, dt):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rotate((h @ w[p + "q"].to(dt).T).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"], dt)
    k = rotate((h @ w[p + "k"].to(dt).T).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"], dt) * D ** -0.5
    v = (h @ w[p + "v"].to(dt).T).view(T, H, V)
    o = retention_core(q, k, v, m["decay"])
    o = rms(o, eps).reshape(T, H * V) * F.silu(h @ w[p + "g"].to(dt).T)
    return o @ w[p + "o"].to(dt).T


def expert(h, w, p, dt):
    return (F.silu(h @ w[p + "gate"].to(dt).T) * (h @ w[p + "up"].to(dt).T)) @ w[p + "down"].to(dt).T


def route(h, wr, corr, top):
    """(softmax scores [T, E], chosen experts [T, top]): chosen by score + correction."""
    s = torch.softmax(h @ wr.T, -1)
    return s, torch.topk(s + corr, top, dim=-1).indices


def moe(h, w, p, f, dt):
    top = f["router"]["top"]
    s, idx = route(h, w[p + "router"].to(dt), w[p + "correction"].to(dt), top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        sel = s[t, idx[t]]
        wt = sel / (sel.sum() + 1e-20)
        for e, a in zip(idx[t].tolist(), wt):
            out[t] += a * expert(h[t:t + 1], w, p + f"e{e}.", dt)[0]
    if f.get("shared"):
        out = out + expert(h, w, p + "shared.", dt)
    return out


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], dt=torch.float64,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence."""
    eps = cfg["norm"]["eps"]

    def ln(x, name):
        return layer_norm(x, w[name].to(dt), w[name + ".b"].to(dt), eps)

    x = ln(w["embed"].to(dt)[torch.tensor(tokens)], "embed.norm")
    X = [x]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        hin = ln(x, p + "norm1")
        if L["type"] == "parallel":
            y = parallel_mixer(hin, w, p + "mix.", L["mixer"], eps, dt)
        elif L["type"] == "retention":
            y = retention(hin, w, p + "mix.", L["mixer"], eps, dt)
        else:
            raise ValueError(L["type"])
        x = x + ln(y, p + "norm1b")
        if L.get("mlp") is not None:
            x = x + ln(moe(ln(x, p + "norm2"), w, p + "mlp.", L["mlp"], dt), p + "norm2b")
        X.append(x)
        d = w[p + "dwa"].to(dt)
        x = sum(d[j] * X[j] for j in range(i + 2))
        if layers_out is not None:
            layers_out.append(x.clone())
    z = ln(x, "final.norm") @ w["head"].to(dt).T * cfg.get("logit_scale", 1.0)
    cap = cfg.get("logit_softcap", 0.0)
    return cap * torch.tanh(z / cap) if cap else z
