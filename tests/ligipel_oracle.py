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


def window_attention(h, w, p, m, dt):
    """Sliding window, log-distance bias, softmax with a zero-score sink, heads' weights mixed."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    win, scale = m["mask"]["size"], m["scale"]
    q = (h @ w[p + "q"].to(dt).T).view(T, H, D)
    k = (h @ w[p + "k"].to(dt).T).view(T, G, D)
    v = (h @ w[p + "v"].to(dt).T).view(T, G, V)
    r1, r2, talk = w[p + "r1"].to(dt), w[p + "r2"].to(dt), w[p + "talk"].to(dt)
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
    return out.reshape(T, H * V) @ w[p + "o"].to(dt).T


def mamba(h, w, p, m, dt):
    T = h.shape[0]
    C, N, R, taps = m["inner"], m["state"], m["dt_rank"], m["conv"]
    xz = h @ w[p + "in"].to(dt).T
    x, z = xz[:, :C], xz[:, C:]
    cw, cb = w[p + "conv"].to(dt), w[p + "conv.b"].to(dt)
    xp = torch.cat([torch.zeros(taps - 1, C, dtype=dt), x])
    xc = torch.zeros(T, C, dtype=dt)
    for t in range(T):
        xc[t] = (xp[t:t + taps] * cw.T).sum(0) + cb
    xc = F.silu(xc)
    dbc = xc @ w[p + "x"].to(dt).T
    dlt = F.softplus(dbc[:, :R] @ w[p + "dt"].to(dt).T + w[p + "dt.b"].to(dt))
    B, Cm = dbc[:, R:R + N], dbc[:, R + N:R + 2 * N]
    A = -torch.exp(w[p + "A_log"].to(dt))
    S = torch.zeros(C, N, dtype=dt)
    y = torch.zeros(T, C, dtype=dt)
    for t in range(T):
        S = torch.exp(dlt[t][:, None] * A) * S + (dlt[t] * xc[t])[:, None] * B[t][None, :]
        y[t] = S @ Cm[t] + w[p + "D"].to(dt) * xc[t]
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


def retention(h, w, p, m, eps, dt):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rotate((h @ w[p + "q"].to(dt).T).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"], dt)
    k = rotate((h @ w[p + "k"].to(dt).T).view(T, H, D), pos, m["rot"]["dims"], m["rot"]["base"], dt) * D ** -0.5
    v = (h @ w[p + "v"].to(dt).T).view(T, H, V)
    o = torch.zeros(T, H, V, dtype=dt)
    for hh in range(H):
        S = torch.zeros(D, V, dtype=dt)
        for t in range(T):
            S = m["decay"][hh] * S + k[t, hh][:, None] * v[t, hh][None, :]
            o[t, hh] = S.T @ q[t, hh]
    o = rms(o, eps).reshape(T, H * V) * F.silu(h @ w[p + "g"].to(dt).T)
    return o @ w[p + "o"].to(dt).T


def expert(h, w, p, dt):
    return (F.silu(h @ w[p + "gate"].to(dt).T) * (h @ w[p + "up"].to(dt).T)) @ w[p + "down"].to(dt).T


def moe(h, w, p, f, dt):
    E, top = f["router"]["experts"], f["router"]["top"]
    s = torch.softmax(h @ w[p + "router"].to(dt).T, -1)
    choice = s + w[p + "correction"].to(dt)
    idx = torch.topk(choice, top, dim=-1).indices
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
    z = ln(x, "final.norm") @ w["head"].to(dt).T * cfg["logit_scale"]
    cap = cfg["logit_softcap"]
    return cap * torch.tanh(z / cap)
