"""Plain, slow Zasapel forward written from the design's equations: one function
per mechanism, whole sequences at a time, no cache and no batching.  It shares
no code with the package; the tests compare the engine's kernels, state manager
and scheduler against it.

Weights are a dict name -> tensor with the checkpoint's names (``embed``,
``l<i>.norm1``, ``l<i>.mix.dq`` ...); ``cfg`` is the parsed config.json dict.
Everything is computed in ``dt`` (float64 by default).
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_plain(x, w, eps):
    return rms_unit(x, eps) * w


def norm_zero_centered(x, w, eps):
    return rms_unit(x, eps) * (1.0 + w)


def sin_positions(n: int, width: int, dt) -> torch.Tensor:
    out = torch.zeros(n, width, dtype=dt)
    p = torch.arange(n, dtype=dt)
    for e in range(width):
        i = e // 2
        ang = p * (10000.0 ** (-2.0 * i / width))
        out[:, e] = torch.sin(ang) if e % 2 == 0 else torch.cos(ang)
    return out


def causal_conv(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """h [T, C], w [C, taps]; out_t = sum_j w[:, j] * h_(t - taps + 1 + j)."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros_like(h)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def mingru(h, W, pre):
    z = torch.sigmoid(h @ W[pre + "z"].T + W[pre + "z.b"])
    u = h @ W[pre + "x"].T + W[pre + "x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = h @ W[pre + "g"].T
    S = torch.zeros(z.shape[1], dtype=h.dtype)
    ys = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        ys.append(S * (g[t] * torch.sigmoid(g[t])))
    return torch.stack(ys) @ W[pre + "o"].T


def latent_of(h, W, pre, eps):
    return norm_plain(h @ W[pre + "dkv"].T, W[pre + "dkv.norm"], eps)


def latent_attention(h, c, W, pre, m, eps):
    """c: the latents this layer attends over (its own or another layer's)."""
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    cq = norm_plain(h @ W[pre + "dq"].T, W[pre + "dq.norm"], eps)
    q = (cq @ W[pre + "uq"].T).view(T, H, D)
    k = (c @ W[pre + "uk"].T).view(T, H, D)
    v = (c @ W[pre + "uv"].T).view(T, H, V)
    gate = torch.sigmoid(h @ W[pre + "g"].T)            # [T, H]
    out = torch.zeros(T, H, V, dtype=h.dtype)
    for i in range(T):
        for hd in range(H):
            s = (k[: i + 1, hd] @ q[i, hd]) * m["scale"]
            p = torch.softmax(s, 0)
            out[i, hd] = (p[:, None] * v[: i + 1, hd]).sum(0) * gate[i, hd]
    return out.reshape(T, H * V) @ W[pre + "o"].T


def polynorm(z, coef, eps):
    a, b, c, e = [float(x) for x in coef]
    return a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e


def dense_ff(h, W, pre, eps):
    return polynorm(h @ W[pre + "up"].T, W[pre + "act"], eps) @ W[pre + "down"].T


def expert_ff(x, W, pre, limit):
    g = torch.clamp(x @ W[pre + "gate"].T, max=limit)
    u = torch.clamp(x @ W[pre + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ W[pre + "down"].T


def moe_ff(h, W, pre, mlp):
    E, top, limit = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["limit"]
    s = torch.sigmoid(h @ W[pre + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            out[t] += expert_ff((s[t, e] * h[t])[None], W, f"{pre}e{e}.", limit)[0]
    return out


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dt=torch.float64,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence."""
    W = {k: (v.to(dt) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, alpha, width = cfg["norm"]["eps"], cfg["postln_alpha"], cfg["width"]
    T = len(tokens)
    x = W["embed"][torch.tensor(tokens)] + sin_positions(T, width, dt)
    latents = {}
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = x + causal_conv(x, W[p + "canon1"])
        if L["type"] == "mingru":
            y = mingru(h, W, p + "mix.")
        else:
            m = L["mixer"]
            if "kv_from" in m and m["kv_from"] is not None:
                c = latents[m["kv_from"]]
            else:
                c = latents[i] = latent_of(h, W, p + "mix.", eps)
            y = latent_attention(h, c, W, p + "mix.", m, eps)
        x = norm_zero_centered(alpha * x + y, W[p + "norm1"], eps)
        if L.get("mlp") is not None:
            h = x + causal_conv(x, W[p + "canon2"])
            y = dense_ff(h, W, p + "mlp.", eps) if L["mlp"]["kind"] == "dense" else moe_ff(h, W, p + "mlp.", L["mlp"])
            x = norm_zero_centered(alpha * x + y, W[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_zero_centered(x, W["final.norm"], eps) @ W["head"].T
