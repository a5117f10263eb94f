"""A plain, slow Ratasun forward pass: whole sequences, no cache, one function per mechanism.

Ratasun is a decoder-only design whose layers read one layer norm (a weight, no bias) and add a mixer and a routed
mixture of experts, both computed from that one normed input, into the stream. The mixers: a latent attention (keys and
values rebuilt per head from one cached low-rank latent plus one rotated key part that all heads share), a delta rule
whose state decays per key channel, and a Mamba-2 state-space layer. A run of layers may be repeated with one set of
weights; before every pass the stream is mixed with the embedding output by a [width, 2 width] matrix and a learned
vector joins it. This file shares no code with the engine. Everything is torch on the CPU in the dtype of its inputs
(tests use float64). The config is the raw config.json dict, read here independently of the engine's parser.

Notation: h is a sublayer's input [T, width]; W are stored [out, in] and applied as W h.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    return torch.einsum("tc,rc->tr", x, w)


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(mean of squared deviations + eps) * w over the last axis."""
    mu = x.mean(dim=-1, keepdim=True)
    var = ((x - mu) ** 2).mean(dim=-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ----------------------------------------------------------------------------------------------- rotation


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, ..., n]: entries 2i and 2i + 1 (i < dims / 2) of the last axis turn by the angle p * base^(-2i / dims);
    entries from dims on pass unchanged."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    a = positions.to(torch.float64)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(a).to(x.dtype).view(shape), torch.sin(a).to(x.dtype).view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ----------------------------------------------------------------------------------------------- short convolution


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, K - 1 - j] x[t - j, c] (+ bias[c]), zeros before the start."""
    T, C = x.shape
    K = taps.shape[1]
    y = torch.zeros_like(x)
    for j in range(K):
        if j < T:
            y[j:] += x[:T - j] * taps[:, K - 1 - j]
    return y if bias is None else y + bias


# ----------------------------------------------------------------------------------------------- mixers


def latent_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float, positions: torch.Tensor):
    T = h.shape[0]
    H, dim, rd, vd, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = linear(h, w["q"]).view(T, H, dim + rd)
    dkv = linear(h, w["dkv"])
    c = rms(dkv[:, :R], eps) * w["dkv.norm"]
    kr = dkv[:, R:]
    ku = linear(c, w["uk"]).view(T, H, dim)
    v = linear(c, w["uv"]).view(T, H, vd)
    dims, base = int(m["rot"]["dims"]), float(m["rot"]["base"])
    qr = rotate_pairs(q[:, :, dim:], positions, dims, base)
    kr = rotate_pairs(kr, positions, dims, base)
    scores = (torch.einsum("thd,jhd->htj", q[:, :, :dim], ku) + torch.einsum("thd,jd->htj", qr, kr)) * float(m["scale"])
    mask = positions[None, :] <= positions[:, None]
    scores = scores.masked_fill(~mask[None], float("-inf"))
    p = torch.softmax(scores, dim=-1)
    o = torch.einsum("htj,jhd->thd", p, v).reshape(T, H * vd)
    return linear(o, w["o"])


def channel_delta(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float):
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(linear(h, w["q"]), w["q.conv"])).view(T, G, dk)
    k = silu(causal_conv(linear(h, w["k"]), w["k.conv"])).view(T, G, dk)
    v = silu(causal_conv(linear(h, w["v"]), w["v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(linear(h, w["b"]))  # [T, H]
    a = linear(linear(h, w["a1"]), w["a2"]) + w["dt_bias"]
    g = torch.exp(-torch.exp(w["A_log"])[None, :, None] * softplus(a).view(T, H, dk))  # [T, H, dk]
    gate = torch.sigmoid(linear(linear(h, w["g1"]), w["g2"])).view(T, H, dv)
    per = H // G
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(dk, dv, dtype=h.dtype)
        kh = hd // per
        for t in range(T):
            S = g[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            out[t, hd] = S.T @ q[t, kh]
    out = rms(out, eps) * w["norm"] * gate
    return linear(out.reshape(T, H * dv), w["o"])


def mamba2(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float):
    T = h.shape[0]
    H, P, N, G, NG = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * P
    y = linear(h, w["in"])
    z, xbc, dt = y[:, :inner], y[:, inner:2 * inner + 2 * G * N], y[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w["conv"], w["conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w["dt_bias"])  # [T, H]
    dA = torch.exp(-torch.exp(w["A_log"])[None, :] * dt)
    per = H // G
    out = torch.zeros(T, H, P, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(N, P, dtype=h.dtype)
        gr = hd // per
        for t in range(T):
            S = dA[t, hd] * S + dt[t, hd] * torch.outer(B[t, gr], x[t, hd])
            out[t, hd] = S.T @ C[t, gr] + w["D"][hd] * x[t, hd]
    o = out.reshape(T, inner) * silu(z)
    o = rms(o.view(T, NG, inner // NG), eps).reshape(T, inner) * w["norm"]
    return linear(o, w["o"])


# ----------------------------------------------------------------------------------------------- feed-forward


def route(h: torch.Tensor, r: dict, w_router: torch.Tensor, correction: torch.Tensor):
    """Chosen experts [T, top] and their weights [T, top]."""
    E, top = r["experts"], r["top"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    count, keep = int(groups["count"]), int(groups["keep"])
    s = torch.sigmoid(linear(h, w_router))
    choice = s + correction
    T = h.shape[0]
    per = E // count
    grouped = choice.view(T, count, per)
    score = grouped.topk(min(2, per), dim=-1).values.sum(-1)  # [T, count]
    best = score.topk(keep, dim=-1).indices
    allowed = torch.zeros(T, count, dtype=torch.bool)
    allowed.scatter_(1, best, True)
    masked = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(T, E)
    chosen = masked.topk(top, dim=-1).indices
    sc = s.gather(1, chosen)
    weights = sc / (sc.sum(-1, keepdim=True) + 1e-20) * float(r["scale"])
    return chosen, weights


def moe(h: torch.Tensor, mlp: dict, w: Dict[str, torch.Tensor]):
    r = mlp["router"]
    chosen, weights = route(h, r, w["router"], w["correction"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t].tolist(), weights[t]):
            x = h[t:t + 1]
            y = linear(silu(linear(x, w[f"e{e}.gate"])) * linear(x, w[f"e{e}.up"]), w[f"e{e}.down"])
            out[t] += wt * y[0]
    return out


def mixer(h: torch.Tensor, weights: Dict[str, torch.Tensor], i: int, layer: dict, eps: float, positions: torch.Tensor):
    """Layer i's mixer alone on the input rows h of one sequence."""
    mw = _sub(weights, f"l{i}.mix.")
    kind = layer["type"]
    if kind == "latent_attention":
        return latent_attention(h, layer["mixer"], mw, eps, positions)
    if kind == "channel_delta":
        return channel_delta(h, layer["mixer"], mw, eps)
    if kind == "mamba2":
        return mamba2(h, layer["mixer"], mw, eps)
    raise ValueError(kind)


# ----------------------------------------------------------------------------------------------- the model


def _sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def layer_runs(cfg: dict) -> List[tuple]:
    """(layer, pass or None, first of its pass) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, None, False) for i in range(start)]
    for t in range(times):
        runs += [(i, t, i == start) for i in range(start, stop)]
    return runs + [(i, None, False) for i in range(stop, n)]


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=torch.float64, streams: Optional[list] = None):
    """Logits [T, vocab] of one sequence from position 0. ``streams``: a list that gets the stream after every layer
    run."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(cfg["norm"]["eps"])
    ids = torch.tensor(tokens, dtype=torch.long)
    positions = torch.arange(len(tokens))
    x0 = W["embed"][ids]
    x = x0.clone()
    for i, t, first in layer_runs(cfg):
        if first:
            x = linear(torch.cat([x, x0], dim=-1), W["loop.in"]) + W["loop.step"][t]
        layer = cfg["layers"][i]
        h = layer_norm(x, W[f"l{i}.norm1"], eps)
        y = mixer(h, W, i, layer, eps, positions)
        if layer.get("mlp") is not None:
            y = y + moe(h, layer["mlp"], _sub(W, f"l{i}.mlp."))
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    xn = layer_norm(x, W["final.norm"], eps)
    return linear(xn, W["head"]) * float(cfg.get("logit_scale", 1.0))


def greedy(cfg: dict, weights: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    """The n_new tokens that follow the prompt when the largest logit (the lowest index among equals) is always taken."""
    toks = list(prompt)
    for _ in range(n_new):
        row = forward(cfg, weights, toks)[-1]
        toks.append(int(torch.argmax(row)))
    return toks[len(prompt):]
