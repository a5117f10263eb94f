"""A plain, slow Pivipel forward pass: whole sequences, no cache, one function per mechanism.

Pivipel is a decoder-only design with a learned position table added at the input, Dynamic-Tanh norms (no statistics:
tanh(alpha x) w + b), several residual streams that every sublayer reads as one weighted sum and writes back through a
small mixing matrix (hyper-connections), two attention mixers (a rotated one with a sliding window, a learned sink in
the softmax's denominator and one output gate per head; an unrotated one with per-head q/k RMS norms, a sliding window
that also keeps the first tokens, and an output gate per channel), dense feed-forwards with a clamped gate, and
router-chosen experts (softmax scores, groups of which the best stay open, a shared expert with a gate per token). A
layer may run with another layer's weights. The head is the embedding table. This file shares no code with the engine.
Everything is torch on the CPU in the dtype of its inputs (tests use float64). The config is the raw config.json dict,
read here independently of the engine's parser.

Notation: h is a sublayer's input [T, width]; W are stored [out, in] and applied as W h.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    return torch.einsum("tc,rc->tr", x, w)


def dyn_tanh(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, alpha: torch.Tensor) -> torch.Tensor:
    """tanh(alpha x) w + b, element by element: a norm without a mean or a variance."""
    return torch.tanh(alpha * x) * w + b


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


# ----------------------------------------------------------------------------------------------- rotation


def rotary_frequencies(dims: int, base: float, scaling: Optional[dict]) -> torch.Tensor:
    """f_i = base^(-2i / dims) for i < dims / 2, rescaled by wavelength l = 2 pi / f: unchanged where l < original /
    high; f / factor where l > original / low; in between (1 - s) f / factor + s f with s = (original / l - low) /
    (high - low)."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
    if not scaling:
        return f
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.clone()
    for n in range(dims // 2):
        wl = 2.0 * math.pi / float(f[n])
        if wl < orig / high:
            continue
        if wl > orig / low:
            out[n] = f[n] / factor
        else:
            s = (orig / wl - low) / (high - low)
            out[n] = (1.0 - s) * f[n] / factor + s * f[n]
    return out


def rotate_half(x: torch.Tensor, positions: torch.Tensor, dims: int, freqs: torch.Tensor) -> torch.Tensor:
    """x [T, heads, n]: entry i and entry i + dims / 2 (i < dims / 2) turn by the angle p f_i; entries from dims on
    pass unchanged."""
    out = x.clone()
    half = dims // 2
    a = positions.to(torch.float64)[:, None] * freqs[None, :]
    c, s = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ----------------------------------------------------------------------------------------------- attention


def visible(T: int, window: int, keep_first: int = 0) -> torch.Tensor:
    """[T, T] bool: query i sees key j when j <= i and (i - j < window or j < keep_first)."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    return (j <= i) & ((i - j < window) | (j < keep_first))


def attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, mask: torch.Tensor,
           sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads key/value head h // (H / G). Scores (q . k) scale,
    softmax over the visible keys; with ``sink`` [H] the denominator also holds exp(sink_h), which has no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        sc = torch.einsum("id,jd->ij", q[:, h], k[:, g]) * scale
        sc = sc.masked_fill(~mask, float("-inf"))
        if sink is not None:
            sc = torch.cat([sc, sink[h].expand(T, 1).to(sc.dtype)], dim=1)
        p = torch.softmax(sc, dim=-1)
        out[:, h] = p[:, :T] @ v[:, g]
    return out


def sink_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], positions: torch.Tensor) -> torch.Tensor:
    """Mixer 'attention': rotation of (i, i + dims / 2) on the first rot.dims entries of every q and k head, a sliding
    window, a sink per head, one sigmoid gate per head on the head's output."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w["q"]).view(T, H, d)
    k = linear(h, w["k"]).view(T, G, d)
    v = linear(h, w["v"]).view(T, G, dv)
    rot = m.get("rot")
    if rot:
        f = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q = rotate_half(q, positions, rot["dims"], f)
        k = rotate_half(k, positions, rot["dims"], f)
    o = attend(q, k, v, m["scale"], visible(T, (m.get("mask") or {}).get("size", T)), sink=w.get("sink"))
    gate = torch.sigmoid(linear(h, w["g"]))  # [T, H]
    o = o * gate[:, :, None]
    return linear(o.reshape(T, H * dv), w["o"])


def normed_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float) -> torch.Tensor:
    """Mixer 'attention_2': RMS norm of every q and k head with one gain vector each, no rotation, a sliding window
    that also keeps the first keep_first keys, plain softmax, a sigmoid gate per channel of the concatenated heads."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms(linear(h, w["q"]).view(T, H, d), eps) * w["q.norm"]
    k = rms(linear(h, w["k"]).view(T, G, d), eps) * w["k.norm"]
    v = linear(h, w["v"]).view(T, G, dv)
    o = attend(q, k, v, m["scale"], visible(T, (m.get("mask") or {}).get("size", T), (m.get("mask") or {}).get("keep_first", 0)))
    o = o.reshape(T, H * dv) * torch.sigmoid(linear(h, w["g"]))
    return linear(o, w["o"])


# ----------------------------------------------------------------------------------------------- feed-forwards


def clamped_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], limit: float) -> torch.Tensor:
    """g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(linear(h, w["gate"]), max=limit)
    u = torch.clamp(linear(h, w["up"]), min=-limit, max=limit)
    return linear(g * torch.sigmoid(1.702 * g) * (u + 1.0), w["down"])


def route(z: torch.Tensor, r: dict):
    """z [T, E] router logits -> (chosen [T, top], weights [T, top]): s = softmax(z); the experts form groups.count
    equal groups of neighbours whose score is their largest s, only the groups.keep best are open; the top largest s
    among the open ones win (the lowest index among equals); weights are their s times router.scale."""
    T, E = z.shape
    s = torch.softmax(z, dim=-1)
    choice = s.clone()
    groups = r.get("groups")
    if groups:
        n, keep = groups["count"], groups["keep"]
        per = E // n
        gs = s.view(T, n, per).max(dim=-1).values
        open_ = torch.zeros(T, n, dtype=torch.bool)
        for t in range(T):
            left = gs[t].clone()
            for _ in range(keep):
                b = int(torch.argmax(left))  # the first of equals
                open_[t, b] = True
                left[b] = float("-inf")
        choice = choice.masked_fill(~open_.repeat_interleave(per, dim=1), float("-inf"))
    chosen = torch.zeros(T, r["top"], dtype=torch.long)
    for t in range(T):
        c = choice[t].clone()
        for n_ in range(r["top"]):
            b = int(torch.argmax(c))
            chosen[t, n_] = b
            c[b] = float("-inf")
    weights = torch.gather(s, 1, chosen) * float(r.get("scale", 1.0))
    return chosen, weights


def expert_mix(h: torch.Tensor, mlp: dict, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    """The routed experts' weighted sum plus the shared expert times sigmoid(W_sg h) (one number per token)."""
    r = mlp["router"]
    z = linear(h, w["router"])
    chosen, weights = route(z, r)
    out = torch.zeros_like(h)
    limit = mlp["expert"]["limit"]
    for t in range(h.shape[0]):
        for n in range(r["top"]):
            e = int(chosen[t, n])
            we = {k: w[f"e{e}.{k}"] for k in ("gate", "up", "down")}
            out[t] += weights[t, n] * clamped_ff(h[t:t + 1], we, limit)[0]
    if mlp.get("shared"):
        ws = {k: w[f"shared.{k}"] for k in ("gate", "up", "down")}
        out = out + clamped_ff(h, ws, mlp["shared"]["limit"]) * torch.sigmoid(linear(h, w["shared.sg"]))
    return out


def feed_forward(h: torch.Tensor, mlp: dict, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return clamped_ff(h, w, mlp["limit"])
    return expert_mix(h, mlp, w)


# ----------------------------------------------------------------------------------------------- streams


def streams_read(xs: torch.Tensor, w_in: torch.Tensor) -> torch.Tensor:
    """xs [S, T, width] -> sum_s in[s] xs[s]."""
    return torch.einsum("s,stc->tc", w_in, xs)


def streams_write(xs: torch.Tensor, y: torch.Tensor, mix: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """Every stream from the previous streams together: new[t] = sum_s mix[s, t] old[s] + out[t] y."""
    return torch.einsum("sr,stc->rtc", mix, xs) + out[:, None, None] * y[None]


# ----------------------------------------------------------------------------------------------- model


def sub(weights: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def norm_of(weights: Dict[str, torch.Tensor], name: str):
    return weights[name], weights[name + ".b"], weights[name + ".alpha"]


def forward(cfg: dict, weights: Dict[str, torch.Tensor], tokens: List[int], watch=None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0. ``watch(run, x)`` gets the sum of the streams after every
    layer run."""
    T = len(tokens)
    positions = torch.arange(T)
    eps = float(cfg["norm"]["eps"])
    x = weights["embed"][torch.tensor(tokens)] + weights["pos"][positions]
    x = dyn_tanh(x, *norm_of(weights, "embed.norm"))
    hyper = "streams" in cfg  # without the key there is one stream and the plain residual sum
    S = int(cfg.get("streams", 1))
    xs = x[None].repeat(S, 1, 1)
    for i, layer in enumerate(cfg["layers"]):
        owner = layer.get("weights_of", i)
        p = f"l{owner}."
        m = layer["mixer"]
        u = streams_read(xs, weights[p + "hc1.in"]) if hyper else xs[0]
        hn = dyn_tanh(u, *norm_of(weights, p + "norm1"))
        if layer["type"] == "attention":
            y = sink_attention(hn, m, sub(weights, p + "mix."), positions)
        elif layer["type"] == "attention_2":
            y = normed_attention(hn, m, sub(weights, p + "mix."), eps)
        else:
            raise ValueError(f"unknown mixer '{layer['type']}'")
        xs = streams_write(xs, y, weights[p + "hc1.mix"], weights[p + "hc1.out"]) if hyper else xs + y[None]
        if layer.get("mlp"):
            u = streams_read(xs, weights[p + "hc2.in"]) if hyper else xs[0]
            hn = dyn_tanh(u, *norm_of(weights, p + "norm2"))
            y = feed_forward(hn, layer["mlp"], sub(weights, p + "mlp."))
            xs = streams_write(xs, y, weights[p + "hc2.mix"], weights[p + "hc2.out"]) if hyper else xs + y[None]
        if watch is not None:
            watch(i, xs.sum(dim=0))
    x = dyn_tanh(xs.sum(dim=0), *norm_of(weights, "final.norm"))
    return linear(x, weights["embed"])
