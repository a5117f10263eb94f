"""Tiny Pivipel configurations for the tests, their weights, and helpers shared by the tests.

PA varies what a layer can vary: three streams, both mixers, a layer that borrows another's weights, a layer without a
feed-forward, a rotation with and without rescaled frequencies and over a part of the head, a window shorter than a
page and one longer than the prompts, kept first keys of 0, 3 and more than a window, key heads equal to the heads and
a single one, routers with and without groups, with and without a shared expert, top 1 and top 3. PB has sizes in
multiples of 16 / 32 / 64 (what the matrix-core kernels take), two streams, windows that end on and off a 64-key block.
PC has odd sizes everywhere and no ``streams`` key (one stream, the plain residual sum). PD has one stream WITH the
stream weights (``streams``: 1) and value sizes that differ from the key sizes in both directions.
"""
import json
import os
import random

import torch


def _att(heads, kv, dim, vdim, size, scale, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size}}
    if rot:
        m["rot"] = rot
    return m


def _att2(heads, kv, dim, vdim, size, keep, scale):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "mask": {"size": size, "keep_first": keep}}


def _dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _moe(experts, top, ff, limit, scale, count=None, keep=None, shared=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if count:
        r["groups"] = {"count": count, "keep": keep}
    out = {"kind": "moe", "router": r, "expert": {"ff": ff, "limit": limit}}
    if shared:
        out["shared"] = {"ff": shared[0], "limit": shared[1]}
    return out


def _layer(kind, mixer, mlp, weights_of=None):
    out = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


_SC = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}

_A1 = _att(6, 2, 12, 20, 7, 0.3, rot={"base": 100.0, "dims": 8, "scaling": _SC})
_M1 = _moe(8, 3, 24, 1.2, 2.0, 4, 3, shared=(40, 0.8))
P_A = {
    "architecture": "Pivipel", "vocab": 150, "width": 96, "max_positions": 512, "norm": {"eps": 1e-5}, "streams": 3,
    "layers": [
        _layer("attention_2", _att2(4, 4, 10, 6, 9, 3, 0.4), _dense(56, 1.5)),
        _layer("attention", _A1, _M1),
        _layer("attention_2", _att2(3, 1, 16, 8, 20, 30, 0.25), None),
        _layer("attention", _A1, _M1, weights_of=1),
        _layer("attention", _att(2, 2, 8, 8, 400, 0.35, rot={"base": 30.0, "dims": 8}), _moe(5, 1, 32, 2.0, 1.0)),
        _layer("attention_2", _att2(2, 1, 24, 12, 33, 0, 0.2), _moe(6, 2, 16, 0.7, 0.5, 2, 1, shared=(24, 1.0))),
    ],
}

P_B = {
    "architecture": "Pivipel", "vocab": 320, "width": 128, "max_positions": 1024, "norm": {"eps": 1e-6}, "streams": 2,
    "layers": [
        _layer("attention", _att(8, 2, 32, 64, 64, 0.18, rot={"base": 50000.0, "dims": 32, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 256}}),
               _moe(16, 4, 64, 1.0, 2.5, 4, 2, shared=(128, 1.0))),
        _layer("attention_2", _att2(4, 4, 64, 32, 100, 5, 0.125), _dense(256, 1.5)),
        _layer("attention_2", _att2(4, 4, 64, 32, 100, 5, 0.125), _dense(256, 1.5), weights_of=1),
        _layer("attention_2", _att2(8, 4, 16, 16, 48, 70, 0.25), _moe(8, 2, 128, 1.5, 1.0, 1, 1)),
    ],
}

P_C = {
    "architecture": "Pivipel", "vocab": 97, "width": 70, "max_positions": 300, "norm": {"eps": 1e-6},
    "layers": [
        _layer("attention", _att(5, 5, 6, 7, 11, 0.4, rot={"base": 77.0, "dims": 6}), _moe(7, 2, 10, 1.0, 3.0, 7, 3, shared=(9, 2.0))),
        _layer("attention_2", _att2(3, 1, 10, 5, 5, 2, 0.3), _dense(33, 0.9)),
        _layer("attention", _att(1, 1, 14, 9, 64, 0.27, rot={"base": 1000.0, "dims": 4, "scaling": _SC}), None),
    ],
}

P_D = {
    "architecture": "Pivipel", "vocab": 64, "width": 48, "max_positions": 256, "norm": {"eps": 1e-5}, "streams": 1,
    "layers": [
        _layer("attention_2", _att2(2, 2, 32, 8, 16, 16, 0.2), _dense(64, 1.0)),
        _layer("attention", _att(4, 2, 8, 24, 17, 0.35, rot={"base": 500.0, "dims": 8}), _moe(4, 4, 16, 1.0, 1.5, 2, 2)),
    ],
}

# name -> (config, weight seed, page size)
CONFIGS = {"PA": (P_A, 41, 8), "PB": (P_B, 42, 16), "PC": (P_C, 43, 4), "PD": (P_D, 44, 16)}


def write_model(folder, cfg, seed, std=0.09):
    """A model folder with random weights wide enough that every mechanism moves the logits: matrices N(0, std) (the
    query, key, output and down projections twice as wide), gains 1 + N(0, 0.1); the norms' slopes near 0.6 and their biases N(0, 0.1); the position table N(0, 0.3); sinks N(0.5, 1)
    (large enough to take a visible share of the denominator); the routers' weights N(0, 0.25); the gate of the shared
    expert N(0, 0.2); the streams' mixing matrices near the identity with off-diagonal entries of 0.2 in size, their
    read and write weights 1 + N(0, 0.3)."""
    from jllm_serve_amd.weights.random_init import random_source
    from jllm_serve_amd.weights.safetensors_io import write_safetensors
    src = random_source(cfg, seed, std=std)
    tensors = {n: src.get(n) for n in src.names()}
    g = torch.Generator().manual_seed(seed + 77)

    def normal(shape, mean, sd):
        return (torch.randn(shape, generator=g) * sd + mean).to(torch.bfloat16)

    for n, t in tensors.items():
        last = n.rsplit(".", 1)[-1]
        if last == "alpha":
            tensors[n] = normal(t.shape, 0.6, 0.1)
        elif n == "pos":
            tensors[n] = normal(t.shape, 0.0, 0.3)
        elif last == "sink":
            tensors[n] = normal(t.shape, 0.5, 1.0)
        elif last == "router":
            tensors[n] = normal(t.shape, 0.0, 0.25)
        elif last == "sg":
            tensors[n] = normal(t.shape, 0.0, 0.2)
        elif last in ("q", "k", "o", "down") and t.dim() == 2:
            tensors[n] = normal(t.shape, 0.0, 2 * std)  # scores with a spread; sublayers that move the stream
        elif last == "mix" and ".hc" in n:
            tensors[n] = (torch.eye(t.shape[0]) + torch.randn(t.shape, generator=g) * 0.2).to(torch.bfloat16)
        elif last in ("in", "out") and ".hc" in n:
            tensors[n] = normal(t.shape, 1.0, 0.3)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return folder


def load_weights(folder):
    """The folder's tensors through the safetensors package (not the engine's reader): floats as float64."""
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for k in f.keys():
            t = f.get_tensor(k)
            out[k] = t.to(torch.float64) if t.is_floating_point() else t
    return out


def prompt(name, length, seed=0):
    rng = random.Random(f"{name}/{length}/{seed}")
    v = CONFIGS[name][0]["vocab"]
    return [rng.randrange(v) for _ in range(length)]


def tolerance(dtype, ref):
    """Against float64, for one row. In bfloat16 a row may sit on a near-tie of the router's scores, which the rounding
    of the normed input then decides the other way: such a row is off by a part of one expert's output. So a single row
    gets a wide bound, which a wrong key, page or window edge still breaks (they move logits by their own size),
    ``typical`` bounds the median over many rows, and the float32 run, which takes the same path through cache and
    batching, is held tightly."""
    m = float(ref.abs().max())
    return 5e-5 * m + 1e-6 if dtype == "float32" else 0.2 * m


def flipped(dtype):
    """The part of a whole model's rows that may lie beyond ``tolerance``: rows whose router scores nearly tie (see
    ``tolerance``). The float32 run is held at (nearly) every row."""
    return 0.0025 if dtype == "float32" else 0.2


def typical(dtype):
    """What the median over many rows of |difference| / largest |logit| may be. (The bfloat16 bound is what the rounding
    of activations, keys and values to 8 bits of mantissa gives on these weights, whose wide query and key projections
    spread the scores; a key, page or window edge that is off moves a row by 20 % and more of its largest logit, and
    the float32 run, which walks the same path, is held a thousand times tighter.)"""
    return 5e-6 if dtype == "float32" else 4e-2
