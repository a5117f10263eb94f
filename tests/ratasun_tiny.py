"""Tiny Ratasun configurations for the tests, their weights, and helpers shared by the tests.

RA varies what a layer can vary: a loop over two middle layers, a layer without a feed-forward, a rotation over half of
the rotated key part, a delta rule with fewer key heads than value heads, state-space layers with one and with several
groups, routers with one group, with all groups kept and with a narrow choice. RB has sizes in multiples of 16 / 32 /
64 and a loop from the first layer. RC has odd sizes everywhere, no loop, one key head, convolutions of 2 and 5 taps,
top-1 routing and a logit scale of 1.
"""
import json
import os
import random

import torch


def _latent(heads, dim, rot_dim, vdim, kv_rank, dims=None, base=10000.0, scale=None):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
            "scale": scale or (dim + rot_dim) ** -0.5 * 1.4, "rot": {"base": base, "dims": dims or rot_dim}}


def _delta(heads, kv, dim, vdim, conv):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}


def _ssm(heads, vdim, state, groups, norm_groups, conv):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}


def _moe(experts, top, ff, scale, count=None, keep=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if count:
        r["groups"] = {"count": count, "keep": keep}
    return {"kind": "moe", "router": r, "expert": {"ff": ff}}


def _layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


R_A = {
    "architecture": "Ratasun", "vocab": 150, "width": 96, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
    "layers": [
        _layer("channel_delta", _delta(4, 2, 12, 8, 3), _moe(6, 2, 40, 1.5, 3, 2)),
        _layer("latent_attention", _latent(3, 12, 8, 20, 40, dims=4), _moe(8, 3, 24, 2.5, 4, 3)),
        _layer("mamba2", _ssm(6, 8, 12, 3, 2, 4), None),
        _layer("latent_attention", _latent(2, 24, 4, 8, 24, base=300.0), _moe(5, 2, 32, 1.0)),
        _layer("mamba2", _ssm(2, 20, 7, 1, 1, 2), _moe(4, 4, 16, 0.7, 2, 2)),
    ],
    "loop": {"start": 1, "stop": 3, "times": 3},
}

R_B = {
    "architecture": "Ratasun", "vocab": 320, "width": 128, "norm": {"eps": 1e-6}, "logit_scale": 2.0,
    "layers": [
        _layer("latent_attention", _latent(8, 32, 32, 32, 64, base=50000.0), _moe(8, 2, 64, 2.0, 4, 2)),
        _layer("channel_delta", _delta(4, 4, 64, 32, 4), _moe(16, 4, 64, 1.0, 4, 1)),
        _layer("mamba2", _ssm(4, 32, 64, 2, 4, 4), _moe(8, 2, 128, 1.0, 1, 1)),
    ],
    "loop": {"start": 0, "stop": 2, "times": 2},
}

R_C = {
    "architecture": "Ratasun", "vocab": 97, "width": 70, "norm": {"eps": 1e-6},
    "layers": [
        _layer("mamba2", _ssm(3, 5, 9, 3, 3, 5), _moe(3, 1, 22, 1.3)),
        _layer("latent_attention", _latent(5, 6, 6, 7, 18, dims=6, base=77.0), _moe(7, 2, 10, 3.0, 7, 3)),
        _layer("channel_delta", _delta(3, 1, 10, 7, 2), None),
        _layer("channel_delta", _delta(5, 5, 6, 9, 5), _moe(9, 3, 14, 1.1, 3, 1)),
    ],
}

# name -> (config, weight seed, page size)
CONFIGS = {"RA": (R_A, 31, 8), "RB": (R_B, 32, 16), "RC": (R_C, 33, 4)}


def write_model(folder, cfg, seed, std=0.09):
    """A model folder with random weights wide enough that every mechanism moves the logits: matrices N(0, std), gains
    1 + N(0, 0.1); convolution taps N(0, 0.5) and their biases N(0, 0.3); A_log N(0, 0.7) and dt_bias N(-1, 1) (decays
    between nearly none and strong); the skip weights 1 + N(0, 0.3); the routers' weights N(0, 0.25) and corrections
    N(0, 0.15), some of them negative enough to make choice scores negative; the loop's vectors N(0, 0.5) and its mixing
    matrix near [I | 0.5 I]."""
    from jllm_serve_amd.weights.random_init import random_source
    from jllm_serve_amd.weights.safetensors_io import write_safetensors
    src = random_source(cfg, seed, std=std)
    tensors = {n: src.get(n) for n in src.names()}
    g = torch.Generator().manual_seed(seed + 77)

    def normal(shape, mean, sd):
        return (torch.randn(shape, generator=g) * sd + mean).to(torch.bfloat16)

    for n, t in tensors.items():
        last = n.rsplit(".", 1)[-1]
        if n.endswith(".conv"):
            tensors[n] = normal(t.shape, 0.0, 0.5)
        elif n.endswith(".conv.b"):
            tensors[n] = normal(t.shape, 0.0, 0.3)
        elif last == "A_log":
            tensors[n] = normal(t.shape, 0.0, 0.7)
        elif last == "dt_bias":
            tensors[n] = normal(t.shape, -1.0, 1.0)
        elif last == "D":
            tensors[n] = normal(t.shape, 1.0, 0.3)
        elif last == "router":
            tensors[n] = normal(t.shape, 0.0, 0.25)
        elif last == "correction":
            tensors[n] = normal(t.shape, -0.3, 0.4)
        elif n == "loop.step":
            tensors[n] = normal(t.shape, 0.0, 0.5)
        elif n == "loop.in":
            w = t.shape[0]
            tensors[n] = (torch.cat([torch.eye(w), 0.5 * torch.eye(w)], dim=1) + torch.randn(t.shape, generator=g) * 0.05).to(torch.bfloat16)
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
    """Against float64, for one row. In bfloat16 a row may sit on a near-tie of the router's choice scores, which the
    rounding of the normed input then decides the other way: such a row is off by a part of one expert's output, and
    heads that are divided by their root mean square blow rounding up where they nearly cancel. So a single row gets a
    wide bound, which a wrong key, page or state still breaks (they move logits by their own size), ``typical`` bounds
    the median over many rows, and the float32 run, which takes the same path through cache, state and batching, is
    held tightly."""
    m = float(ref.abs().max())
    return 5e-5 * m + 1e-6 if dtype == "float32" else 0.2 * m


def flipped(dtype):
    """The part of a whole model's rows that may lie beyond ``tolerance``. A router's choice is a step function of its
    input: in bfloat16 the normed rows carry a rounding of a few parts in a thousand, which decides a near-tie between
    two experts, or between two groups of experts, the other way than float64 does at some rows of every routed layer,
    and such a row takes other experts from there on. Random weights (unlike trained ones) spread the choice scores
    evenly, so these rows are not rare. The float32 run, whose rounding is a hundred thousand times smaller, walks the
    same path through router, cache, state and batching and is held at (nearly) every row."""
    return 0.0025 if dtype == "float32" else 0.2


def typical(dtype):
    """What the median over many rows of |difference| / largest |logit| may be."""
    return 5e-6 if dtype == "float32" else 2.5e-2
