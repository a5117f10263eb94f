"""Kebepel on the CPU: the parser, the layer schedule of a loop, the cache groups and state of a model, the engine's
rotation table against the plain formulas, the random-weights mode, and invariants of the plain implementation that its
plausible misreadings fail."""
import json
import math
import os

import pytest
import torch

import kebepel_tiny as kt
from plain import kebepel_plain as P


def test_parser_reads_every_size_and_constant_from_the_config():
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.config.schema import GatedDeltaSpec, ParallelMixerSpec, WideAttentionSpec
    c = parse_config(kt.K_A)
    assert c.architecture == "Kebepel" and c.hidden == 96 and c.vocab == 160 and len(c.layers) == 5
    a = c.layers[0].mixer
    assert isinstance(a, WideAttentionSpec) and (a.maps, a.heads, a.kv_heads, a.dim, a.vdim) == (2, 4, 2, 12, 20)
    assert (a.diff, a.q_temp_coef, a.q_temp_every, a.position, a.softcap, a.qk_norm) == (0.25, 0.7, 5, None, 0.0, None)
    p = c.layers[1].mixer
    assert isinstance(p, ParallelMixerSpec) and p.scales == (0.6, 1.3) and p.prefixes == ("left", "right")
    left, right = p.branches
    assert (left.maps, left.softcap, left.qk_norm, left.vdim) == (1, 3.0, "whole", 24)
    rope = c.positions[left.position]
    assert (rope.rotary_dim, rope.pairing, rope.scaling.kind, rope.scaling.factor) == (8, "interleaved", "yarn", 2.0)
    assert rope.scaling.attention_factor == pytest.approx(0.1 * math.log(2.0) + 1.0)
    assert isinstance(right, GatedDeltaSpec) and (right.heads, right.kv_heads, right.dim, right.vdim, right.conv) == (4, 2, 12, 8, 3)
    assert c.layers[2].ffn is None and c.layers[0].ffn.hidden == 72 and c.layers[0].ffn.activation == "silu"
    assert c.layers[4].mixer.branches[0].position is None  # no rot: nothing is rotated
    assert c.positions[c.layers[3].mixer.branches[0].position].scaling.kind == "none"
    # the loop: layers 1 and 2 twice in a row, the pass's vector in front of its first layer only
    assert [(e.layer, e.add_before.row if e.add_before else None) for e in c.schedule] == \
        [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None), (4, None)]
    assert c.schedule[1].add_before.name == "loop.step" and c.schedule[1].add_before.rows == 2
    assert [e.layer for e in parse_config(kt.K_C).schedule] == [0, 1, 2]


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0].update(type="window"), "not a mixer of this design"),
    (lambda c: c["layers"][0]["mixer"].pop("diff"), "needs 'diff'"),
    (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=3), "do not divide"),
    (lambda c: c["layers"][1]["mixer"]["left"]["rot"].update(dims=7), "even"),
    (lambda c: c["loop"].update(stop=9), "loop runs layers"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "not a feed-forward of this design"),
])
def test_parser_refuses(change, text):
    from jllm_serve_amd.config import ConfigError, parse_config
    c = json.loads(json.dumps(kt.K_A))
    change(c)
    with pytest.raises(ConfigError, match=text):
        parse_config(c)


def test_every_run_of_a_looped_layer_has_pages_and_state_of_its_own():
    from jllm_serve_amd.cache import CacheManager
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.parts import DecoderModel
    cfg = parse_config(kt.K_A)
    model = DecoderModel(cfg, torch.float32, "cpu", 64)
    plans = model.cache_plans()
    assert len(plans) == 7 and all(p.kv is not None and p.cache_from is None for p in plans)
    # attention runs keep no state; a parallel run keeps the matrix per head and the convolutions' last inputs
    assert [p.state is None for p in plans] == [True, False, True, False, True, False, False]
    matrix, tail = plans[1].state
    assert matrix.shape == (4, 8, 12) and tail.shape == (2, 2 * 2 * 12 + 4 * 8) and matrix.dtype == torch.float32
    cm = CacheManager(plans, 8, 256, 3, allocate=False)
    # the two runs of layer 1 share a page spec (one group, two of its runs), and so do the two runs of layer 2
    runs = sorted(tuple(g.runs) for g in cm.groups)
    assert (1, 3) in runs and (2, 4) in runs and sum(len(r) for r in runs) == 7
    names = {s.name for s in model.weight_specs()}
    assert {"loop.step", "l1.mix.left.q.norm", "l1.mix.right.q.conv", "l0.mix.lq1", "l0.norm1b.b", "final.norm.b"} <= names
    assert not any(n.startswith("l2.mlp") or n.startswith("l2.norm2") for n in names)  # a layer without a feed-forward


def test_engine_rotation_table_is_the_plain_one():
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.parts.rope import rope_table
    for cfg in (kt.K_A, kt.K_B, kt.K_C):
        c = parse_config(cfg)
        for layer, raw in zip(c.layers, cfg["layers"]):
            if raw["type"] != "parallel" or "rot" not in raw["mixer"]["left"]:
                continue
            rot = raw["mixer"]["left"]["rot"]
            cos, sin = rope_table(c.positions[layer.mixer.branches[0].position], 50)
            f, amp = P.yarn_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
            ang = torch.arange(50, dtype=torch.float64)[:, None] * f[None]
            assert torch.allclose(torch.from_numpy(cos).double(), torch.cos(ang) * amp, atol=1e-6)
            assert torch.allclose(torch.from_numpy(sin).double(), torch.sin(ang) * amp, atol=1e-6)


def test_random_weights_mode_writes_what_the_model_loads(tmp_path):
    from jllm_serve_amd.weights import write_random_model
    folder = write_random_model(str(tmp_path / "m"), kt.K_C, 5)
    w = kt.load_weights(folder)
    assert w["l0.mix.right.q.conv"].shape == (10, 2) and w["l2.mix.right.b"].shape == (5, 70) and "loop.step" not in w
    logits = P.forward(kt.K_C, w, kt.prompt("KC", 9))
    assert logits.shape == (9, 97) and bool(torch.isfinite(logits).all())


# ------------------------------------------------------------------------------------------------ the plain implementation


def test_plain_convolution_is_causal_and_ends_with_the_current_token():
    x = torch.zeros(6, 1, dtype=torch.float64)
    x[2] = 1.0
    taps = torch.tensor([[2.0, 3.0, 5.0]], dtype=torch.float64)
    assert P.short_convolution(x, taps)[:, 0].tolist() == [0.0, 0.0, 5.0, 3.0, 2.0, 0.0]


def test_plain_delta_rule_stores_and_recalls():
    """Without decay and with full write strength, orthonormal keys recall their values exactly, also the first one
    after many others; writing a key again replaces its value; the read-out of a token sees that token's write."""
    torch.manual_seed(0)
    T, d, dv = 8, 8, 3
    k = torch.linalg.qr(torch.randn(d, d, dtype=torch.float64))[0][:T].unsqueeze(1)
    v = torch.randn(T, 1, dv, dtype=torch.float64)
    ones = torch.ones(T, 1, dtype=torch.float64)
    o = P.delta_rule(k, k, v, ones, ones)
    assert torch.allclose(o, v)
    q = k.clone()
    q[-1] = k[0]
    assert torch.allclose(P.delta_rule(q, k, v, ones, ones)[-1], v[0])
    k2, v2 = torch.cat([k, k[:1]]), torch.cat([v, v[:1] * 3])
    ones2 = torch.ones(T + 1, 1, dtype=torch.float64)
    assert torch.allclose(P.delta_rule(k2, k2, v2, ones2, ones2)[-1], v[0] * 3)
    g = torch.full((T, 1), 0.5, dtype=torch.float64)
    q[-1] = k[0]
    assert torch.allclose(P.delta_rule(q, k, v, ones, g)[-1], v[0] * 0.5 ** (T - 1))


def test_plain_query_temperature_steps_with_the_position():
    t = P.query_temperature(torch.arange(12), 0.5, 4)
    assert t[:3].tolist() == [1.0, 1.0, 1.0] and t[3] == pytest.approx(1 + 0.5 * math.log(2)) and t[6] == t[3]
    assert t[7] == pytest.approx(1 + 0.5 * math.log(3)) and t[11] == pytest.approx(1 + 0.5 * math.log(4))


def test_plain_pair_rotation_is_relative_and_leaves_the_tail():
    torch.manual_seed(1)
    rot = {"base": 100.0, "dims": 4}
    q, k = torch.randn(1, 1, 6, dtype=torch.float64), torch.randn(1, 1, 6, dtype=torch.float64)

    def score(pq, pk):
        return float((P.rotate_pairs(q, torch.tensor([pq]), rot) * P.rotate_pairs(k, torch.tensor([pk]), rot)).sum())
    assert score(9, 4) == pytest.approx(score(25, 20)) and score(9, 4) != pytest.approx(score(9, 5))
    assert torch.equal(P.rotate_pairs(q, torch.tensor([7]), rot)[..., 4:], q[..., 4:])
    # pairs are neighbours: a vector with only entry 0 set moves into entry 1, not into entry 2
    e = torch.zeros(1, 1, 6, dtype=torch.float64)
    e[..., 0] = 1.0
    r = P.rotate_pairs(e, torch.tensor([1]), rot)
    assert abs(float(r[..., 1])) > 0.5 and float(r[..., 2]) == 0.0


def test_plain_capped_scores_and_differential_maps():
    torch.manual_seed(2)
    T = 5
    q, k, v = (torch.randn(T, 2, 4, dtype=torch.float64) * 4 for _ in range(3))
    free = P.causal_softmax_attention(q, k, v, 1.0)
    capped = P.causal_softmax_attention(q, k, v, 1.0, softcap=0.01)
    mean = torch.cumsum(v, 0) / torch.arange(1, T + 1, dtype=torch.float64)[:, None, None]
    assert torch.allclose(capped, mean, atol=0.1) and not torch.allclose(free, mean, atol=0.5)
    # the whole model: a loop of one pass with a zero vector is no loop at all
    cfg = json.loads(json.dumps(kt.K_C))
    from jllm_serve_amd.weights.random_init import random_source
    src = random_source(cfg, 3, std=0.09)
    w = {n: src.get(n).double() for n in src.names()}
    toks = kt.prompt("KC", 11)
    base = P.forward(cfg, w, toks)
    cfg["loop"] = {"start": 0, "stop": 3, "times": 1}
    w2 = dict(w)
    w2["loop.step"] = torch.zeros(1, 70, dtype=torch.float64)
    assert torch.equal(P.forward(cfg, w2, toks), base)
    w2["loop.step"] = torch.linspace(-1, 1, 70, dtype=torch.float64)[None] ** 2  # not a constant: every layer norm removes one
    assert not torch.allclose(P.forward(cfg, w2, toks), base)
