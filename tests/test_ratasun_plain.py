"""Ratasun on the CPU: the parser, the layer schedule of a loop, the pages and state a model asks for, the engine's
rotation table against the plain formulas, the random-weights mode, and invariants of the plain implementation that its
plausible misreadings fail."""
import json
import math

import pytest
import torch

import ratasun_tiny as rt
from plain import ratasun_plain as P

F64 = torch.float64


def test_parser_reads_every_size_and_constant_from_the_config():
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.config.schema import GatedDeltaSpec, LatentAttentionSpec, RoutedMoeSpec, StateSpaceSpec
    c = parse_config(rt.R_A)
    assert c.architecture == "Ratasun" and c.hidden == 96 and c.vocab == 150 and len(c.layers) == 5 and c.logit_scale == 0.5
    assert all(l.arrangement == "parallel" and l.norm.kind == "layernorm" and not l.norm.bias and l.norm.eps == 1e-5 for l in c.layers)
    d = c.layers[0].mixer
    assert isinstance(d, GatedDeltaSpec) and (d.heads, d.kv_heads, d.dim, d.vdim, d.conv) == (4, 2, 12, 8, 3)
    assert (d.decay, d.gate_fn, d.eps) == ("channel", "sigmoid", 1e-5) and d.decay_rank != 0 and d.gate_rank != 0
    a = c.layers[1].mixer
    assert isinstance(a, LatentAttentionSpec) and (a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.q_rank) == (3, 12, 8, 20, 40, 0)
    assert a.window == 0 and not a.sink and not a.out_gate and a.scale == rt.R_A["layers"][1]["mixer"]["scale"]
    rope = c.positions[a.position]
    assert (rope.rotary_dim, rope.theta, rope.pairing) == (4, 10000.0, "interleaved")
    assert c.positions[c.layers[3].mixer.position].theta == 300.0 and len(c.positions) == 2
    s = c.layers[2].mixer
    assert isinstance(s, StateSpaceSpec) and (s.heads, s.vdim, s.state, s.groups, s.norm_groups, s.conv) == (6, 8, 12, 3, 2, 4)
    assert c.layers[2].ffn is None
    m = c.layers[1].ffn
    assert isinstance(m, RoutedMoeSpec) and (m.experts, m.top, m.hidden, m.scale, m.groups, m.keep) == (8, 3, 24, 2.5, 4, 3)
    assert (c.layers[3].ffn.groups, c.layers[3].ffn.keep) == (1, 1), "no groups: one group that is kept"
    # the loop: layers 1 and 2 three times in a row; the mix with the embedding output and the pass's vector in front
    # of a pass's first layer only
    assert [(e.layer, e.add_before.row if e.add_before else None, e.mix_before is not None) for e in c.schedule] == \
        [(0, None, False), (1, 0, True), (2, None, False), (1, 1, True), (2, None, False), (1, 2, True), (2, None, False),
         (3, None, False), (4, None, False)]
    assert c.schedule[1].add_before.name == "loop.step" and c.schedule[1].add_before.rows == 3 and c.schedule[1].mix_before.name == "loop.in"
    b = parse_config(rt.R_B)
    assert [e.layer for e in b.schedule] == [0, 1, 0, 1, 2] and b.schedule[0].mix_before is not None and b.logit_scale == 2.0
    n = parse_config(rt.R_C)
    assert [e.layer for e in n.schedule] == [0, 1, 2, 3] and n.logit_scale == 1.0
    assert all(e.mix_before is None and e.add_before is None for e in n.schedule)


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0].update(type="window"), "not a mixer of this design"),
    (lambda c: c["layers"][0]["mixer"].pop("conv"), "needs 'conv'"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "do not divide"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "at most rot_dim"),
    (lambda c: c["layers"][2]["mixer"].update(groups=4), "do not divide"),
    (lambda c: c["layers"][2]["mixer"].update(norm_groups=5), "norm_groups"),
    (lambda c: c["loop"].update(stop=9), "loop runs layers"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "not a feed-forward of this design"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top=7"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), "experts in 3 groups"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_parser_refuses(change, text):
    from jllm_serve_amd.config import ConfigError, parse_config
    c = json.loads(json.dumps(rt.R_A))
    change(c)
    with pytest.raises(ConfigError, match=text):
        parse_config(c)


def test_every_run_of_a_looped_layer_has_pages_and_state_of_its_own():
    from jllm_serve_amd.cache import CacheManager
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.parts import DecoderModel
    cfg = parse_config(rt.R_A)
    model = DecoderModel(cfg, torch.float32, "cpu", 64)
    plans = model.cache_plans()
    assert len(plans) == 9 and all(p.cache_from is None for p in plans)
    # the attention runs have pages and no state, the recurrent runs a state and no pages
    assert [p.kv is not None for p in plans] == [False, True, False, True, False, True, False, True, False]
    assert [p.state is not None for p in plans] == [True, False, True, False, True, False, True, False, True]
    matrix, tail = plans[0].state  # the delta rule: S per head, the last conv - 1 inputs of q | k | v
    assert matrix.shape == (4, 8, 12) and tail.shape == (2, 2 * 2 * 12 + 4 * 8) and matrix.dtype == torch.float32
    matrix, tail = plans[2].state  # the state-space layer: S per head, the last conv - 1 inputs of x | B | C
    assert matrix.shape == (6, 8, 12) and tail.shape == (3, 6 * 8 + 2 * 3 * 12) and tail.dtype == torch.float32
    cm = CacheManager(plans, 8, 256, 3, allocate=False)
    runs = sorted(tuple(g.runs) for g in cm.groups)
    assert (1, 3, 5) in runs, "the three passes of layer 1 have pages of their own of one kind"
    names = {s.name for s in model.weight_specs()}
    assert {"loop.step", "loop.in", "l0.mix.q.conv", "l0.mix.a1", "l0.mix.g2", "l1.mix.dkv.norm", "l1.mlp.e7.down", "l1.mlp.correction",
            "l2.mix.conv.b", "l2.mix.D", "final.norm", "head", "embed"} <= names
    assert not any(n.startswith("l2.mlp") for n in names), "a layer without a feed-forward"
    assert not any(n.endswith("norm1.b") or n == "final.norm.b" for n in names), "the layer norms have no bias"
    free = {s.name: s.shape for s in model.weight_specs() if -1 in s.shape}
    assert set(free) == {"l0.mix.a1", "l0.mix.a2", "l0.mix.g1", "l0.mix.g2"}, "the narrow middles are the checkpoint's to size"


def test_engine_rotation_table_is_the_plain_one():
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.parts.rope import rope_table
    for cfg in (rt.R_A, rt.R_B, rt.R_C):
        c = parse_config(cfg)
        for layer, raw in zip(c.layers, cfg["layers"]):
            if raw["type"] != "latent_attention":
                continue
            rot = raw["mixer"]["rot"]
            cos, sin = rope_table(c.positions[layer.mixer.position], 70)
            i = torch.arange(rot["dims"] // 2, dtype=F64)
            ang = torch.arange(70, dtype=F64)[:, None] * torch.pow(torch.tensor(rot["base"], dtype=F64), -2.0 * i / rot["dims"])[None]
            assert torch.allclose(torch.from_numpy(cos).double(), torch.cos(ang), atol=1e-6)
            assert torch.allclose(torch.from_numpy(sin).double(), torch.sin(ang), atol=1e-6)


def test_random_weights_mode_writes_what_the_model_loads(tmp_path):
    from jllm_serve_amd.weights import write_random_model
    folder = write_random_model(str(tmp_path / "m"), rt.R_C, 5)
    w = rt.load_weights(folder)
    assert w["l0.mix.conv"].shape == (3 * 5 + 2 * 3 * 9, 5) and w["l2.mix.b"].shape == (3, 70) and "loop.step" not in w
    assert w["l2.mix.a2"].shape[0] == 3 * 10 and w["l2.mix.a2"].shape[1] == w["l2.mix.a1"].shape[0]
    assert w["l1.mlp.correction"].shape == (7,) and w["l1.mix.q"].shape == (5 * 12, 70)
    logits = P.forward(rt.R_C, w, rt.prompt("RC", 9))
    assert logits.shape == (9, 97) and bool(torch.isfinite(logits).all())


# ------------------------------------------------------------------------------------------------ the plain implementation


def test_plain_convolution_is_causal_ends_with_the_current_token_and_adds_its_bias():
    x = torch.zeros(6, 1, dtype=F64)
    x[2] = 1.0
    taps = torch.tensor([[2.0, 3.0, 5.0]], dtype=F64)
    assert P.causal_conv(x, taps)[:, 0].tolist() == [0.0, 0.0, 5.0, 3.0, 2.0, 0.0]
    assert P.causal_conv(x, taps, torch.tensor([0.5], dtype=F64))[:, 0].tolist() == [0.5, 0.5, 5.5, 3.5, 2.5, 0.5]


def test_plain_pair_rotation_is_relative_and_leaves_the_tail():
    torch.manual_seed(1)
    q, k = torch.randn(1, 10, dtype=F64), torch.randn(1, 10, dtype=F64)

    def score(pq, pk):
        return float((P.rotate_pairs(q, torch.tensor([pq]), 6, 50.0) * P.rotate_pairs(k, torch.tensor([pk]), 6, 50.0)).sum())
    assert score(9, 4) == pytest.approx(score(25, 20), abs=1e-12) and abs(score(9, 4) - score(9, 5)) > 1e-3
    r = P.rotate_pairs(q, torch.tensor([7]), 6, 50.0)
    assert torch.equal(r[:, 6:], q[:, 6:]) and not torch.allclose(r[:, :6], q[:, :6])
    # neighbours turn together: the pair (0, 1) by 7 radians
    assert r[0, 0] == pytest.approx(q[0, 0] * math.cos(7) - q[0, 1] * math.sin(7))
    assert r[0, 1] == pytest.approx(q[0, 1] * math.cos(7) + q[0, 0] * math.sin(7))


def _delta_weights(H, G, dk, dv, width, taps=1):
    """Weights of a delta-rule mixer that passes chosen q, k, v through: identity-like projections and a convolution
    of one tap of weight 1, so the inputs of the recurrence are silu of the input's columns."""
    w = {}
    eye = torch.eye(width, dtype=F64)
    w["q"], w["k"], w["v"] = eye[:G * dk], eye[G * dk:2 * G * dk], eye[2 * G * dk:2 * G * dk + H * dv]
    for n, c in (("q", G * dk), ("k", G * dk), ("v", H * dv)):
        w[n + ".conv"] = torch.zeros(c, taps, dtype=F64)
        w[n + ".conv"][:, -1] = 1.0
    w["b"] = torch.zeros(H, width, dtype=F64)
    w["a1"], w["a2"] = torch.zeros(2, width, dtype=F64), torch.zeros(H * dk, 2, dtype=F64)
    w["g1"], w["g2"] = torch.zeros(2, width, dtype=F64), torch.zeros(H * dv, 2, dtype=F64)
    w["dt_bias"] = torch.full((H * dk,), -40.0, dtype=F64)  # softplus ~ 0: nothing decays
    w["A_log"] = torch.zeros(H, dtype=F64)
    w["norm"] = torch.ones(dv, dtype=F64)
    w["o"] = torch.eye(H * dv, dtype=F64)
    return w


def test_plain_delta_rule_decays_each_key_channel_by_its_own_factor():
    """One head, keys along single channels: what was written along channel i fades by that channel's factor per
    token and by no other's; the read-out sees the current token's write."""
    H = G = 1
    dk, dv, T = 4, 3, 5
    width = 2 * dk + dv
    w = _delta_weights(H, G, dk, dv, width)
    w["b"][0, 0] = 50.0  # every token's first input entry is large: beta = 1
    rates = torch.tensor([0.0, 0.3, 1.1, 2.0], dtype=F64)
    # g_i = exp(-exp(A_log) softplus(dt_bias_i)): choose dt_bias so that softplus gives the rate
    w["dt_bias"] = torch.log(torch.expm1(rates.clamp(min=1e-12)))
    big = 30.0  # silu(30) = 30: unit vectors come out exact
    h = torch.zeros(T, width, dtype=F64)
    vals = torch.tensor([[1.0, 2.0, 3.0], [2.0, -1.0, 0.5], [0.3, 0.2, 0.1]], dtype=F64)
    for t, ch in enumerate((1, 2, 3)):  # token t writes vals[t] along channel ch
        h[t, dk + ch] = big
        h[t, 2 * dk:] = vals[t]
    h[:, 0] = 1.0  # also a query entry (channel 0): harmless for the rows that only write
    # the last rows ask along channels 1 and 3
    h[3, 1], h[4, 3] = big, big
    h[3, 0] = h[4, 0] = 1.0
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "conv": 1}
    w["norm"] = torch.ones(dv, dtype=F64)
    w["g2"] = torch.zeros(H * dv, 2, dtype=F64)  # gate = sigmoid(0) = 1/2
    o = P.channel_delta(h, m, w, 0.0)
    sv = P.silu(vals)
    g = torch.exp(-rates)
    # row 3 asks along channel 1: written at t = 0, faded three times by g_1 (rows 1, 2, 3); rows 3 and 4 write nothing new
    # along the asked channels because their keys are zero vectors (k = 0 / sqrt(1e-6) = 0)
    want3 = sv[0] * g[1] ** 3
    want4 = sv[2] * g[3] ** 2
    for row, want in ((3, want3), (4, want4)):
        want = want / torch.sqrt((want * want).mean()) * 0.5
        assert torch.allclose(o[row], want, atol=1e-9), (row, o[row], want)


def test_plain_delta_rule_reads_its_own_write_and_replaces_a_value():
    H = G = 1
    dk, dv = 3, 2
    width = 2 * dk + dv
    w = _delta_weights(H, G, dk, dv, width)
    w["b"][0, :] = 0.0
    w["b"][0, 2 * dk] = 50.0  # beta = sigmoid(50 v_0): v_0 > 0 in every row below
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "conv": 1}
    h = torch.zeros(3, width, dtype=F64)
    for t, v in enumerate(([1.0, 2.0], [3.0, -1.0], [0.5, 0.25])):
        h[t, 0] = h[t, dk] = 30.0  # q and k along channel 0
        h[t, 2 * dk:] = torch.tensor(v, dtype=F64)
    o = P.channel_delta(h, m, w, 0.0)
    for t in range(3):  # with beta = 1 and a unit key, a write replaces what the key held; the row reads it back
        v = P.silu(h[t, 2 * dk:])
        want = v / torch.sqrt((v * v).mean()) * 0.5
        assert torch.allclose(o[t], want, atol=1e-6)


def test_plain_state_space_layer_is_the_sum_over_earlier_tokens():
    """y_t = sum over s <= t of (product of the decays after s) dt_s (C_t . B_s) x_s + D x_t, the gate before the norm,
    the norm in equal parts of the row."""
    torch.manual_seed(3)
    m = {"heads": 4, "vdim": 3, "state": 5, "groups": 2, "norm_groups": 3, "conv": 3}
    H, Pd, N, G = 4, 3, 5, 2
    inner, width, T = H * Pd, 16, 9
    w = {"in": torch.randn(2 * inner + 2 * G * N + H, width, dtype=F64) * 0.4, "conv": torch.randn(inner + 2 * G * N, 3, dtype=F64) * 0.5,
         "conv.b": torch.randn(inner + 2 * G * N, dtype=F64) * 0.3, "dt_bias": torch.randn(H, dtype=F64), "A_log": torch.randn(H, dtype=F64) * 0.5,
         "D": torch.randn(H, dtype=F64), "norm": torch.randn(inner, dtype=F64), "o": torch.eye(inner, dtype=F64)}
    h = torch.randn(T, width, dtype=F64)
    got = P.mamba2(h, m, w, 1e-5)
    y = P.linear(h, w["in"])
    z, xbc, dt = y[:, :inner], y[:, inner:2 * inner + 2 * G * N], y[:, 2 * inner + 2 * G * N:]
    xbc = P.silu(P.causal_conv(xbc, w["conv"], w["conv.b"]))
    x, B, C = xbc[:, :inner].view(T, H, Pd), xbc[:, inner:inner + G * N].view(T, G, N), xbc[:, inner + G * N:].view(T, G, N)
    dt = torch.log1p(torch.exp(dt + w["dt_bias"]))
    la = -torch.exp(w["A_log"])[None] * dt  # log of the decay per token and head
    out = torch.zeros(T, H, Pd, dtype=F64)
    for hd in range(H):
        gr = hd // 2
        for t in range(T):
            for s in range(t + 1):
                out[t, hd] += torch.exp(la[s + 1:t + 1, hd].sum()) * dt[s, hd] * (C[t, gr] @ B[s, gr]) * x[s, hd]
            out[t, hd] += w["D"][hd] * x[t, hd]
    o = out.reshape(T, inner) * P.silu(z)
    o = o.view(T, 3, 4)
    o = (o / torch.sqrt((o * o).mean(-1, keepdim=True) + 1e-5)).reshape(T, inner) * w["norm"]
    assert torch.allclose(got, o, atol=1e-10)


def test_plain_router_groups_correction_and_weights():
    r = {"experts": 6, "top": 2, "scale": 3.0, "groups": {"count": 3, "keep": 1}}
    w_router = torch.eye(6, dtype=F64)
    h = torch.tensor([[2.0, -9.0, 1.5, 1.4, 0.0, 0.0]], dtype=F64)
    zero = torch.zeros(6, dtype=F64)
    chosen, weights = P.route(h, r, w_router, zero)
    # group scores are sums of the two largest: (0, 1): s(2) + s(-9) = 0.88; (2, 3): s(1.5) + s(1.4) = 1.62 wins although
    # expert 0 has the largest score of all; only its group's experts can be chosen
    assert sorted(chosen[0].tolist()) == [2, 3]
    s = torch.sigmoid(h[0])
    assert torch.allclose(weights[0].sum(), torch.tensor(3.0, dtype=F64)) and weights[0, 0] / weights[0, 1] == pytest.approx(float(s[2] / s[3]))
    # the correction moves the choice and not the weights: it lifts group (4, 5); the weights are still sigmoid(0) each
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.9, 0.2], dtype=F64)
    chosen, weights = P.route(h, r, w_router, corr)
    assert chosen[0].tolist() == [4, 5] and torch.allclose(weights[0], torch.tensor([1.5, 1.5], dtype=F64))
    # negative choice scores: a closed group counts as minus infinity and not as 0, so the open group's negative
    # scores still win
    corr = torch.tensor([-3.0, -3.0, -1.2, -1.1, -3.0, -3.0], dtype=F64)
    h0 = torch.zeros(1, 6, dtype=F64)
    chosen, _ = P.route(h0, r, w_router, corr)
    assert sorted(chosen[0].tolist()) == [2, 3]
    # with every group kept the groups decide nothing
    r2 = {"experts": 6, "top": 2, "scale": 1.0, "groups": {"count": 3, "keep": 3}}
    assert sorted(P.route(h, r2, w_router, zero)[0][0].tolist()) == [0, 2]
    assert sorted(P.route(h, {"experts": 6, "top": 2, "scale": 1.0}, w_router, zero)[0][0].tolist()) == [0, 2]


def test_plain_loop_of_one_pass_that_mixes_nothing_is_no_loop(tmp_path):
    cfg = json.loads(json.dumps(rt.R_C))
    folder = rt.write_model(str(tmp_path / "a"), cfg, 3)
    w = rt.load_weights(folder)
    toks = rt.prompt("RC", 12)
    base = P.forward(cfg, w, toks)
    looped = dict(cfg, loop={"start": 1, "stop": 3, "times": 1})
    d = cfg["width"]
    w2 = dict(w)
    w2["loop.in"] = torch.cat([torch.eye(d, dtype=F64), torch.zeros(d, d, dtype=F64)], dim=1)
    w2["loop.step"] = torch.zeros(1, d, dtype=F64)
    assert torch.allclose(P.forward(looped, w2, toks), base, atol=1e-12)
    w2["loop.in"] = torch.cat([torch.eye(d, dtype=F64), 0.3 * torch.eye(d, dtype=F64)], dim=1)
    assert not torch.allclose(P.forward(looped, w2, toks), base, atol=1e-3), "the embedding output joins the stream again"
    # two passes run the looped layers twice with one set of weights: one more run per looped layer and pass
    twice = dict(cfg, loop={"start": 1, "stop": 3, "times": 2})
    assert [i for i, _, _ in P.layer_runs(twice)] == [0, 1, 2, 1, 2, 3]
    assert [f for _, _, f in P.layer_runs(twice)] == [False, True, False, True, False, False]


def test_plain_logits_of_a_position_depend_on_earlier_tokens_only(tmp_path):
    folder = rt.write_model(str(tmp_path / "a"), rt.R_A, 3)
    w = rt.load_weights(folder)
    toks = rt.prompt("RA", 20)
    a = P.forward(rt.R_A, w, toks)
    b = P.forward(rt.R_A, w, toks[:11] + [(t + 1) % 150 for t in toks[11:]])
    assert torch.allclose(a[:11], b[:11], atol=1e-12) and not torch.allclose(a[11:], b[11:], atol=1e-3)
    # every mixer carries something from the first token to the last: changing token 0 moves the last logits
    c = P.forward(rt.R_A, w, [(toks[0] + 1) % 150] + toks[1:])
    assert float((a[-1] - c[-1]).abs().max()) > 1e-4
