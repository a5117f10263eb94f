"""Pivipel on the CPU: the parser, the layer schedule of borrowed weights, the pages a model asks for and how a window
with kept first keys gives pages back, the engine's rotation table against the plain formulas, the random-weights mode,
and invariants of the plain implementation that its plausible misreadings fail."""
import json
import math

import pytest
import torch

import pivipel_tiny as pt
from plain import pivipel_plain as P

F64 = torch.float64


def test_parser_reads_every_size_and_constant_from_the_config():
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.config.schema import GatedMlpSpec, RoutedMoeSpec, WideAttentionSpec
    c = parse_config(pt.P_A)
    assert c.architecture == "Pivipel" and c.hidden == 96 and c.vocab == 150 and c.streams == 3 and c.max_positions == 512
    assert c.tie_embeddings and c.embed_norm.kind == "dyntanh" and c.final_norm.kind == "dyntanh"
    assert len(c.layers) == 5, "a layer that borrows weights is a run, not a layer with tensors"
    assert [e.layer for e in c.schedule] == [0, 1, 2, 1, 3, 4] and all(e.cache_from is None for e in c.schedule)
    assert [l.prefix for l in c.layers] == ["l0", "l1", "l2", "l4", "l5"]
    assert all(l.arrangement == "hyper" and l.streams == 3 and l.norm.kind == "dyntanh" for l in c.layers)
    assert c.positions[0].kind == "learned_position" and c.positions[0].rows == 512
    a2 = c.layers[0].mixer
    assert isinstance(a2, WideAttentionSpec) and (a2.heads, a2.kv_heads, a2.dim, a2.vdim) == (4, 4, 10, 6)
    assert (a2.window, a2.keep_first, a2.scale, a2.qk_norm, a2.eps) == (9, 3, 0.4, "head", 1e-5)
    assert a2.position is None and not a2.sink and a2.out_gate and not a2.gate_per_head and not a2.bias
    a = c.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.keep_first, a.scale) == (6, 2, 12, 20, 7, 0, 0.3)
    assert a.sink and a.gate_per_head and a.qk_norm is None
    rope = c.positions[a.position]
    assert (rope.rotary_dim, rope.theta, rope.pairing, rope.scaling.kind) == (8, 100.0, "half", "llama3")
    assert (rope.scaling.factor, rope.scaling.low_freq_factor, rope.scaling.high_freq_factor,
            rope.scaling.original_max_positions) == (8.0, 1.0, 4.0, 64)
    plain_rope = c.positions[c.layers[3].mixer.position]
    assert plain_rope.scaling.kind == "none" and plain_rope.theta == 30.0 and len(c.positions) == 3
    assert c.layers[2].ffn is None and c.layers[2].mixer.keep_first == 30
    d = c.layers[0].ffn
    assert isinstance(d, GatedMlpSpec) and (d.hidden, d.activation, d.limit) == (56, "swish_clamped", 1.5)
    m = c.layers[1].ffn
    assert isinstance(m, RoutedMoeSpec) and (m.experts, m.top, m.hidden, m.limit, m.scale, m.groups, m.keep) == (8, 3, 24, 1.2, 2.0, 4, 3)
    assert (m.score, m.group_score, m.normalize, m.correction, m.activation) == ("softmax", "max", False, False, "swish_clamped")
    assert m.shared.hidden == 40 and m.shared.limit == 0.8 and m.shared_gate
    lone = c.layers[3].ffn
    assert (lone.groups, lone.keep, lone.top) == (1, 1, 1) and lone.shared is None and not lone.shared_gate
    n = parse_config(pt.P_C)
    assert n.streams == 1 and all(l.arrangement == "prenorm" for l in n.layers), "no streams key: the plain residual sum"
    one = parse_config(pt.P_D)
    assert one.streams == 1 and all(l.arrangement == "hyper" for l in one.layers), "one stream with its weights"


@pytest.mark.parametrize("change, text", [
    (lambda c: c["layers"][0].update(type="window"), "not a mixer of this design"),
    (lambda c: c["layers"][0]["mixer"].pop("vdim"), "needs 'vdim'"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=4), "do not divide"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=14), "at most dim"),
    (lambda c: c["layers"][3].update(weights_of=3), "names no layer"),
    (lambda c: c["layers"][3].update(weights_of=0), "borrows the weights"),
    (lambda c: c["layers"][0]["mlp"].update(kind="table"), "not a feed-forward of this design"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top=7"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), "3 groups"),
    (lambda c: c["layers"][1]["mlp"]["expert"].pop("limit"), "needs 'limit'"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c.update(streams=0), "streams"),
])
def test_parser_refuses(change, text):
    from jllm_serve_amd.config import ConfigError, parse_config
    c = json.loads(json.dumps(pt.P_A))
    change(c)
    with pytest.raises(ConfigError, match=text):
        parse_config(c)


def test_every_run_has_pages_of_its_own_and_the_tensors_are_the_owners():
    from jllm_serve_amd.cache import CacheManager
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.parts import DecoderModel
    model = DecoderModel(parse_config(pt.P_A), torch.float32, "cpu", 64)
    plans = model.cache_plans()
    assert len(plans) == 6 and all(p.kv is not None and p.cache_from is None and p.state is None for p in plans)
    assert [(p.kv.window, p.kv.keep_first) for p in plans] == [(9, 3), (7, 0), (20, 30), (7, 0), (400, 0), (33, 0)]
    cm = CacheManager(plans, 8, 256, 3, allocate=False)
    runs = sorted(tuple(g.runs) for g in cm.groups)
    assert (1, 3) in runs, "the layer and the run that borrows its weights hold pages of one kind, each its own"
    names = {s.name for s in model.weight_specs() if not s.optional}
    assert {"embed", "pos", "embed.norm", "embed.norm.b", "embed.norm.alpha", "final.norm.alpha", "l0.hc1.in", "l0.hc2.mix",
            "l0.mix.q.norm", "l0.mix.k.norm", "l0.mix.g", "l1.mix.sink", "l1.mlp.e7.down", "l1.mlp.router", "l1.mlp.shared.sg",
            "l1.mlp.shared.up", "l2.hc1.out", "l5.norm2.b"} <= names
    assert not any(n.startswith("l3.") for n in names), "a layer that borrows weights has no tensors"
    assert not any(n.startswith("l2.mlp") or n.startswith("l2.norm2") or n.startswith("l2.hc2") for n in names)
    assert "l4.mlp.shared.sg" not in names and "l0.mix.sink" not in names and "l1.mix.q.norm" not in names and "head" not in names
    shapes = {s.name: s.shape for s in model.weight_specs()}
    assert shapes["l1.mix.g"] == (6, 96) and shapes["l0.mix.g"] == (4 * 6, 96) and shapes["l0.hc1.mix"] == (3, 3)
    assert shapes["l0.norm1.alpha"] == () and shapes["l1.mlp.shared.sg"] == (1, 96) and shapes["pos"] == (512, 96)


def test_a_window_gives_pages_back_but_never_those_of_the_kept_first_keys():
    from jllm_serve_amd.cache import CacheManager
    from jllm_serve_amd.cache.manager import CacheEntryPlan, CacheRow, PageSpec
    rows = (CacheRow("k", (1, 4), 1), CacheRow("v", (1, 4), 1))
    plans = [CacheEntryPlan(kv=PageSpec(rows, 10, 6)), CacheEntryPlan(kv=PageSpec(rows, 10, 0)), CacheEntryPlan(kv=PageSpec(rows, 0, 0))]
    cm = CacheManager(plans, 4, 400, 2, allocate=False)
    cm.open("a")
    for n in (3, 9, 1, 1, 30, 2):
        cm.begin_write("a", n)
        cm.commit("a", n)
        cm.check()
    length = cm.length("a")
    assert length == 46
    kept, plain, full = (list(cm.requests["a"].tables[g]) for g in range(3))
    first_needed = length + 1 - 10  # the oldest key the next query sees
    assert all(p >= 0 for p in kept[:2]), "positions 0..5 lie in pages 0 and 1: they stay"
    assert all(p < 0 for p in kept[2:first_needed // 4]) and all(p >= 0 for p in kept[first_needed // 4:])
    assert all(p < 0 for p in plain[:first_needed // 4]) and all(p >= 0 for p in plain[first_needed // 4:])
    assert all(p >= 0 for p in full)
    with pytest.raises(ValueError):
        cm.truncate("a", 20)
    cm.close("a")
    cm.check()
    assert all(g.pool.used_pages == 0 for g in cm.groups)


def test_engine_rotation_table_is_the_plain_one():
    from jllm_serve_amd.config import parse_config
    from jllm_serve_amd.parts.rope import rope_table
    seen = 0
    for cfg in (pt.P_A, pt.P_B, pt.P_C, pt.P_D):
        c = parse_config(cfg)
        owners = [l for l in cfg["layers"] if "weights_of" not in l]
        for layer, raw in zip(c.layers, owners):
            rot = raw["mixer"].get("rot")
            if not rot:
                assert layer.mixer.position is None
                continue
            cos, sin = rope_table(c.positions[layer.mixer.position], 300)
            ang = torch.arange(300, dtype=F64)[:, None] * P.rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))[None]
            assert torch.allclose(torch.from_numpy(cos).double(), torch.cos(ang), atol=1e-6)
            assert torch.allclose(torch.from_numpy(sin).double(), torch.sin(ang), atol=1e-6)
            seen += 1
    assert seen >= 6


def test_plain_frequencies_are_rescaled_by_wavelength():
    sc = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    f0 = P.rotary_frequencies(16, 100.0, None)
    f = P.rotary_frequencies(16, 100.0, sc)
    wl = 2 * math.pi / f0
    assert bool((wl < 16).any()) and bool((wl > 64).any()) and bool(((wl > 16) & (wl < 64)).any()), "the test needs all three bands"
    for i in range(8):
        if wl[i] < 16:
            assert f[i] == f0[i]
        elif wl[i] > 64:
            assert abs(float(f[i]) - float(f0[i]) / 8.0) < 1e-15
        else:
            s = (64 / float(wl[i]) - 1.0) / 3.0
            assert abs(float(f[i]) - ((1 - s) * float(f0[i]) / 8.0 + s * float(f0[i]))) < 1e-15
            assert float(f0[i]) / 8.0 < float(f[i]) < float(f0[i])


def test_random_weights_mode_writes_what_the_model_loads(tmp_path):
    from jllm_serve_amd.weights import write_random_model
    folder = write_random_model(str(tmp_path / "m"), pt.P_C, 5)
    w = pt.load_weights(folder)
    assert w["l0.mix.sink"].shape == (5,) and w["l0.mix.g"].shape == (5, 70) and w["l1.mix.g"].shape == (15, 70)
    assert w["l1.mix.q.norm"].shape == (10,) and w["embed.norm.alpha"].shape == () and "l0.hc1.in" not in w and "head" not in w
    logits = P.forward(pt.P_C, w, pt.prompt("PC", 9))
    assert logits.shape == (9, 97) and bool(torch.isfinite(logits).all())
    folder = write_random_model(str(tmp_path / "s"), pt.P_A, 6)
    w = pt.load_weights(folder)
    assert float((w["l0.hc1.mix"] - torch.eye(3, dtype=F64)).abs().max()) < 0.2, "mixing matrices start near the identity"


# ------------------------------------------------------------------------------------------------ the plain implementation


def test_plain_norm_takes_no_statistics():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(3, 8, generator=g, dtype=F64)
    w, b, a = torch.randn(8, generator=g, dtype=F64), torch.randn(8, generator=g, dtype=F64), torch.tensor(0.7, dtype=F64)
    y = P.dyn_tanh(x, w, b, a)
    x2 = x.clone()
    x2[:, 3] += 100.0  # another entry of the row changes nothing elsewhere: no mean, no variance
    y2 = P.dyn_tanh(x2, w, b, a)
    keep = [i for i in range(8) if i != 3]
    assert torch.equal(y[:, keep], y2[:, keep])
    assert torch.allclose(P.dyn_tanh(torch.full((1, 8), 1e9, dtype=F64), w, b, a), (w + b)[None])
    assert torch.allclose(P.dyn_tanh(torch.zeros(1, 8, dtype=F64), w, b, a), b[None])


def test_plain_window_and_kept_first_keys():
    m = P.visible(12, 4)
    assert m[7].tolist() == [False] * 4 + [True] * 4 + [False] * 4, "itself and the three keys before it"
    m = P.visible(12, 4, 2)
    assert m[7].tolist() == [True, True, False, False] + [True] * 4 + [False] * 4
    assert m[1].tolist() == [True, True] + [False] * 10 and m[0].tolist() == [True] + [False] * 11
    assert P.visible(5, 9, 0).tolist() == torch.tril(torch.ones(5, 5)).bool().tolist()


def test_plain_sink_is_one_more_term_of_the_denominator_without_a_value():
    g = torch.Generator().manual_seed(2)
    T, H, d = 6, 2, 4
    q, k, v = (torch.randn(T, H, d, generator=g, dtype=F64) for _ in range(3))
    sink = torch.tensor([0.3, -1.2], dtype=F64)
    mask = P.visible(T, T)
    with_sink = P.attend(q, k, v, 0.5, mask, sink=sink)
    without = P.attend(q, k, v, 0.5, mask)
    for h in range(H):
        sc = torch.einsum("id,jd->ij", q[:, h], k[:, h]) * 0.5
        denom = torch.where(mask, sc.exp(), torch.zeros_like(sc)).sum(dim=1)
        share = denom / (denom + sink[h].exp())  # the sink enters as it is, one term
        assert torch.allclose(with_sink[:, h], without[:, h] * share[:, None])
    none = P.attend(q, k, v, 0.5, mask, sink=torch.tensor([-80.0, -80.0], dtype=F64))
    assert torch.allclose(none, without)


def test_plain_rotation_is_relative_pairs_the_halves_and_leaves_the_tail():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 2, 10, generator=g, dtype=F64)
    f = P.rotary_frequencies(6, 50.0, None)
    pos = torch.tensor([0, 1, 7, 8, 14])
    y = P.rotate_half(x, pos, 6, f)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0]), "the tail passes; position 0 turns nothing"
    a = float(pos[2]) * float(f[1])  # entry 1 is paired with entry 1 + 3
    assert torch.allclose(y[2, :, 1], x[2, :, 1] * math.cos(a) - x[2, :, 4] * math.sin(a))
    assert torch.allclose(y[2, :, 4], x[2, :, 4] * math.cos(a) + x[2, :, 1] * math.sin(a))
    k = torch.randn(5, 2, 10, generator=g, dtype=F64)
    s1 = (P.rotate_half(x, pos, 6, f)[2] * P.rotate_half(k, pos, 6, f)[1]).sum()
    xs, ks = x.clone(), k.clone()
    xs[4], ks[3] = x[2], k[1]  # the same vectors at positions 14 and 8 instead of 7 and 1: the same distance
    s2 = (P.rotate_half(xs, pos, 6, f)[4] * P.rotate_half(ks, pos, 6, f)[3]).sum()
    assert abs(float(s1 - s2)) < 1e-12


def test_plain_gates_one_per_head_and_one_per_channel(tmp_path):
    folder = pt.write_model(str(tmp_path / "m"), pt.P_A, 3)
    w = pt.load_weights(folder)
    g = torch.Generator().manual_seed(4)
    h = torch.randn(7, 96, generator=g, dtype=F64)
    pos = torch.arange(7)
    m1 = pt.P_A["layers"][1]["mixer"]
    w1 = P.sub(w, "l1.mix.")
    base = P.sink_attention(h, m1, w1, pos)
    w1z = dict(w1)
    w1z["g"] = w1["g"].clone()
    w1z["g"][2] = 0.0  # head 2's gate becomes sigmoid(0) = 1/2 for the whole head
    w1o = dict(w1z)
    w1o["o"] = w1["o"].clone()
    w1o["o"][:, :2 * 20] = 0.0
    w1o["o"][:, 3 * 20:] = 0.0  # only head 2 reaches the output
    only = P.sink_attention(h, m1, w1o, pos)
    gate = torch.sigmoid(P.linear(h, w1["g"]))[:, 2]
    w1b = dict(w1o)
    w1b["g"] = w1["g"]
    assert torch.allclose(P.sink_attention(h, m1, w1b, pos), only * (gate / 0.5)[:, None])
    assert base.shape == (7, 96)
    m0 = pt.P_A["layers"][0]["mixer"]
    w0 = P.sub(w, "l0.mix.")
    assert w0["g"].shape == (4 * 6, 96) and w1["g"].shape == (6, 96)
    w0z = dict(w0)
    w0z["g"] = torch.zeros_like(w0["g"])
    w0z["g"][5] = w0["g"][5]  # one channel keeps its gate, all others sit at 1/2
    a, b = P.normed_attention(h, m0, w0, 1e-5), P.normed_attention(h, m0, w0z, 1e-5)
    assert not torch.allclose(a, b)


def test_plain_clamped_gate():
    w = {"gate": torch.eye(3, dtype=F64), "up": torch.eye(3, dtype=F64), "down": torch.eye(3, dtype=F64)}
    h = torch.tensor([[5.0, -5.0, 0.5]], dtype=F64)
    y = P.clamped_ff(h, w, 2.0)
    g = torch.tensor([2.0, -5.0, 0.5], dtype=F64)  # the gate is capped above only
    u = torch.tensor([2.0, -2.0, 0.5], dtype=F64)  # the up branch on both sides
    assert torch.allclose(y[0], g * torch.sigmoid(1.702 * g) * (u + 1.0))


def test_plain_router_softmax_groups_by_their_best_and_keeps_the_scores():
    r = {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 1}}
    # the best single expert is in group 0; group 2 has the two next best: the best member decides, not a sum
    z = torch.tensor([[3.0, -9.0, 0.0, 0.0, 2.5, 2.4]], dtype=F64)
    chosen, weights = P.route(z, r)
    assert chosen.tolist() == [[0, 1]], "only group 0 is open, so its second expert is taken although it scores least"
    s = torch.softmax(z, dim=-1)
    assert torch.allclose(weights, s[:, [0, 1]] * 2.0), "the scores as they are, times the scale: not renormalised"
    r2 = {"experts": 6, "top": 3, "scale": 1.0, "groups": {"count": 3, "keep": 2}}
    chosen, weights = P.route(z, r2)
    assert chosen.tolist() == [[0, 4, 5]] and abs(float(weights.sum()) - float(s[0, [0, 4, 5]].sum())) < 1e-12
    r3 = {"experts": 6, "top": 2}
    chosen, weights = P.route(z, r3)
    assert chosen.tolist() == [[0, 4]] and torch.allclose(weights, s[:, [0, 4]])
    tie = torch.zeros(1, 6, dtype=F64)
    assert P.route(tie, r2)[0].tolist() == [[0, 1, 2]], "the lowest index among equals, for groups and experts"


def test_plain_shared_expert_is_weighed_per_token(tmp_path):
    folder = pt.write_model(str(tmp_path / "m"), pt.P_A, 3)
    w = P.sub(pt.load_weights(folder), "l1.mlp.")
    mlp = pt.P_A["layers"][1]["mlp"]
    g = torch.Generator().manual_seed(5)
    h = torch.randn(4, 96, generator=g, dtype=F64)
    full = P.expert_mix(h, mlp, w)
    no_shared = P.expert_mix(h, {k: v for k, v in mlp.items() if k != "shared"}, w)
    ws = {k: w[f"shared.{k}"] for k in ("gate", "up", "down")}
    gate = torch.sigmoid(P.linear(h, w["shared.sg"]))
    assert gate.shape == (4, 1)
    assert torch.allclose(full - no_shared, P.clamped_ff(h, ws, mlp["shared"]["limit"]) * gate)


def test_plain_streams(tmp_path):
    g = torch.Generator().manual_seed(6)
    xs = torch.randn(3, 4, 5, generator=g, dtype=F64)
    y = torch.randn(4, 5, generator=g, dtype=F64)
    mix = torch.randn(3, 3, generator=g, dtype=F64)
    out = torch.randn(3, generator=g, dtype=F64)
    new = P.streams_write(xs, y, mix, out)
    assert torch.allclose(new[1], mix[0, 1] * xs[0] + mix[1, 1] * xs[1] + mix[2, 1] * xs[2] + out[1] * y), "mix: row = the stream read, column = the stream written"
    assert torch.allclose(P.streams_read(xs, torch.tensor([1.0, 0.0, 2.0], dtype=F64)), xs[0] + 2 * xs[2])
    # identity mixing, every stream read and written with weight 1 / streams resp. 1: the plain residual sum
    folder = pt.write_model(str(tmp_path / "m"), pt.P_D, 7)
    w = pt.load_weights(folder)
    for k in w:
        if k.endswith(".mix") and ".hc" in k:
            w[k] = torch.eye(1, dtype=F64)
        elif ".hc" in k:
            w[k] = torch.ones(1, dtype=F64)
    plain_cfg = {k: v for k, v in pt.P_D.items() if k != "streams"}
    toks = pt.prompt("PD", 12)
    assert torch.allclose(P.forward(pt.P_D, w, toks), P.forward(plain_cfg, w, toks))


def test_plain_borrowed_weights_run_as_a_layer_of_their_own(tmp_path):
    folder = pt.write_model(str(tmp_path / "m"), pt.P_A, 3)
    w = pt.load_weights(folder)
    toks = pt.prompt("PA", 20)
    seen = []
    P.forward(pt.P_A, w, toks, watch=lambda i, x: seen.append(x.clone()))
    assert len(seen) == 6
    own = json.loads(json.dumps(pt.P_A))
    del own["layers"][3]["weights_of"]
    w2 = dict(w)
    for k, v in w.items():
        if k.startswith("l1."):
            w2["l3." + k[3:]] = v
    assert torch.equal(P.forward(own, w2, toks), P.forward(pt.P_A, w, toks))


def test_plain_logits_of_a_position_depend_on_earlier_tokens_only(tmp_path):
    folder = pt.write_model(str(tmp_path / "m"), pt.P_A, 3)
    w = pt.load_weights(folder)
    toks = pt.prompt("PA", 30)
    a = P.forward(pt.P_A, w, toks)
    b = P.forward(pt.P_A, w, toks[:17] + [(t + 1) % 150 for t in toks[17:]])
    assert torch.equal(a[:17], b[:17]) and not torch.allclose(a[17:], b[17:])
    tied = P.forward(pt.P_A, w, toks[:3])
    assert tied.shape == (3, 150), "the head is the embedding table"
