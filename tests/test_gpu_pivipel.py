"""Pivipel on the GPU against the plain implementation (tests/plain/pivipel_plain.py): the stream kernels, the router
and the experts' sum alone, every feed-forward and every mixer alone through the cache, both attentions with one key that
decides (at the first position, just inside and just outside the kept first keys and the window, at a page's last and
first place, hundreds of keys back; as rows of portions and as single rows; on pages whose unused and given-back places
hold NaN), the streams after every layer run, whole prompts against token-by-token decoding, portions down to two tokens,
mixed batches on a pool that is used again, long decoding through captured steps until every window has passed, greedy
generation through the engine, and the replay program."""
import json
import os

import numpy as np
import pytest
import torch

import pivipel_tiny as pt
import replay
from plain import pivipel_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
F64 = torch.float64


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: pt.write_model(str(tmp_path_factory.mktemp("pivipel_" + name)), cfg, seed)
            for name, (cfg, seed, page) in pt.CONFIGS.items()}


@pytest.fixture(scope="module")
def built(folders):
    from jllm_serve_amd.engine import build_runner, load_model
    cache = {}

    def get(name, dtype, graphs=False):
        if (name, dtype, graphs) not in cache:
            longest = min(1024, pt.CONFIGS[name][0]["max_positions"])
            model = load_model(folders[name], dtype, torch.device(DEV), max_positions=longest)
            cache[(name, dtype, graphs)] = (model, build_runner(model, page_size=pt.CONFIGS[name][2], pool_tokens=1024,
                                                                max_requests=4, graphs=graphs))
        return cache[(name, dtype, graphs)]
    return get


@pytest.fixture(scope="module")
def plain_logits(folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            memo[key] = P.forward(pt.CONFIGS[name][0], pt.load_weights(folders[name]), list(tokens))
        return memo[key]
    return get


def close(got, want, dtype, what=""):
    err = float((got.double().cpu() - want).abs().max())
    assert err <= pt.tolerance(dtype, want), f"{what}: {err} > {pt.tolerance(dtype, want)}"


def act_type(dtype):
    return torch.float32 if dtype == "float32" else torch.bfloat16


def owners(cfg):
    """(config layer index, engine layer index) of the layers that have tensors of their own."""
    return [(i, n) for n, i in enumerate(i for i, l in enumerate(cfg["layers"]) if "weights_of" not in l)]


def runs(cfg):
    """Per layer run: (config layer whose tensors it uses, engine layer index)."""
    own = dict(owners(cfg))
    return [(l.get("weights_of", i), own[l.get("weights_of", i)]) for i, l in enumerate(cfg["layers"])]


# ------------------------------------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("S, width, T", [(1, 48, 5), (2, 128, 300), (3, 70, 33), (5, 1024, 7), (16, 24, 9)])
def test_stream_kernels(S, width, T):
    """The norm without statistics, read from one row or from a weighted sum of streams, over all rows or a list of
    them, written once or once per stream; the streams' update with and without the next sublayer's input."""
    from jllm_serve_amd.kernels import ops
    g = torch.Generator().manual_seed(S * 1000 + width)
    x = torch.randn(T, S, width, generator=g) * 2.0
    w, b = torch.randn(width, generator=g), torch.randn(width, generator=g) * 0.3
    alpha = torch.tensor([0.7])
    read = torch.randn(S, generator=g)
    xd = x.reshape(T, S * width).to(DEV).contiguous()
    args = (w.to(DEV), b.to(DEV), alpha.to(DEV))
    want = torch.tanh(0.7 * torch.einsum("s,tsc->tc", read.double(), x.double())) * w.double() + b.double()
    got = ops.dyntanh(xd, *args, torch.float32, streams=S, read=read.to(DEV))
    assert float((got.double().cpu() - want).abs().max()) < 2e-6
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
    got = ops.dyntanh(xd, *args, torch.bfloat16, streams=S, read=read.to(DEV), rows=rows.to(DEV))
    assert got.dtype == torch.bfloat16 and float((got.double().cpu() - want[rows.long()]).abs().max()) < 2e-2
    one = x[:, 0].contiguous().to(DEV)
    got = ops.dyntanh(one, *args, torch.float32, copies=S)
    want1 = torch.tanh(0.7 * x[:, 0].double()) * w.double() + b.double()
    assert got.shape == (T, S * width) and float((got.view(T, S, width).double().cpu() - want1[:, None]).abs().max()) < 2e-6
    # the update: every stream from the previous ones together
    y = torch.randn(T, width, generator=g)
    mix = torch.eye(S) + torch.randn(S, S, generator=g) * 0.3
    outw = torch.randn(S, generator=g)
    new = torch.einsum("sr,tsc->trc", mix.double(), x.double()) + outw.double()[None, :, None] * y.double()[:, None, :]
    xs = xd.clone()
    assert ops.streams_write(xs, y.to(DEV), mix.to(DEV).contiguous(), outw.to(DEV)) is None
    assert float((xs.view(T, S, width).double().cpu() - new).abs().max()) < 1e-5
    xs = xd.clone()
    nxt = ops.streams_write(xs, y.to(DEV), mix.to(DEV).contiguous(), outw.to(DEV), nxt=(read.to(DEV),) + args, out_dtype=torch.float32)
    assert float((xs.view(T, S, width).double().cpu() - new).abs().max()) < 1e-5
    want2 = torch.tanh(0.7 * torch.einsum("s,tsc->tc", read.double(), new)) * w.double() + b.double()
    assert float((nxt.double().cpu() - want2).abs().max()) < 1e-5


@pytest.mark.parametrize("E, groups, keep, top", [(16, 2, 1, 2), (8, 4, 3, 3), (6, 1, 1, 2), (9, 9, 4, 4), (64, 8, 2, 6), (5, 5, 5, 5),
                                                  (3, 1, 1, 1), (130, 2, 1, 7), (12, 4, 2, 3)])
def test_router_chooses_what_the_plain_router_chooses(E, groups, keep, top):
    """The router's kernel on given logits: softmax scores, groups that count by their best member, weights that are
    the scores times the scale without a division by their sum."""
    from jllm_serve_amd.kernels import ops
    g = torch.Generator().manual_seed(E * 100 + top)
    T = 300
    z = torch.randn(T, E, generator=g) * 2.0
    r = {"experts": E, "top": top, "scale": 1.7, "groups": {"count": groups, "keep": keep}}
    want_e, want_w = P.route(z.double(), r)
    got_e, got_w = ops.moe_router(z.to(DEV), None, groups, keep, top, 1.7, score="softmax", group_score="max", normalize=False)
    same = (got_e.cpu().long() == want_e).all(dim=1)
    assert int((~same).sum()) <= 1, "fp32 and float64 may order one near-tie differently"
    assert float((got_w.cpu().double()[same] - want_w[same]).abs().max()) < 1e-6
    assert float(want_w.sum(dim=1).max()) <= 1.7 + 1e-9
    assert top == E or float(want_w.sum(dim=1).min()) < 1.6, "not renormalised"


def test_experts_sum_takes_a_gated_shared_row():
    from jllm_serve_amd.kernels import ops
    g = torch.Generator().manual_seed(8)
    T, top, width = 37, 3, 50
    y = torch.randn(T * top, width, generator=g)
    res = torch.randn(T, width, generator=g)
    wts = torch.rand(T, top, generator=g)
    shared = torch.randn(T, width, generator=g)
    z = torch.randn(T, 5, generator=g)
    experts = torch.einsum("tk,tkc->tc", wts.double(), y.view(T, top, width).double())
    gate = torch.sigmoid(z[:, 4].double())[:, None]
    r = res.clone().to(DEV)
    ops.moe_combine(y.to(DEV), r, top, 1.0, weights=wts.to(DEV), shared=shared.to(DEV), shared_gate=z.to(DEV)[:, 4])
    assert float((r.double().cpu() - (res.double() + experts + gate * shared.double())).abs().max()) < 1e-5
    r = torch.full((T, width), float("nan"), device=DEV)
    ops.moe_combine(y.to(DEV), r, top, 1.0, weights=wts.to(DEV), shared=shared.to(DEV), shared_gate=z.to(DEV)[:, 4], overwrite=True)
    assert float((r.double().cpu() - (experts + gate * shared.double())).abs().max()) < 1e-5
    r = torch.full((T, width), float("nan"), device=DEV)
    ops.moe_combine(y.to(DEV), r, top, 1.0, weights=wts.to(DEV), shared=shared.to(DEV), overwrite=True)
    assert float((r.double().cpu() - (experts + shared.double())).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["PA", "PB", "PC", "PD"])
def test_feed_forwards_alone(name, dtype, built, folders):
    """Every layer's feed-forward on random rows: one row, a few, and so many that the experts get tiles of many rows;
    added into a stream (``forward``) and as rows of its own (``output``)."""
    from jllm_serve_amd.engine.step import StepEntry
    cfg = pt.CONFIGS[name][0]
    w = pt.load_weights(folders[name])
    model, runner = built(name, dtype)
    act = act_type(dtype)
    torch.manual_seed(3)
    for T in (1, 7, 45, min(700, cfg["max_positions"])):
        ctx = runner.prepare([StepEntry("ff", pt.prompt(name, T, seed=T), [])])
        xb = (torch.randn(T, cfg["width"]) * 1.5).to(act)
        res = torch.randn(T, cfg["width"])
        for i, n in owners(cfg):
            mlp = cfg["layers"][i]["mlp"]
            if mlp is None:
                assert model.layers[n].ffn is None
                continue
            r = res.clone().to(DEV)
            model.layers[n].ffn.forward(xb.to(DEV), r, ctx)
            own = model.layers[n].ffn.output(xb.to(DEV), ctx)
            y = P.feed_forward(xb.double(), mlp, P.sub(w, f"l{i}.mlp."))
            tol = pt.tolerance(dtype, y)
            # a row whose router scores nearly tie may take another expert in fp32 than in float64: at most a few rows
            for got, want, what in ((r, res.double() + y, "added"), (own, y, "alone")):
                err = (got.double().cpu() - want).abs().amax(dim=1)
                off = int((err > tol).sum())
                assert off <= (0 if T < 45 else max(1, T // 100)), \
                    f"{name} layer {i} feed-forward {what}, {T} rows: {off} rows differ, worst {float(err.max())}"
        runner.finish("ff")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["PA", "PB", "PC", "PD"])
def test_mixers_alone_through_the_cache(name, dtype, built, folders):
    """Every layer run's mixer on random inputs: a portion from position 0, further portions and single rows from the
    cache (a run with borrowed weights has pages of its own), until the windows have passed."""
    from jllm_serve_amd.engine.step import StepEntry
    cfg = pt.CONFIGS[name][0]
    eps = cfg["norm"]["eps"]
    w = pt.load_weights(folders[name])
    model, runner = built(name, dtype)
    act = act_type(dtype)
    torch.manual_seed(4)
    cuts = (29, 6, 1, 1, 2, 17, 1, 1, 1, 70, 1, 2)
    T = sum(cuts)
    rr = runs(cfg)
    xs = [(torch.randn(T, cfg["width"]) * 0.8).to(act) for _ in rr]
    pos = torch.arange(T)

    def plain(r, i):
        layer = cfg["layers"][i]
        ws = P.sub(w, f"l{i}.mix.")
        if layer["type"] == "attention":
            return P.sink_attention(xs[r].double(), layer["mixer"], ws, pos)
        return P.normed_attention(xs[r].double(), layer["mixer"], ws, eps)
    want = [plain(r, i) for r, (i, _) in enumerate(rr)]
    got = [[] for _ in rr]
    at = 0
    for n in cuts:
        ctx = runner.prepare([StepEntry("mix", [0] * n, [])])
        for r, (i, eng) in enumerate(rr):
            res = torch.zeros(n, cfg["width"], device=DEV)
            model.layers[eng].mixer.forward(xs[r][at:at + n].to(DEV), res, ctx, runner.cache.slots[r])
            got[r].append(res.cpu())
        runner.cache.commit("mix", n)
        at += n
    runner.finish("mix")
    for r, (i, _) in enumerate(rr):
        close(torch.cat(got[r]), want[r], dtype, f"{name} run {r} (layer {i}, {cfg['layers'][i]['type']}) mixer")


def _one_layer(kind, heads, kv, dim, vdim, window, keep):
    mixer = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": 2.0 if kind == "attention_2" else 1.0,
             "mask": {"size": window}}
    if kind == "attention_2":
        mixer["mask"]["keep_first"] = keep
    else:
        mixer["rot"] = {"base": 100.0, "dims": 4}
    return {"architecture": "Pivipel", "vocab": 50, "width": 64, "max_positions": 1024, "norm": {"eps": 1e-6}, "streams": 2,
            "layers": [{"type": kind, "mixer": mixer, "mlp": None}]}


# (kind, heads, kv heads, dim, vdim, window, kept first keys, position of the key that decides)
EDGES = [
    ("attention_2", 4, 2, 32, 16, 44, 5, 0), ("attention_2", 4, 2, 32, 16, 44, 5, 4), ("attention_2", 4, 2, 32, 16, 44, 5, 5),
    ("attention_2", 4, 2, 32, 16, 44, 5, 7), ("attention_2", 4, 2, 32, 16, 44, 5, 8), ("attention_2", 4, 2, 32, 16, 44, 5, 63),
    ("attention_2", 4, 2, 32, 16, 44, 5, 64), ("attention_2", 4, 2, 32, 16, 44, 70, 69), ("attention_2", 4, 2, 32, 16, 44, 70, 70),
    ("attention_2", 4, 2, 32, 16, 500, 0, 3), ("attention_2", 3, 1, 10, 6, 44, 5, 4), ("attention_2", 3, 1, 10, 6, 44, 5, 31),
    ("attention_2", 2, 2, 64, 64, 64, 1, 0), ("attention_2", 2, 2, 64, 64, 64, 1, 1),
    ("attention", 4, 2, 32, 16, 44, 0, 0), ("attention", 4, 2, 32, 16, 44, 0, 31), ("attention", 4, 2, 32, 16, 44, 0, 32),
    ("attention", 4, 1, 32, 48, 80, 0, 77), ("attention", 4, 2, 32, 16, 500, 0, 2), ("attention", 3, 3, 12, 20, 9, 0, 15),
]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind, heads, kv, dim, vdim, window, keep, hot", EDGES)
def test_attention_finds_one_key(dtype, kind, heads, kv, dim, vdim, window, keep, hot, tmp_path):
    """Weights and inputs made so that one key decides: only the row at ``hot`` has a part along input entry 0, which
    the key projection turns into a fixed direction of every key head, and every query has a part (input entry 1) along
    that direction (in the unrotated tail of the head, so that the distance does not matter). A row that sees the key
    puts nearly all its weight on it; the rows from ``hot`` + window on do not see it unless it is one of the kept first
    keys. One sink is as large as the deciding score. The rows run as one portion, and again with single rows around
    the window's edge; places of the pages that hold nothing (never written, or given back) are filled with NaN."""
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.weights.safetensors_io import write_safetensors
    cfg = _one_layer(kind, heads, kv, dim, vdim, window, keep)
    folder = pt.write_model(str(tmp_path / "edge"), cfg, 11)
    w = pt.load_weights(folder)
    d = cfg["width"]
    g = torch.Generator().manual_seed(5)
    a = torch.zeros(dim, dtype=F64)
    a[4:] = torch.nn.functional.normalize(torch.randn(dim - 4, generator=g, dtype=F64), dim=0)  # the unrotated part
    amp = 30.0 ** 0.5
    w["l0.mix.k"] *= 0.3  # what the other input entries add to q and k stays small beside the crafted part
    w["l0.mix.q"] *= 0.3
    wk = w["l0.mix.k"].view(kv, dim, d)
    wk[:, :, 0] = (a * amp / 6.0).to(torch.bfloat16).double()
    wk[:, :, 1] = 0.0
    wq = w["l0.mix.q"].view(heads, dim, d)
    wq[:, :, 1] = (a * amp).to(torch.bfloat16).double()
    wq[:, :, 0] = 0.0
    if kind == "attention":
        w["l0.mix.sink"] = torch.linspace(-2.0, 29.0, heads, dtype=F64).to(torch.bfloat16).double()
    write_safetensors(os.path.join(folder, "model.safetensors"), {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in w.items()})
    w = pt.load_weights(folder)
    T = hot + window + 60 if window < 400 else 620
    near = hot + window - 12  # single rows from here on cross the window's edge
    cut_lists = [[T], ([near] if near > 0 else []) + [1] * 25 + [T - max(near, 0) - 25] if window < 400 else [40, 400, 2, 1, 1, 1, T - 445]]
    act = act_type(dtype)
    h = torch.randn(T, d, generator=g) * 0.3
    h[:, 0] = 0.0
    h[hot, 0] = 6.0
    h[:, 1] = 1.0
    h = h.to(act)
    pos = torch.arange(T)
    ws = P.sub(w, "l0.mix.")
    m = cfg["layers"][0]["mixer"]

    def plain(x):
        return P.sink_attention(x.double(), m, ws, pos) if kind == "attention" else P.normed_attention(x.double(), m, ws, 1e-6)
    want = plain(h)
    h_no = h.clone()
    h_no[hot, 0] = 0.0
    gap = (want - plain(h_no)).abs().amax(dim=1)
    sees = [t for t in range(hot + 1, T) if t - hot < window or hot < keep]
    blind = [t for t in range(hot + 1, T) if not (t - hot < window or hot < keep)]
    assert float(gap[sees].min()) > 0.1 * float(want.abs().max()), "the key decides every row that sees it, or the test is blind"
    assert not blind or float(gap[blind].max()) < 1e-9
    if window < 400:
        assert (hot + window - 1 in sees) and ((hot + window in blind) or hot < keep)
    model = load_model(folder, dtype, torch.device(DEV), max_positions=1024)
    runner = build_runner(model, page_size=8, pool_tokens=1024, max_requests=2)
    grp = runner.cache.groups[0]
    for cuts in cut_lists:
        for t in grp.storage.values():
            t.fill_(float("nan"))
        got, at = [], 0
        for n in cuts:
            ctx = runner.prepare([StepEntry("edge", [0] * n, [])])
            res = torch.zeros(n, d, device=DEV)
            model.layers[0].mixer.forward(h[at:at + n].to(DEV), res, ctx, runner.cache.slots[0])
            got.append(res.cpu())
            runner.cache.commit("edge", n)
            at += n
            held = [p for p in runner.cache.requests["edge"].tables[0] if p >= 0]
            free = torch.ones(grp.pool.num_pages, dtype=torch.bool)
            free[held] = False
            for t in grp.storage.values():  # what the window gave back holds NaN from now on
                t[:, free.to(DEV)] = float("nan")
        runner.finish("edge")
        out = torch.cat(got).double()
        assert bool(torch.isfinite(out).all()), "a place that holds nothing was read"
        err = (out - want).abs().amax(dim=1)
        tol = (1e-4 if dtype == "float32" else 4e-2) * float(want.abs().max())
        bad = (err > tol).nonzero().flatten().tolist()
        assert not bad, f"cuts {cuts[:4]}..: rows at positions {bad[:8]} differ by up to {float(err.max())} (the key is at {hot})"
    if window < 400:
        assert runner.cache.pages_given_back_by_window > 0, "the window gives pages back"


# ------------------------------------------------------------------------------------------------ whole models


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["PA", "PB", "PC", "PD"])
def test_stream_after_every_run(name, dtype, built, folders):
    """The residual stream (the sum of the streams) after every layer run against the plain one."""
    from jllm_serve_amd.engine.step import StepEntry
    model, runner = built(name, dtype)
    cfg = pt.CONFIGS[name][0]
    toks = pt.prompt(name, 37)
    streams = []
    P.forward(cfg, pt.load_weights(folders[name]), toks, watch=lambda i, x: streams.append(x.clone()))
    got = []
    model.watch = lambda run, x: got.append(x.detach().cpu().clone())
    try:
        runner.step([StepEntry("w", toks, [])])
    finally:
        model.watch = None
        runner.finish("w")
    assert len(got) == len(streams) == len(cfg["layers"])
    for r, (g, s) in enumerate(zip(got, streams)):
        tol = (2e-5 if dtype == "float32" else 6e-2) * float(s.abs().max())
        err = (g.double() - s).abs().amax(dim=1)
        # in bfloat16 a row whose router scores nearly tie takes another expert than float64 does (see pt.flipped)
        assert int((err > tol).sum()) <= len(toks) * pt.flipped(dtype), f"{name} {dtype}: the stream after run {r}"
        assert float(err.median()) <= tol / 2


def build_trace(name):
    t = replay.Trace(page=pt.CONFIGS[name][2])
    lens = [1, 2, 3, 9, 40, 131]
    toks = {f"r{n}": pt.prompt(name, n) for n in lens}
    longest = toks[f"r{lens[-1]}"]
    replay.whole(t, "whole", longest)
    replay.tail_one_by_one(t, "tail", longest, tail=80)
    replay.portions(t, "cut", longest)
    for rid, tk in toks.items():
        replay.whole(t, "w" + rid, tk)
    more = dict(toks)
    more["x1"] = pt.prompt(name, 45, seed=1)
    more["x2"] = pt.prompt(name, 2, seed=2)
    more["x3"] = pt.prompt(name, 66, seed=3)
    replay.mixed(t, more, seed=len(name))
    req_tokens = {"whole": longest, "tail": longest, "cut": longest, **{"w" + k: v for k, v in toks.items()}, **more}
    return t, req_tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["PA", "PB", "PC", "PD"])
def test_replay_matches_plain(name, dtype, folders, plain_logits, tmp_path):
    """bin/trace_run: whole, the last 80 tokens one by one, portions down to two tokens, mixed batches with at most four
    live requests on a pool exactly as large as the busiest step (pages are used again; the free pages are reordered
    before every step). In float32 a position's logits are the same bits however it was reached."""
    cfg, _, page = pt.CONFIGS[name]
    trace, req_tokens = build_trace(name)
    got = replay.run(folders[name], dtype, trace, str(tmp_path), page_size=page, max_tokens=trace.peak, shuffle_free=len(name) + 7)
    V = cfg["vocab"]
    by_place = {}
    ratios, over = [], []
    for step, rows in trace.rows.items():
        arr = got[step].reshape(len(rows), V)
        for i, (rid, pos) in enumerate(rows):
            ref = plain_logits(name, req_tokens[rid])[pos]
            tol = pt.tolerance(dtype, ref)
            err = float(np.abs(arr[i].astype(np.float64) - ref.numpy()).max())
            if err > tol:
                over.append((step, rid, pos, err, tol))
            ratios.append(err / float(ref.abs().max()))
            by_place[(rid, pos)] = arr[i]
    assert len(over) <= len(ratios) * pt.flipped(dtype), f"{name} {dtype}: {len(over)} of {len(ratios)} positions differ, first {over[:3]}"
    assert float(np.median(ratios)) <= pt.typical(dtype), f"{name} {dtype}: median error {np.median(ratios):.3g} of the largest logit"
    if dtype == "float32":
        pairs = [("whole", "tail"), ("whole", "cut")] + [("w" + rid, rid) for rid in req_tokens if "w" + rid in req_tokens]
        for a, b in pairs:
            for pos in range(len(req_tokens[a])):
                assert np.array_equal(by_place[(a, pos)], by_place[(b, pos)]), \
                    f"{name}: position {pos} of '{b}' differs in bits from the same position of '{a}'"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_reused_pages(dtype, built, plain_logits):
    """A short prompt, then 230 tokens one by one (bfloat16: through captured steps), far beyond every window of the
    model, beside a second request that joins late; then both end and a third request takes over their pages."""
    from jllm_serve_amd.engine.step import StepEntry
    name = "PB"
    model, runner = built(name, dtype, graphs=dtype == "bfloat16")
    a, b, c = pt.prompt(name, 240, seed=5), pt.prompt(name, 70, seed=6), pt.prompt(name, 30, seed=7)
    ra, rb, rc = plain_logits(name, a), plain_logits(name, b), plain_logits(name, c)
    out = runner.step([StepEntry("a", a[:10], range(10))])
    close(out, ra[:10], dtype, "prompt")
    errs, over, rows = [], [], 0

    def held(got, ref, what):  # one row against the plain one; rows beyond the bound are counted (see pt.flipped)
        nonlocal rows
        rows += 1
        err = float((got.double().cpu() - ref).abs().max())
        if err > pt.tolerance(dtype, ref):
            over.append((what, err))
        return err / float(ref.abs().max())
    for i in range(10, 240):
        entries = [StepEntry("a", a[i:i + 1], [0])]
        j = i - 150
        if j == 0:
            entries.append(StepEntry("b", b[:20], [19]))
        elif 0 < j and 20 + j - 1 < 70:
            entries.append(StepEntry("b", b[20 + j - 1:20 + j], [0]))
        out = runner.step(entries)
        errs.append(held(out[0], ra[i], f"a at {i}"))
        if len(entries) == 2:
            held(out[1], rb[19 if j == 0 else 20 + j - 1], f"b beside a at {i}")
    assert len(over) <= rows * pt.flipped(dtype), f"{len(over)} of {rows} rows differ, first {over[:3]}"
    assert float(np.median(errs)) <= pt.typical(dtype), "the error does not grow with the decoded tokens"
    assert float(np.median(errs[-30:])) <= 2 * max(float(np.median(errs[:30])), pt.typical(dtype) / 4)
    assert runner.cache.pages_given_back_by_window > 0
    if dtype == "bfloat16":
        assert runner.graphs.replays > 100
    runner.finish("a")
    runner.finish("b")
    out = runner.step([StepEntry("c", c, range(len(c)))]).double().cpu()
    bad = [p for p in range(len(c)) if float((out[p] - rc[p]).abs().max()) > pt.tolerance(dtype, rc[p])]
    assert len(bad) <= len(c) * pt.flipped(dtype), f"a request on used pages: positions {bad} differ"
    # (a short prompt: few keys per row, so a row's rounding errors average out less than in the long request)
    assert float(np.median([float((out[p] - rc[p]).abs().max() / rc[p].abs().max()) for p in range(len(c))])) <= 2 * pt.typical(dtype)
    runner.finish("c")
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(dtype, folders):
    """Engine.generate with more requests than places and a pool so small that requests are preempted and computed
    again: the tokens of the plain implementation."""
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    from jllm_serve_amd.sampling import SamplingParams
    name = "PA"
    cfg = pt.CONFIGS[name][0]
    w = pt.load_weights(folders[name])
    model = load_model(folders[name], dtype, torch.device(DEV), max_positions=128)
    runner = build_runner(model, page_size=8, pool_tokens=160, max_requests=3)
    eng = Engine(runner, SchedulerConfig(max_batch_tokens=40, prefill_chunk=16, max_positions=128), eos_token_ids=())
    prompts = [pt.prompt(name, n, seed=9) for n in (1, 5, 23, 40, 12)]
    n_new = 12
    got = [r.tokens for r in eng.generate(prompts, SamplingParams.greedy_params(max_tokens=n_new))]
    # random weights make near-ties that rounding decides: every token the engine chose must be one of the plain
    # implementation's best, given the engine's own tokens before it (float32: within its own small bound)
    for p, g in zip(prompts, got):
        assert len(g) == n_new
        ref = P.forward(cfg, w, p + g)
        for i, tok in enumerate(g):
            row = ref[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 2 * pt.tolerance(dtype, row), f"token {i} after a prompt of {len(p)}"
    runner.cache.check()
    assert not runner.cache.requests


def test_command_line_runs_the_design(folders, tmp_path):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "jllm"), "run", "--model", folders["PC"], "--dtype", "float32",
                        "--prompt", "3 1 4 1 5", "--max-tokens", "6", "--temp", "0", "--json", "--ctx", "128", "--ignore-eos"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    w = pt.load_weights(folders["PC"])
    ref = P.forward(pt.P_C, w, [3, 1, 4, 1, 5] + out["tokens"])
    assert len(out["tokens"]) == 6
    for i, tok in enumerate(out["tokens"]):
        row = ref[4 + i]
        assert float(row.max() - row[tok]) <= 2 * pt.tolerance("float32", row)
