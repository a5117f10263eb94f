"""Ratasun on the GPU against the plain implementation (tests/plain/ratasun_plain.py): every mechanism alone, the
router's choice on crafted scores, the latent attention with one far key that decides (at the first position, at a
page's last and first place, hundreds of keys back), both recurrences on crafted memories (written by the first token,
read hundreds of tokens later) in portions against the whole, whole prompts against token-by-token decoding, portions
down to two tokens, mixed batches on a pool that is used again, the stream after every layer run, long decoding through
captured steps, greedy generation through the engine, and the replay program."""
import json
import os

import numpy as np
import pytest
import torch

import ratasun_tiny as rt
import replay
from plain import ratasun_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"
F64 = torch.float64


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: rt.write_model(str(tmp_path_factory.mktemp("ratasun_" + name)), cfg, seed)
            for name, (cfg, seed, page) in rt.CONFIGS.items()}


@pytest.fixture(scope="module")
def built(folders):
    from jllm_serve_amd.engine import build_runner, load_model
    cache = {}

    def get(name, dtype, graphs=False):
        if (name, dtype, graphs) not in cache:
            model = load_model(folders[name], dtype, torch.device(DEV), max_positions=1024)
            cache[(name, dtype, graphs)] = (model, build_runner(model, page_size=rt.CONFIGS[name][2], pool_tokens=1024,
                                                                max_requests=4, graphs=graphs))
        return cache[(name, dtype, graphs)]
    return get


@pytest.fixture(scope="module")
def plain_logits(folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            memo[key] = P.forward(rt.CONFIGS[name][0], rt.load_weights(folders[name]), list(tokens))
        return memo[key]
    return get


def close(got, want, dtype, what=""):
    err = float((got.double().cpu() - want).abs().max())
    assert err <= rt.tolerance(dtype, want), f"{what}: {err} > {rt.tolerance(dtype, want)}"


def act_type(dtype):
    return torch.float32 if dtype == "float32" else torch.bfloat16


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# ------------------------------------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("E, groups, keep, top", [(16, 2, 1, 2), (8, 4, 3, 3), (6, 1, 1, 2), (9, 9, 4, 4), (64, 8, 2, 6), (5, 5, 5, 5),
                                                  (3, 1, 1, 1), (130, 2, 1, 7)])
def test_router_chooses_what_the_plain_router_chooses(E, groups, keep, top):
    """The router's kernel on given logits: sigmoid scores, a correction (negative for some experts, so that choice
    scores are negative and a closed group must count as minus infinity), groups, weights without the correction."""
    from jllm_serve_amd.kernels import ops
    g = torch.Generator().manual_seed(E * 100 + top)
    T = 300
    z = torch.randn(T, E, generator=g) * 2.0
    corr = torch.randn(E, generator=g) * 0.5 - 0.8
    r = {"experts": E, "top": top, "scale": 1.7, "groups": {"count": groups, "keep": keep}}
    want_e, want_w = P.route(z.double(), r, torch.eye(E, dtype=F64), corr.double())
    for c in (corr, corr.to(torch.bfloat16)):
        if c.dtype == torch.bfloat16:
            want_e, want_w = P.route(z.double(), r, torch.eye(E, dtype=F64), c.double())
        got_e, got_w = ops.moe_router(z.to(DEV), c.to(DEV), groups, keep, top, 1.7)
        # fp32 sigmoids of logits that differ in the 7th digit may order the other way: such rows are left out (few)
        s = torch.sigmoid(z.double()) + c.double()
        gaps = (s[:, :, None] - s[:, None, :]).abs() + torch.eye(E, dtype=F64)[None] * 9
        sure = gaps.amin(dim=(1, 2)) > 1e-5
        assert int(sure.sum()) > T * 0.7
        assert torch.equal(got_e.cpu().long()[sure], want_e[sure]), "the chosen experts, best first"
        assert torch.allclose(got_w.cpu().double()[sure], want_w[sure], atol=1e-6)
    # without a correction the choice scores are the scores
    got_e, got_w = ops.moe_router(z.to(DEV), None, groups, keep, top, 1.0)
    want_e, want_w = P.route(z.double(), dict(r, scale=1.0), torch.eye(E, dtype=F64), torch.zeros(E, dtype=F64))
    s = torch.sigmoid(z.double())
    sure = ((s[:, :, None] - s[:, None, :]).abs() + torch.eye(E, dtype=F64)[None] * 9).amin(dim=(1, 2)) > 1e-5
    assert torch.equal(got_e.cpu().long()[sure], want_e[sure]) and torch.allclose(got_w.cpu().double()[sure], want_w[sure], atol=1e-6)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["RA", "RB", "RC"])
def test_feed_forwards_alone(name, dtype, built, folders):
    """Every layer's experts on random rows: one row, a few, and so many that the experts get tiles of many rows."""
    from jllm_serve_amd.engine.step import StepEntry
    cfg = rt.CONFIGS[name][0]
    w = rt.load_weights(folders[name])
    model, runner = built(name, dtype)
    act = act_type(dtype)
    torch.manual_seed(3)
    for T in (1, 7, 45, 700):
        ctx = runner.prepare([StepEntry("ff", rt.prompt(name, T, seed=T), [])])
        xb = (torch.randn(T, cfg["width"]) * 1.5).to(act)
        res = torch.randn(T, cfg["width"])
        for i, layer in enumerate(cfg["layers"]):
            if layer["mlp"] is None:
                assert model.layers[i].ffn is None
                continue
            r = res.clone().to(DEV)
            model.layers[i].ffn.forward(xb.to(DEV), r, ctx)
            want = res.double() + P.moe(xb.double(), layer["mlp"], P._sub(w, f"l{i}.mlp."))
            err = (r.double().cpu() - want).abs().amax(dim=1)
            tol = rt.tolerance(dtype, want)
            # a row whose choice scores nearly tie may take another expert in fp32 than in float64: at most a few rows
            off = int((err > tol).sum())
            assert off <= (0 if T < 45 else max(1, T // 100)), f"{name} layer {i} feed-forward, {T} rows: {off} rows differ, worst {float(err.max())}"
        runner.finish("ff")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["RA", "RB", "RC"])
def test_mixers_alone_through_cache_and_state(name, dtype, built, folders):
    """Every layer run's mixer on random inputs: a portion from position 0, further portions and single rows from the
    cache and the state (every pass of a looped layer has its own)."""
    from jllm_serve_amd.engine.step import StepEntry
    cfg = rt.CONFIGS[name][0]
    eps = cfg["norm"]["eps"]
    w = rt.load_weights(folders[name])
    model, runner = built(name, dtype)
    act = act_type(dtype)
    torch.manual_seed(4)
    cuts = (29, 6, 1, 1, 2, 17)
    T = sum(cuts)
    runs = P.layer_runs(cfg)
    xs = [(torch.randn(T, cfg["width"]) * 0.8).to(act) for _ in runs]
    pos = torch.arange(T)
    want = [P.mixer(xs[r].double(), w, i, cfg["layers"][i], eps, pos) for r, (i, _, _) in enumerate(runs)]
    got = [[] for _ in runs]
    at = 0
    for n in cuts:
        ctx = runner.prepare([StepEntry("mix", [0] * n, [])])
        for r, (i, _, _) in enumerate(runs):
            res = torch.zeros(n, cfg["width"], device=DEV)
            model.layers[i].mixer.forward(xs[r][at:at + n].to(DEV), res, ctx, runner.cache.slots[r])
            got[r].append(res.cpu())
        runner.cache.commit("mix", n)
        at += n
    runner.finish("mix")
    for r, (i, _, _) in enumerate(runs):
        close(torch.cat(got[r]), want[r], dtype, f"{name} run {r} (layer {i}, {cfg['layers'][i]['type']}) mixer")


FAR = {"architecture": "Ratasun", "vocab": 50, "width": 64, "norm": {"eps": 1e-6},
       "layers": [{"type": "latent_attention", "mlp": None,
                   "mixer": {"heads": 4, "dim": 16, "rot_dim": 8, "vdim": 16, "kv_rank": 32, "scale": 0.2, "rot": {"base": 100.0, "dims": 8}}}]}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hot", [0, 31, 32, 77])
def test_latent_attention_finds_one_far_key(dtype, hot, tmp_path):
    """Weights and inputs made so that one key decides: only the row at ``hot`` has a part along input entry 0, which
    the latent's projection blows up, and every head's query has a part (input entry 1) along that row's unrotated key.
    Rows after ``hot`` put nearly all their weight on it, in a portion, in later portions and as single rows, up to 300
    keys later; a kernel that misses it (the first key, a page's last or first place, a key far back) is off by the
    size of the values."""
    from jllm_serve_amd.engine import build_runner, load_model
    from jllm_serve_amd.engine.step import StepEntry
    from jllm_serve_amd.weights.safetensors_io import write_safetensors
    folder = rt.write_model(str(tmp_path / "far"), FAR, 11)
    w = rt.load_weights(folder)
    m = FAR["layers"][0]["mixer"]
    H, dim, rd, R, d = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"], FAR["width"]
    g = torch.Generator().manual_seed(5)
    a = torch.nn.functional.normalize(torch.randn(R, generator=g, dtype=F64), dim=0)
    w["l0.mix.dkv"][:, 0] = 0.0
    w["l0.mix.dkv"][:R, 0] = (a * 3.0).to(torch.bfloat16).double()
    w["l0.mix.dkv"][:, 1] = 0.0
    c_hot = P.rms((w["l0.mix.dkv"][:R, 0] * 6.0)[None], 1e-6)[0] * w["l0.mix.dkv.norm"]
    k_hot = (w["l0.mix.uk"] @ c_hot).view(H, dim)
    q_rows = w["l0.mix.q"].view(H, dim + rd, d)
    q_rows[:, :, 1] = 0.0
    q_rows[:, :dim, 1] = (torch.nn.functional.normalize(k_hot, dim=1) * 40.0).to(torch.bfloat16).double()
    w["l0.mix.q"] = q_rows.view(H * (dim + rd), d)
    write_safetensors(os.path.join(folder, "model.safetensors"), {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in w.items()})
    w = rt.load_weights(folder)
    cuts = [40, 200, 2, 1, 1, 1, 85, 1, 1]
    T = sum(cuts)
    act = act_type(dtype)
    h = torch.randn(T, d, generator=g) * 0.3
    h[:, 0] = 0.0
    h[hot, 0] = 6.0
    h[:, 1] = 1.0
    h = h.to(act)
    pos = torch.arange(T)
    want = P.mixer(h.double(), w, 0, FAR["layers"][0], 1e-6, pos)
    h_no = h.clone()
    h_no[hot, 0] = 0.0
    blind = P.mixer(h_no.double(), w, 0, FAR["layers"][0], 1e-6, pos)
    gap = (want - blind)[hot + 1:].abs().amax(dim=1)
    assert float(gap.min()) > 0.15 * float(want.abs().max()), "the far key decides every later row, or the test is blind"
    model = load_model(folder, dtype, torch.device(DEV), max_positions=512)
    runner = build_runner(model, page_size=8, pool_tokens=1024, max_requests=2)
    got, at = [], 0
    for n in cuts:
        ctx = runner.prepare([StepEntry("far", [0] * n, [])])
        res = torch.zeros(n, d, device=DEV)
        model.layers[0].mixer.forward(h[at:at + n].to(DEV), res, ctx, runner.cache.slots[0])
        got.append(res.cpu())
        runner.cache.commit("far", n)
        at += n
    runner.finish("far")
    err = (torch.cat(got).double() - want).abs().amax(dim=1)
    tol = (1e-4 if dtype == "float32" else 4e-2) * float(want.abs().max())
    bad = (err > tol).nonzero().flatten().tolist()
    assert not bad, f"rows at positions {bad[:8]} differ by up to {float(err.max())} (the far key is at {hot})"


def _plain_channel_delta(qkv, beta_in, decay_in, a_log, dt_bias, H, G, dk, dv):
    """float64, one request: the recurrence with one decay per head and key channel; returns the raw read-outs."""
    T = qkv.shape[0]
    q = qkv[:, :G * dk].view(T, G, dk)
    k = qkv[:, G * dk:2 * G * dk].view(T, G, dk)
    v = qkv[:, 2 * G * dk:].view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(beta_in)
    gch = torch.exp(-torch.exp(a_log)[None, :, None] * softplus(decay_in + dt_bias).view(T, H, dk))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        kh = hd // (H // G)
        for t in range(T):
            S = gch[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            out[t, hd] = S.T @ q[t, kh]
    return out.reshape(T, H * dv)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, dk, dv", [(2, 1, 16, 8), (3, 3, 40, 24), (2, 2, 128, 128), (1, 1, 7, 5), (4, 2, 200, 40)])
def test_channel_delta_recalls_a_far_memory(dtype, H, G, dk, dv):
    """The recurrence with a decay per key channel over 600 tokens in portions, with inputs chosen so that a fault
    shows: the first token writes a value along key channel 0, which no later key touches and whose decay is nearly
    none while every other channel decays fast; the last token asks along channel 0. A second request beside it has
    the decays the other way round and must have forgotten. Then the same tokens whole: the same bits."""
    from jllm_serve_amd.kernels import ops
    act = act_type(dtype)
    torch.manual_seed(dk)
    T = 600
    C = 2 * G * dk + H * dv

    def make(keeps):
        qkv = torch.randn(T, C)
        k = qkv[:, G * dk:2 * G * dk].view(T, G, dk)
        q = qkv[:, :G * dk].view(T, G, dk)
        k[1:, :, 0] = 0.0
        k[0] = 0.0
        k[0, :, 0] = 3.0
        q[-1] = 0.0
        q[-1, :, 0] = 2.0
        proj = torch.randn(T, H + 3)
        proj[0, :H] = 30.0  # b of the first token: written in full
        decay = torch.randn(T, H * dk) * 0.3 + 1.0
        decay.view(T, H, dk)[:, :, 0] = -30.0 if keeps else 3.0  # softplus(-30 + dt_bias) ~ 0: channel 0 keeps
        return qkv.to(act), proj.to(act), decay

    a_log, dt_bias = torch.randn(H) * 0.3, torch.randn(H * dk) * 0.3
    reqs = [make(True), make(False)]
    wants = [_plain_channel_delta(r[0].double(), r[1].double()[:, :H], r[2].double(), a_log.double(), dt_bias.double(), H, G, dk, dv) for r in reqs]
    v0 = reqs[0][0].double()[0, 2 * G * dk:]
    assert torch.allclose(wants[0][-1], v0 * dk ** -0.5, atol=1e-3), "the last row of the first request reads the first token's value"
    assert float(wants[1][-1].abs().max()) < 1e-3 * float(v0.abs().max()) + 1e-6, "the second request has forgotten it"
    dev = lambda t: t.to(DEV)
    results = []
    for cuts in ([300, 2, 1, 1, 296], [T]):
        state = torch.zeros(5, H, dv, dk, device=DEV)
        slots = torch.tensor([3, 1], dtype=torch.int32, device=DEV)
        got = [[], []]
        at = 0
        for n in cuts:
            qkv = torch.cat([r[0][at:at + n] for r in reqs])
            proj = torch.cat([r[1][at:at + n] for r in reqs])
            decay = torch.cat([r[2][at:at + n] for r in reqs])
            row_req = torch.tensor([0] * n + [1] * n, dtype=torch.int32, device=DEV)
            raw = ops.gated_delta(dev(qkv), dev(proj), 0, 0, dev(a_log), dev(dt_bias), state, row_req, slots, 2, H, G, dk, dv,
                                  decay_rows=dev(decay)).cpu()
            got[0].append(raw[:n])
            got[1].append(raw[n:])
            at += n
        assert float(state[[0, 2, 4]].abs().max()) == 0.0, "a state row of no request was written"
        results.append([torch.cat(x) for x in got])
        for i in range(2):
            tol = 3e-5 if dtype == "float32" else 3e-2
            err = float((results[-1][i].double() - wants[i]).abs().max())
            assert err <= tol * max(1.0, float(wants[i].abs().max())), f"request {i} cut {cuts}: {err}"
    for i in range(2):
        assert torch.equal(results[0][i], results[1][i]), "the recurrence depends on how the tokens were cut"


def _plain_ssm(xbc, dt_in, a_log, dt_bias, skip, H, G, N, Pd):
    T = xbc.shape[0]
    inner = H * Pd
    x, B, C = xbc[:, :inner].view(T, H, Pd), xbc[:, inner:inner + G * N].view(T, G, N), xbc[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt_in + dt_bias)
    dA = torch.exp(-torch.exp(a_log)[None] * dt)
    out = torch.zeros(T, H, Pd, dtype=F64)
    for hd in range(H):
        S = torch.zeros(N, Pd, dtype=F64)
        gr = hd // (H // G)
        for t in range(T):
            S = dA[t, hd] * S + dt[t, hd] * torch.outer(B[t, gr], x[t, hd])
            out[t, hd] = S.T @ C[t, gr] + skip[hd] * x[t, hd]
    return out.reshape(T, inner)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, N, Pd", [(2, 1, 16, 8), (3, 3, 40, 24), (4, 2, 128, 64), (1, 1, 7, 5), (6, 2, 9, 100), (2, 2, 250, 20)])
def test_state_space_scan_recalls_a_far_memory(dtype, H, G, N, Pd):
    """The state-space recurrence over 600 tokens in portions: the first token writes along state row 0 with a large
    step, later tokens have no part along it and steps so small that nothing decays; the last token reads along row 0.
    A second request beside it takes large steps and forgets. Then whole: the same bits."""
    from jllm_serve_amd.kernels import ops
    act = act_type(dtype)
    torch.manual_seed(N)
    T = 600
    inner = H * Pd

    def make(keeps):
        xbc = torch.randn(T, inner + 2 * G * N)
        B = xbc[:, inner:inner + G * N].view(T, G, N)
        Cc = xbc[:, inner + G * N:].view(T, G, N)
        B[1:, :, 0] = 0.0
        B[0] = 0.0
        B[0, :, 0] = 2.0
        Cc[-1] = 0.0
        Cc[-1, :, 0] = 1.5
        proj = torch.randn(T, H + 5)
        proj[:, 2:2 + H] = -12.0 if keeps else 1.0  # the steps' input: softplus(-12 + dt_bias) ~ 1e-5
        proj[0, 2:2 + H] = 1.0
        return xbc.to(act), proj.to(act)

    a_log, dt_bias, skip = torch.randn(H) * 0.3, torch.randn(H) * 0.3, torch.randn(H) * 0.5 + 1
    reqs = [make(True), make(False)]
    wants = [_plain_ssm(r[0].double(), r[1].double()[:, 2:2 + H], a_log.double(), dt_bias.double(), skip.double(), H, G, N, Pd) for r in reqs]
    # what the last row of the first request reads beyond its own skip term is the first token's x, nearly undecayed
    x_first = reqs[0][0].double()[0, :inner].view(H, Pd)
    x_last = reqs[0][0].double()[-1, :inner].view(H, Pd)
    dt0 = softplus(reqs[0][1].double()[0, 2:2 + H] + dt_bias.double())
    far = wants[0][-1].view(H, Pd) - skip.double()[:, None] * x_last
    assert torch.allclose(far, 3.0 * dt0[:, None] * x_first, rtol=0.05, atol=1e-3)
    far2 = wants[1][-1].view(H, Pd) - skip.double()[:, None] * reqs[1][0].double()[-1, :inner].view(H, Pd)
    assert float(far2.abs().max()) < 1e-6
    dev = lambda t: t.to(DEV)
    results = []
    for cuts in ([300, 2, 1, 1, 296], [T]):
        state = torch.zeros(5, H, Pd, N, device=DEV)
        slots = torch.tensor([3, 1], dtype=torch.int32, device=DEV)
        got = [[], []]
        at = 0
        for n in cuts:
            xbc = torch.cat([r[0][at:at + n] for r in reqs])
            proj = torch.cat([r[1][at:at + n] for r in reqs])
            row_req = torch.tensor([0] * n + [1] * n, dtype=torch.int32, device=DEV)
            raw = ops.ssm_scan(dev(xbc), dev(proj), 2, dev(a_log), dev(dt_bias), dev(skip), state, row_req, slots, 2, H, G, N, Pd).cpu()
            got[0].append(raw[:n])
            got[1].append(raw[n:])
            at += n
        assert float(state[[0, 2, 4]].abs().max()) == 0.0, "a state row of no request was written"
        results.append([torch.cat(x) for x in got])
        for i in range(2):
            tol = 3e-5 if dtype == "float32" else 3e-2
            err = float((results[-1][i].double() - wants[i]).abs().max())
            assert err <= tol * max(1.0, float(wants[i].abs().max())), f"request {i} cut {cuts}: {err}"
    for i in range(2):
        assert torch.equal(results[0][i], results[1][i]), "the recurrence depends on how the tokens were cut"


@pytest.mark.parametrize("width, groups", [(12, 3), (192, 2), (70, 1), (1024, 8), (600, 600)])
def test_gated_group_norm_and_convolution_bias(width, groups):
    """The gate comes before the norm, every part of the row has its own root mean square; the convolution adds its bias
    before silu, across steps shorter than its taps."""
    from jllm_serve_amd.kernels import ops
    torch.manual_seed(width)
    T, eps = 11, 1e-5
    y, z, wt = torch.randn(T, width) * 2, torch.randn(T, width + 5), torch.randn(width)
    for act in (torch.float32, torch.bfloat16):
        zz, ww = z.to(act), wt.to(act)
        got = ops.gated_group_norm(y.to(DEV), zz.to(DEV)[:, 5:], ww.to(DEV), eps, groups, torch.float32).cpu().double()
        t = y.double() * P.silu(zz.double()[:, 5:])
        want = P.rms(t.view(T, groups, width // groups), eps).reshape(T, width) * ww.double()
        assert torch.allclose(got, want, atol=2e-5, rtol=1e-5)
        other = P.rms(y.double().view(T, groups, width // groups), eps).reshape(T, width) * ww.double() * P.silu(zz.double()[:, 5:])
        assert not torch.allclose(want, other, atol=1e-2), "gate first and norm first differ: the test tells them apart"
    taps, C = 4, width
    w, b = torch.randn(C, taps), torch.randn(C)
    x = torch.randn(23, C + 3)
    want = P.silu(P.causal_conv(x[:, :C].double(), w.double(), b.double()))
    state = torch.zeros(3, taps - 1, C, device=DEV)
    got, at = [], 0
    for n in (1, 2, 1, 9, 10):
        got.append(ops.short_conv(x[at:at + n].to(DEV), w.to(DEV), state, torch.zeros(n, dtype=torch.int32, device=DEV),
                                  torch.tensor([1], dtype=torch.int32, device=DEV), 1, bias=b.to(DEV)).cpu())
        at += n
    assert torch.allclose(torch.cat(got).double(), want, atol=1e-5)
    assert float(state[[0, 2]].abs().max()) == 0.0


# ------------------------------------------------------------------------------------------------ whole models


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["RA", "RB", "RC"])
def test_stream_after_every_run(name, dtype, built, folders):
    """The residual stream after every layer run against the plain one (before every pass of a loop the stream is
    mixed with the embedding output and the pass's vector joins)."""
    from jllm_serve_amd.engine.step import StepEntry
    model, runner = built(name, dtype)
    cfg = rt.CONFIGS[name][0]
    toks = rt.prompt(name, 37)
    streams = []
    P.forward(cfg, rt.load_weights(folders[name]), toks, streams=streams)
    got = []
    model.watch = lambda run, x: got.append(x.detach().cpu().clone())
    try:
        runner.step([StepEntry("w", toks, [])])
    finally:
        model.watch = None
        runner.finish("w")
    assert len(got) == len(streams) == len(P.layer_runs(cfg))
    for r, (g, s) in enumerate(zip(got, streams)):
        tol = (2e-5 if dtype == "float32" else 6e-2) * float(s.abs().max())
        assert float((g.double() - s).abs().max()) <= tol, f"{name} {dtype}: the stream after run {r}"


def build_trace(name):
    t = replay.Trace(page=rt.CONFIGS[name][2])
    lens = [1, 2, 3, 9, 40, 131]
    toks = {f"r{n}": rt.prompt(name, n) for n in lens}
    longest = toks[f"r{lens[-1]}"]
    replay.whole(t, "whole", longest)
    replay.tail_one_by_one(t, "tail", longest, tail=40)
    replay.portions(t, "cut", longest)
    for rid, tk in toks.items():
        replay.whole(t, "w" + rid, tk)
    more = dict(toks)
    more["x1"] = rt.prompt(name, 45, seed=1)
    more["x2"] = rt.prompt(name, 2, seed=2)
    more["x3"] = rt.prompt(name, 66, seed=3)
    replay.mixed(t, more, seed=len(name))
    req_tokens = {"whole": longest, "tail": longest, "cut": longest, **{"w" + k: v for k, v in toks.items()}, **more}
    return t, req_tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["RA", "RB", "RC"])
def test_replay_matches_plain(name, dtype, folders, plain_logits, tmp_path):
    """bin/trace_run: whole, the last 40 tokens one by one, portions down to two tokens, mixed batches with at most four
    live requests on a pool exactly as large as the busiest step (pages and state slots are used again; the free pages
    are reordered before every step). In float32 a position's logits are the same bits however it was reached."""
    cfg, _, page = rt.CONFIGS[name]
    trace, req_tokens = build_trace(name)
    got = replay.run(folders[name], dtype, trace, str(tmp_path), page_size=page, max_tokens=trace.peak, shuffle_free=len(name) + 7)
    V = cfg["vocab"]
    by_place = {}
    ratios, over = [], []
    for step, rows in trace.rows.items():
        arr = got[step].reshape(len(rows), V)
        for i, (rid, pos) in enumerate(rows):
            ref = plain_logits(name, req_tokens[rid])[pos]
            tol = rt.tolerance(dtype, ref)
            err = float(np.abs(arr[i].astype(np.float64) - ref.numpy()).max())
            if err > tol:
                over.append((step, rid, pos, err, tol))
            ratios.append(err / float(ref.abs().max()))
            by_place[(rid, pos)] = arr[i]
    assert len(over) <= len(ratios) * rt.flipped(dtype), f"{name} {dtype}: {len(over)} of {len(ratios)} positions differ, first {over[:3]}"
    assert float(np.median(ratios)) <= rt.typical(dtype), f"{name} {dtype}: median error {np.median(ratios):.3g} of the largest logit"
    if dtype == "float32":
        pairs = [("whole", "tail"), ("whole", "cut")] + [("w" + rid, rid) for rid in req_tokens if "w" + rid in req_tokens]
        for a, b in pairs:
            for pos in range(len(req_tokens[a])):
                assert np.array_equal(by_place[(a, pos)], by_place[(b, pos)]), \
                    f"{name}: position {pos} of '{b}' differs in bits from the same position of '{a}'"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_reused_slots(dtype, built, plain_logits):
    """A short prompt, then 150 tokens one by one (bfloat16: through captured steps) beside a second request that joins
    late; then both end and a third request takes over their pages and state rows."""
    from jllm_serve_amd.engine.step import StepEntry
    name = "RB"
    model, runner = built(name, dtype, graphs=dtype == "bfloat16")
    a, b, c = rt.prompt(name, 160, seed=5), rt.prompt(name, 70, seed=6), rt.prompt(name, 30, seed=7)
    ra, rb, rc = plain_logits(name, a), plain_logits(name, b), plain_logits(name, c)
    out = runner.step([StepEntry("a", a[:10], range(10))])
    close(out, ra[:10], dtype, "prompt")
    errs, over, rows = [], [], 0

    def held(got, ref, what):  # one row against the plain one; rows beyond the bound are counted (see rt.flipped)
        nonlocal rows
        rows += 1
        err = float((got.double().cpu() - ref).abs().max())
        if err > rt.tolerance(dtype, ref):
            over.append((what, err))
        return err / float(ref.abs().max())
    for i in range(10, 160):
        entries = [StepEntry("a", a[i:i + 1], [0])]
        j = i - 90
        if j == 0:
            entries.append(StepEntry("b", b[:20], [19]))
        elif 0 < j and 20 + j - 1 < 70:
            entries.append(StepEntry("b", b[20 + j - 1:20 + j], [0]))
        out = runner.step(entries)
        errs.append(held(out[0], ra[i], f"a at {i}"))
        if len(entries) == 2:
            held(out[1], rb[19 if j == 0 else 20 + j - 1], f"b beside a at {i}")
    assert len(over) <= rows * rt.flipped(dtype), f"{len(over)} of {rows} rows differ, first {over[:3]}"
    assert float(np.median(errs)) <= rt.typical(dtype), "the error does not grow with the decoded tokens"
    assert float(np.median(errs[-30:])) <= 2 * max(float(np.median(errs[:30])), rt.typical(dtype) / 4)
    if dtype == "bfloat16":
        assert runner.graphs.replays > 100
    runner.finish("a")
    runner.finish("b")
    out = runner.step([StepEntry("c", c, range(len(c)))]).double().cpu()
    bad = [p for p in range(len(c)) if float((out[p] - rc[p]).abs().max()) > rt.tolerance(dtype, rc[p])]
    assert len(bad) <= len(c) * rt.flipped(dtype), f"a request on used pages and used state rows: positions {bad} differ"
    assert float(np.median([float((out[p] - rc[p]).abs().max() / rc[p].abs().max()) for p in range(len(c))])) <= rt.typical(dtype)
    runner.finish("c")
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(dtype, folders):
    """Engine.generate with more requests than places and a pool so small that requests are preempted and computed
    again (their states start from zero again): the tokens of the plain implementation."""
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    from jllm_serve_amd.sampling import SamplingParams
    name = "RA"
    cfg = rt.CONFIGS[name][0]
    w = rt.load_weights(folders[name])
    model = load_model(folders[name], dtype, torch.device(DEV), max_positions=128)
    runner = build_runner(model, page_size=8, pool_tokens=160, max_requests=3)
    eng = Engine(runner, SchedulerConfig(max_batch_tokens=40, prefill_chunk=16, max_positions=128), eos_token_ids=())
    prompts = [rt.prompt(name, n, seed=9) for n in (1, 5, 23, 40, 12)]
    n_new = 12
    got = [r.tokens for r in eng.generate(prompts, SamplingParams.greedy_params(max_tokens=n_new))]
    # random weights make near-ties that rounding decides: every token the engine chose must be one of the plain
    # implementation's best, given the engine's own tokens before it (float32: within its own small bound)
    for p, g in zip(prompts, got):
        assert len(g) == n_new
        ref = P.forward(cfg, w, p + g)
        for i, tok in enumerate(g):
            row = ref[len(p) - 1 + i]
            assert float(row.max() - row[tok]) <= 2 * rt.tolerance(dtype, row), f"token {i} after a prompt of {len(p)}"
    if dtype == "float32":
        want = [P.greedy(cfg, w, p, n_new) for p in prompts]
        assert sum(g == x for g, x in zip(got, want)) >= len(prompts) - 1
    runner.cache.check()
    assert not runner.cache.requests


def test_command_line_runs_the_design(folders, tmp_path):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "jllm"), "run", "--model", folders["RC"], "--dtype", "float32",
                        "--prompt", "3 1 4 1 5", "--max-tokens", "6", "--temp", "0", "--json", "--ctx", "128", "--ignore-eos"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    w = rt.load_weights(folders["RC"])
    ref = P.forward(rt.R_C, w, [3, 1, 4, 1, 5] + out["tokens"])
    assert len(out["tokens"]) == 6
    for i, tok in enumerate(out["tokens"]):
        row = ref[4 + i]
        assert float(row.max() - row[tok]) <= 2 * rt.tolerance("float32", row)
