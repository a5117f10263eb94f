"""Kebepel on the GPU against the plain implementation (tests/plain/kebepel_plain.py): every mechanism alone, the
attention kernels on crafted keys (far keys, page borders, NaN in unused places), the delta rule on crafted memories
(a value written first and read hundreds of tokens later), whole prompts against token-by-token decoding, portions
down to two tokens, mixed batches on a pool that is used again, the stream after every layer run, long decoding
through captured steps, greedy generation through the engine, and the replay program."""
import json
import os
import random

import numpy as np
import pytest
import torch

import kebepel_tiny as kt
import replay
from plain import kebepel_plain as P

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    return {name: kt.write_model(str(tmp_path_factory.mktemp("kebepel_" + name)), cfg, seed)
            for name, (cfg, seed, page) in kt.CONFIGS.items()}


@pytest.fixture(scope="module")
def built(folders):
    from jllm_serve_amd.engine import build_runner, load_model
    cache = {}

    def get(name, dtype, graphs=False):
        if (name, dtype, graphs) not in cache:
            model = load_model(folders[name], dtype, torch.device(DEV), max_positions=1024)
            cache[(name, dtype, graphs)] = (model, build_runner(model, page_size=kt.CONFIGS[name][2], pool_tokens=1024,
                                                                max_requests=4, graphs=graphs))
        return cache[(name, dtype, graphs)]
    return get


@pytest.fixture(scope="module")
def plain_logits(folders):
    memo = {}

    def get(name, tokens):
        key = (name, tuple(tokens))
        if key not in memo:
            memo[key] = P.forward(kt.CONFIGS[name][0], kt.load_weights(folders[name]), list(tokens))
        return memo[key]
    return get


def close(got, want, dtype, what=""):
    err = float((got.double().cpu() - want).abs().max())
    assert err <= kt.tolerance(dtype, want), f"{what}: {err} > {kt.tolerance(dtype, want)}"


def act_type(dtype):
    return torch.float32 if dtype == "float32" else torch.bfloat16


# ------------------------------------------------------------------------------------------------ mechanisms alone


@pytest.mark.parametrize("width", [70, 256, 1100, 5000])
def test_layer_norm_seam(width):
    """The seam kernel's three parts alone and together, one and two branches, fp32 and bf16 operands, a row list."""
    from jllm_serve_amd.kernels import ops
    torch.manual_seed(width)
    n, eps = 9, 1e-5
    for wt in (torch.float32, torch.bfloat16):
        x = torch.randn(n, width) * 3 + 0.7
        a, a2 = torch.randn(n, width) * 2, torch.randn(n, width)
        vec = [(torch.randn(width) * 0.5 + (1 if i % 2 == 0 else 0)).to(wt) for i in range(5)]
        w1, b1, w2, b2, add = vec
        d = [v.double() for v in vec]
        xd = x.to(DEV)
        out = ops.layernorm_seam(xd, eps, nxt=(w2.to(DEV), b2.to(DEV)), out_dtype=torch.float32)
        assert torch.equal(xd.cpu(), x)
        assert torch.allclose(out.cpu().double(), P.layer_norm(x.double(), d[2], d[3], eps), atol=2e-5)
        rows = torch.tensor([7, 0, 3], dtype=torch.int32)
        out = ops.layernorm_seam(xd, eps, nxt=(w2.to(DEV), b2.to(DEV)), out_dtype=torch.float32, rows=rows.to(DEV))
        assert torch.allclose(out.cpu().double(), P.layer_norm(x.double()[rows.long()], d[2], d[3], eps), atol=2e-5)
        for at in (torch.float32, torch.bfloat16):
            aa, aa2 = a.to(at), a2.to(at)
            want_x = x.double() + P.layer_norm(0.6 * aa.double() + 1.3 * aa2.double(), d[0], d[1], eps) + d[4]
            out = ops.layernorm_seam(xd, eps, a=aa.to(DEV), a2=aa2.to(DEV), s1=0.6, s2=1.3, post=(w1.to(DEV), b1.to(DEV)),
                                     add_vec=add.to(DEV), nxt=(w2.to(DEV), b2.to(DEV)), out_dtype=torch.float32)
            assert torch.allclose(xd.cpu().double(), want_x, atol=5e-5)
            assert torch.allclose(out.cpu().double(), P.layer_norm(want_x, d[2], d[3], eps), atol=5e-5)
            xd = x.to(DEV)
            ops.layernorm_seam(xd, eps, a=aa.to(DEV), post=(w1.to(DEV), b1.to(DEV)))
            assert torch.allclose(xd.cpu().double(), x.double() + P.layer_norm(aa.double(), d[0], d[1], eps), atol=5e-5)
            xd = x.to(DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["KA", "KB", "KC"])
def test_mixers_alone_through_cache_and_state(name, dtype, built, folders):
    """Every layer's mixer on random inputs: a portion from position 0, further portions and single rows from the
    cache and the state. The branches of a parallel mixer are also run each alone."""
    from jllm_serve_amd.engine.step import StepEntry
    cfg = kt.CONFIGS[name][0]
    eps = cfg["norm"]["eps"]
    w = kt.load_weights(folders[name])
    model, runner = built(name, dtype)
    act = act_type(dtype)
    torch.manual_seed(4)
    cuts = (29, 6, 1, 1, 2, 17)
    T = sum(cuts)
    runs = P.layer_runs(cfg)
    xs = [(torch.randn(T, cfg["width"]) * 0.8).to(act) for _ in runs]
    pos = torch.arange(T)
    want = [P.mixer(xs[r].double(), w, i, cfg["layers"][i], eps, pos) for r, (i, _) in enumerate(runs)]
    got = [[] for _ in runs]
    at = 0
    for n in cuts:
        ctx = runner.prepare([StepEntry("mix", [0] * n, [])])
        for r, (i, _) in enumerate(runs):
            res = torch.zeros(n, cfg["width"], device=DEV)
            model.layers[i].mixer.forward(xs[r][at:at + n].to(DEV), res, ctx, runner.cache.slots[r])
            got[r].append(res.cpu())
        runner.cache.commit("mix", n)
        at += n
    runner.finish("mix")
    for r, (i, _) in enumerate(runs):
        close(torch.cat(got[r]), want[r], dtype, f"{name} run {r} (layer {i}) mixer")
    # the two sides of a parallel mixer, each alone from a fresh request
    for r, (i, _) in enumerate(runs):
        layer = cfg["layers"][i]
        if layer["type"] != "parallel":
            continue
        m = layer["mixer"]
        from jllm_serve_amd.kernels import ops
        ctx = runner.prepare([StepEntry("side", [0] * T, [])])
        part = model.layers[i].mixer
        assert part.fused, "the two sides share their input and output products"
        y = ops.gemm(xs[r].to(DEV), part.w_in, bias=part.b_in, out_dtype=act, exact=dtype == "float32")
        outs, at = [], 0
        for j, b in enumerate(part.branches):
            lo, hi = part._cols[j]
            heads = b.heads_rows_from(y[:, lo:hi], ctx, part._slot(runner.cache.slots[r], j))
            outs.append(ops.gemm(heads, part.w_o[:, at:at + b.heads_width].contiguous(), out_dtype=torch.float32, exact=dtype == "float32"))
            at += b.heads_width
        runner.cache.commit("side", T)
        runner.finish("side")
        close(outs[0], P.capped_attention(xs[r].double(), w, f"l{i}.mix.left", m["left"], eps, pos), dtype, f"{name} layer {i} left")
        close(outs[1], P.gated_delta_mixer(xs[r].double(), w, f"l{i}.mix.right", m["right"], eps), dtype, f"{name} layer {i} right")


def _pages(T, page, n_pages, seed):
    """A block table for one request of T positions over shuffled pages; the other pages stay unused."""
    rng = random.Random(seed)
    ids = list(range(n_pages))
    rng.shuffle(ids)
    need = -(-T // page)
    return ids[:need]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("maps, softcap", [(1, 0.0), (1, 4.0), (2, 0.0)])
def test_attention_kernel_on_crafted_keys(dtype, maps, softcap):
    """One key is made to dominate a head's scores (a query and a key scaled up along one direction): the first key of
    the request, the last place of a page, the first place of the next page, and a key hundreds of positions back; the
    row must return that key's value. Pages are shuffled and every place no position owns holds NaN. The same rows
    as one long portion and as single rows."""
    from jllm_serve_amd.kernels import ops
    act = act_type(dtype)
    torch.manual_seed(11 + maps)
    H, G, dk, dv, page, T = 4, 2, 32, 40, 16, 700  # sizes the matrix-core kernel takes, in bfloat16
    QS, KS = H * maps, G * maps
    n_pages = 64
    table = _pages(T, page, n_pages, 5)
    q = torch.randn(T, QS, dk) * 0.3
    k = torch.randn(T, KS, dk) * 0.3
    v = torch.randn(T, G, dv)
    targets = {699: 0, 650: 15, 640: 16, 500: 31, 300: 299, 17: 17}  # row -> the key it must find
    for e, (row, key) in enumerate(targets.items()):  # each pair along a direction of its own
        q[:, :, e] = 0.0
        k[:, :, e] = 0.0
    for e, (row, key) in enumerate(targets.items()):
        q[row, :, e] = 9.0
        k[key, :, e] = 9.0
    scale = 1.0
    q, k, v = q.to(act), k.to(act), v.to(act)
    kc = torch.full((n_pages, KS, page, dk), float("nan"), dtype=act)
    vc = torch.full((n_pages, G, page, dv), float("nan"), dtype=act)
    for p in range(T):
        kc[table[p // page], :, p % page] = k[p]
        vc[table[p // page], :, p % page] = v[p]
    # plain: every query slot alone
    per = maps * (H // G)
    qd, kd, vd = q.double(), k.double(), v.double()
    want = torch.zeros(T, QS, dv, dtype=torch.float64)
    for s in range(QS):
        vh = s // per
        ks = vh * maps + s % maps
        want[:, s:s + 1] = P.causal_softmax_attention(qd[:, s:s + 1], kd[:, ks:ks + 1], vd[:, vh:vh + 1], scale, softcap)
    bt = torch.tensor([table + [0] * 3], dtype=torch.int32, device=DEV)
    pos = torch.arange(T, dtype=torch.int32, device=DEV)
    req = torch.zeros(T, dtype=torch.int32, device=DEV)
    tiles = [v for r0 in range(0, T, 128) for v in (0, r0, min(128, T - r0), r0)]
    for exact in ((True,) if dtype == "float32" else (True, False)):
        ops.reset_stats()
        got = ops.attention_dv(q.reshape(T, -1).to(DEV), kc.to(DEV), vc.to(DEV), bt, req, pos, H, G, maps, dk, dv, scale,
                               softcap=softcap, out_dtype=torch.float32, exact=exact,
                               meta={"max_context": T, "requests": 1, "rows": T, "n_tiles": len(tiles) // 4,
                                     "tiles_dev": torch.tensor(tiles, dtype=torch.int32, device=DEV)}).cpu().view(T, QS, dv)
        assert exact or ops.stats()["ran"].get("jllm_attention_dv_bf16") == 1, "the matrix-core kernel did not take the step"
        assert bool(torch.isfinite(got).all()), "a place that no position owns was read"
        tol = 2e-5 if dtype == "float32" else 2e-2
        assert float((got.double() - want).abs().max()) <= tol * float(want.abs().max())
        if softcap == 0.0:
            for row, key in targets.items():
                if key == row:
                    continue
                vh = torch.arange(QS) // per
                assert float((got[row].double() - vd[key][vh]).abs().max()) < 0.05, f"row {row} did not find key {key}"
        # the last rows again, each as a single row of its own step
        rows = sorted(targets)
        sel = torch.tensor(rows, device=DEV)
        one = ops.attention_dv(q.reshape(T, -1).to(DEV)[sel].contiguous(), kc.to(DEV), vc.to(DEV), bt.repeat(len(rows), 1),
                               torch.arange(len(rows), dtype=torch.int32, device=DEV), pos[sel].contiguous(), H, G, maps, dk, dv,
                               scale, softcap=softcap, out_dtype=torch.float32, exact=exact,
                               meta={"max_context": T, "requests": len(rows), "rows": len(rows), "n_tiles": len(rows), "single_rows": True,
                                     "tiles_dev": torch.tensor([v for i in range(len(rows)) for v in (i, i, 1, -1)],
                                                               dtype=torch.int32, device=DEV)}).cpu()
        assert float((one.view(len(rows), QS, dv).double() - want[rows]).abs().max()) <= tol * float(want.abs().max())
        if not exact:  # the same rows with the merge of their key ranges left to the kernel that finishes the heads
            meta = {"max_context": T, "requests": len(rows), "rows": len(rows), "n_tiles": len(rows), "single_rows": True,
                    "tiles_dev": torch.tensor([v for i in range(len(rows)) for v in (i, i, 1, -1)], dtype=torch.int32, device=DEV)}
            parts = ops.attention_dv(q.reshape(T, -1).to(DEV)[sel].contiguous(), kc.to(DEV), vc.to(DEV), bt.repeat(len(rows), 1),
                                     torch.arange(len(rows), dtype=torch.int32, device=DEV), pos[sel].contiguous(), H, G, maps, dk,
                                     dv, scale, softcap=softcap, out_dtype=torch.float32, meta=meta, defer_merge=True)
            assert isinstance(parts, ops.SplitHeads) and parts.splits > 1, "the rows' keys were not shared out"
            kw = dict(lam=0.3, normed=maps == 2, eps=1e-5, norm_mul=0.7)
            merged_late = ops.heads_finish(parts, H, maps, dv, torch.float32, **kw).cpu()
            merged_first = ops.heads_finish(one.to(DEV), H, maps, dv, torch.float32, **kw).cpu()
            assert torch.allclose(merged_late, merged_first, atol=1e-5, rtol=1e-5)


def test_qkv_prepare_options():
    """Whole-projection norm, pair rotation over a part of the head, the query temperature at its steps, and the
    store into shuffled pages, each alone and together; rows without a place store nothing."""
    from jllm_serve_amd.kernels import ops
    torch.manual_seed(3)
    H, G, maps, dk, dv, page, T = 3, 1, 2, 10, 7, 4, 23
    QS, KS = H * maps, G * maps
    nq, nk, nv = QS * dk, KS * dk, G * dv
    y = torch.randn(T, nq + nk + nv + 5)
    gq, gk = torch.randn(nq) * 0.2 + 1, torch.randn(nk) * 0.2 + 1
    rot = {"base": 50.0, "dims": 6, "scaling": {"factor": 3.0, "original": 8, "fast": 4.0, "slow": 1.0}}
    f, amp = P.yarn_frequencies(rot["dims"], rot["base"], rot["scaling"])
    positions = torch.arange(5, 5 + T)
    ang = torch.arange(64, dtype=torch.float64)[:, None] * f[None]
    cos, sin = (torch.cos(ang) * amp).float(), (torch.sin(ang) * amp).float()
    slots = torch.randperm(8 * page)[:T].int()
    slots[4] = -1
    for norm, rotate, temp in ((True, False, None), (False, True, None), (False, False, (0.6, 3)), (True, True, (0.6, 3))):
        yd = y.clone().to(DEV)
        kc = torch.zeros(8, KS, page, dk, device=DEV)
        vc = torch.zeros(8, G, page, dv, device=DEV)
        ops.qkv_prepare(yd, positions.int().to(DEV), slots.to(DEV), H, G, maps, dk, dv, kc, vc,
                        gq=gq.to(DEV) if norm else None, gk=gk.to(DEV) if norm else None, eps=1e-5,
                        cos=cos.to(DEV) if rotate else None, sin=sin.to(DEV) if rotate else None,
                        rot_dims=rot["dims"] if rotate else 0, temp_coef=temp[0] if temp else 0.0, temp_every=temp[1] if temp else 0)
        q, k = y[:, :nq].double(), y[:, nq:nq + nk].double()
        if norm:
            q, k = P.rms(q, 1e-5) * gq.double(), P.rms(k, 1e-5) * gk.double()
        q, k = q.view(T, QS, dk), k.view(T, KS, dk)
        if rotate:
            q, k = P.rotate_pairs(q, positions, rot), P.rotate_pairs(k, positions, rot)
        if temp:
            q = q * P.query_temperature(positions, *temp)[:, None, None]
        assert torch.allclose(yd[:, :nq].cpu().double(), q.reshape(T, nq), atol=1e-5)
        assert torch.equal(yd[:, nq:].cpu(), y[:, nq:])
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            assert torch.allclose(kc[s // page, :, s % page].cpu().double(), k[t], atol=1e-5)
            assert torch.equal(vc[s // page, :, s % page].cpu(), y[t, nq + nk:nq + nk + nv].view(G, dv))
        assert int((kc != 0).any(dim=-1).sum()) == (T - 1) * KS


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, dk, dv", [(2, 1, 16, 8), (3, 3, 40, 24), (2, 2, 128, 128), (1, 1, 7, 5), (2, 1, 200, 40)])
def test_delta_rule_recalls_a_far_memory(dtype, H, G, dk, dv):
    """The kernel against the plain recurrence over 600 tokens cut into portions, with inputs chosen so that a fault
    shows: the first token writes a value along a key that no later token touches, nothing decays, and the last token
    asks for it; a second request beside it decays fast. Then the same tokens whole: the same bits."""
    from jllm_serve_amd.kernels import ops
    act = act_type(dtype)
    torch.manual_seed(dk)
    T, eps = 600, 1e-5
    C = 2 * G * dk + H * dv

    def make(slow):
        qkv = torch.randn(T, C)
        k = qkv[:, G * dk:2 * G * dk].view(T, G, dk)
        q = qkv[:, :G * dk].view(T, G, dk)
        k[1:, :, 0] = 0.0  # later keys have no part along the first direction ...
        k[0] = 0.0
        k[0, :, 0] = 3.0  # ... which the first key is
        q[-1] = 0.0
        q[-1, :, 0] = 2.0  # the last query asks along it
        proj = torch.randn(T, H * dv + 2 * H + 3)
        proj[:, H * dv:H * dv + H] = -30.0 if slow else 2.0  # a: softplus(-30 + dt_bias) ~ 0: no decay
        proj[0, H * dv + H:H * dv + 2 * H] = 30.0  # b of the first token: written in full
        return qkv.to(act), proj.to(act)

    a_log, dt_bias, gain = torch.randn(H) * 0.3, torch.randn(H) * 0.3, torch.randn(dv) * 0.2 + 1

    def plain(qkv, proj):
        qkv, proj = qkv.double(), proj.double()
        rep = H // G
        q = (P.unit(qkv[:, :G * dk].view(T, G, dk)) * dk ** -0.5).repeat_interleave(rep, 1)
        k = P.unit(qkv[:, G * dk:2 * G * dk].view(T, G, dk)).repeat_interleave(rep, 1)
        v = qkv[:, 2 * G * dk:].view(T, H, dv)
        beta = torch.sigmoid(proj[:, H * dv + H:H * dv + 2 * H])
        g = torch.exp(-torch.exp(a_log.double()) * P.softplus(proj[:, H * dv:H * dv + H] + dt_bias.double()))
        o = P.delta_rule(q, k, v, beta, g)
        o = P.rms(o, eps) * gain.double()
        return o.reshape(T, H * dv) * P.silu(proj[:, :H * dv]), o

    reqs = [make(True), make(False)]
    wants = [plain(*r) for r in reqs]
    # the far memory is what the last row of the first request reads: S^T q = v_0 * (k_0 . q) up to the heads' norm
    v0 = reqs[0][0].double()[0, 2 * G * dk:].view(H, dv)
    assert torch.allclose(wants[0][1][-1], P.rms(v0 * dk ** -0.5, eps) * gain.double(), atol=1e-3)
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
            row_req = torch.tensor([0] * n + [1] * n, dtype=torch.int32, device=DEV)
            pd = dev(proj)
            raw = ops.gated_delta(dev(qkv), pd, H * dv, H * dv + H, dev(a_log), dev(dt_bias), state, row_req, slots, 2, H, G, dk, dv)
            out = ops.heads_finish(raw, H, 1, dv, act, normed=True, eps=eps, gain=dev(gain), gate=pd[:, :H * dv], gate_fn="silu").cpu()
            got[0].append(out[:n])
            got[1].append(out[n:])
            at += n
        assert float(state[[0, 2, 4]].abs().max()) == 0.0, "a state row of no request was written"
        results.append([torch.cat(g) for g in got])
        for i in range(2):
            tol = 3e-5 if dtype == "float32" else 3e-2
            err = float((results[-1][i].double() - wants[i][0]).abs().max())
            assert err <= tol * max(1.0, float(wants[i][0].abs().max())), f"request {i} cut {cuts}: {err}"
    for i in range(2):
        assert torch.equal(results[0][i], results[1][i]), "the recurrence depends on how the tokens were cut"


@pytest.mark.parametrize("taps", [1, 2, 4, 7])
def test_short_convolution_across_steps_and_slots(taps):
    """Two requests of unequal lengths in steps of unequal portions (down to one row, shorter than the taps), their
    state rows used again by a third request after they end."""
    from jllm_serve_amd.kernels import ops
    torch.manual_seed(taps)
    C = 37
    w = torch.randn(C, taps)
    xa, xb, xc = torch.randn(40, C + 3), torch.randn(23, C + 3), torch.randn(9, C + 3)
    want = {n: P.silu(P.short_convolution(x[:, :C].double(), w.double())) for n, x in (("a", xa), ("b", xb), ("c", xc))}
    state = torch.full((4, max(taps - 1, 1), C), 0.0, device=DEV)
    slots = torch.tensor([2, 0], dtype=torch.int32, device=DEV)
    got = {"a": [], "b": [], "c": []}
    pa = pb = 0
    for na, nb in ((9, 5), (1, 1), (2, 11), (17, 1), (1, 2), (10, 3)):
        x = torch.cat([xa[pa:pa + na], xb[pb:pb + nb]]).to(DEV)
        req = torch.tensor([0] * na + [1] * nb, dtype=torch.int32, device=DEV)
        y = ops.short_conv(x, w.to(DEV), state, req, slots, 2).cpu()
        got["a"].append(y[:na])
        got["b"].append(y[na:])
        pa += na
        pb += nb
    assert pa == 40 and pb == 23
    state[2].zero_()  # what the cache manager does when a slot is handed to a new request
    y = ops.short_conv(xc.to(DEV), w.to(DEV), state, torch.zeros(9, dtype=torch.int32, device=DEV),
                       torch.tensor([2], dtype=torch.int32, device=DEV), 1).cpu()
    got["c"].append(y)
    for n in got:
        assert torch.allclose(torch.cat(got[n]).double(), want[n], atol=1e-5), n


# ------------------------------------------------------------------------------------------------ whole models


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["KA", "KB", "KC"])
def test_stream_after_every_run(name, dtype, built, folders):
    """The residual stream after every layer run against the plain one (the loop's vector joins before a pass)."""
    from jllm_serve_amd.engine.step import StepEntry
    model, runner = built(name, dtype)
    cfg = kt.CONFIGS[name][0]
    toks = kt.prompt(name, 37)
    streams = []
    P.forward(cfg, kt.load_weights(folders[name]), toks, streams)
    got = []
    model.watch = lambda run, x: got.append(x.detach().cpu().clone())
    try:
        runner.step([StepEntry("w", toks, [])])
    finally:
        model.watch = None
        runner.finish("w")
    assert len(got) == len(streams) == len(P.layer_runs(cfg))
    for r, (g, s) in enumerate(zip(got, streams)):
        tol = (2e-5 if dtype == "float32" else 4e-2) * float(s.abs().max())
        assert float((g.double() - s).abs().max()) <= tol, f"{name} {dtype}: the stream after run {r}"


def build_trace(name):
    t = replay.Trace(page=kt.CONFIGS[name][2])
    lens = [1, 2, 3, 9, 40, 131]
    toks = {f"r{n}": kt.prompt(name, n) for n in lens}
    longest = toks[f"r{lens[-1]}"]
    replay.whole(t, "whole", longest)
    replay.tail_one_by_one(t, "tail", longest, tail=40)
    replay.portions(t, "cut", longest)
    for rid, tk in toks.items():
        replay.whole(t, "w" + rid, tk)
    more = dict(toks)
    more["x1"] = kt.prompt(name, 45, seed=1)
    more["x2"] = kt.prompt(name, 2, seed=2)
    more["x3"] = kt.prompt(name, 66, seed=3)
    replay.mixed(t, more, seed=len(name))
    req_tokens = {"whole": longest, "tail": longest, "cut": longest, **{"w" + k: v for k, v in toks.items()}, **more}
    return t, req_tokens


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["KA", "KB", "KC"])
def test_replay_matches_plain(name, dtype, folders, plain_logits, tmp_path):
    """bin/trace_run: whole, the last 40 tokens one by one, portions down to two tokens, mixed batches with at most four
    live requests on a pool exactly as large as the busiest step (pages and state slots are used again; the free pages
    are reordered before every step). In float32 a position's logits are the same bits however it was reached."""
    cfg, _, page = kt.CONFIGS[name]
    trace, req_tokens = build_trace(name)
    got = replay.run(folders[name], dtype, trace, str(tmp_path), page_size=page, max_tokens=trace.peak, shuffle_free=len(name) + 7)
    V = cfg["vocab"]
    by_place = {}
    ratios = []
    for step, rows in trace.rows.items():
        arr = got[step].reshape(len(rows), V)
        for i, (rid, pos) in enumerate(rows):
            ref = plain_logits(name, req_tokens[rid])[pos]
            tol = kt.tolerance(dtype, ref)
            err = float(np.abs(arr[i].astype(np.float64) - ref.numpy()).max())
            assert err <= tol, f"{name} {dtype}: step {step} request {rid} position {pos}: |diff| {err:.3g} > {tol:.3g}"
            ratios.append(err / float(ref.abs().max()))
            by_place[(rid, pos)] = arr[i]
    assert float(np.median(ratios)) <= kt.typical(dtype), f"{name} {dtype}: median error {np.median(ratios):.3g} of the largest logit"
    if dtype == "float32":
        pairs = [("whole", "tail"), ("whole", "cut")] + [("w" + rid, rid) for rid in req_tokens if "w" + rid in req_tokens]
        for a, b in pairs:
            for pos in range(len(req_tokens[a])):
                assert np.array_equal(by_place[(a, pos)], by_place[(b, pos)]), \
                    f"{name}: position {pos} of '{b}' differs in bits from the same position of '{a}'"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_reused_slots(dtype, built, plain_logits):
    """A short prompt, then 150 tokens one by one (bfloat16: through captured steps) beside a second request that joins
    late; then both end and a third request takes over their pages and state row."""
    from jllm_serve_amd.engine.step import StepEntry
    name = "KB"
    model, runner = built(name, dtype, graphs=dtype == "bfloat16")
    a, b, c = kt.prompt(name, 160, seed=5), kt.prompt(name, 70, seed=6), kt.prompt(name, 30, seed=7)
    ra, rb, rc = plain_logits(name, a), plain_logits(name, b), plain_logits(name, c)
    out = runner.step([StepEntry("a", a[:10], range(10))])
    close(out, ra[:10], dtype, "prompt")
    for i in range(10, 160):
        entries = [StepEntry("a", a[i:i + 1], [0])]
        j = i - 90
        if j == 0:
            entries.append(StepEntry("b", b[:20], [19]))
        elif 0 < j and 20 + j - 1 < 70:
            entries.append(StepEntry("b", b[20 + j - 1:20 + j], [0]))
        out = runner.step(entries)
        close(out[0], ra[i], dtype, f"a at {i}")
        if len(entries) == 2:
            close(out[1], rb[19 if j == 0 else 20 + j - 1], dtype, f"b beside a at {i}")
    if dtype == "bfloat16":
        assert runner.graphs.replays > 100
    runner.finish("a")
    runner.finish("b")
    out = runner.step([StepEntry("c", c, range(len(c)))])
    close(out, rc, dtype, "a request on used pages and a used state row")
    runner.finish("c")
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(dtype, folders):
    """Engine.generate with more requests than places and a pool so small that requests are preempted and computed
    again (their state starts from zero again): the tokens of the plain implementation."""
    from jllm_serve_amd.engine import Engine, SchedulerConfig, build_runner, load_model
    from jllm_serve_amd.sampling import SamplingParams
    name = "KA"
    cfg = kt.CONFIGS[name][0]
    w = kt.load_weights(folders[name])
    model = load_model(folders[name], dtype, torch.device(DEV), max_positions=128)
    runner = build_runner(model, page_size=8, pool_tokens=160, max_requests=3)
    eng = Engine(runner, SchedulerConfig(max_batch_tokens=40, prefill_chunk=16, max_positions=128), eos_token_ids=())
    prompts = [kt.prompt(name, n, seed=9) for n in (1, 5, 23, 40, 12)]
    n_new = 12
    got = [r.tokens for r in eng.generate(prompts, SamplingParams.greedy_params(max_tokens=n_new))]
    want = [P.greedy(cfg, w, p, n_new) for p in prompts]
    if dtype == "float32":
        assert got == want
    else:
        # random weights make near-ties that rounding decides: every token the engine chose must be one of the plain
        # implementation's best, given the engine's own tokens before it
        for p, g in zip(prompts, got):
            ref = P.forward(cfg, w, p + g)
            for i, tok in enumerate(g):
                row = ref[len(p) - 1 + i]
                assert float(row.max() - row[tok]) <= 2 * kt.tolerance(dtype, row), f"token {i} after a prompt of {len(p)}"
    runner.cache.check()
    assert not runner.cache.requests


def test_command_line_runs_the_design(folders, tmp_path):
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "jllm"), "run", "--model", folders["KC"], "--dtype", "float32",
                        "--prompt", "3 1 4 1 5", "--max-tokens", "6", "--temp", "0", "--json", "--ctx", "128", "--ignore-eos"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["tokens"] == P.greedy(kt.K_C, kt.load_weights(folders["KC"]), [3, 1, 4, 1, 5], 6)
