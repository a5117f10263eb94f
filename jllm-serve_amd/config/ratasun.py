"""The Ratasun design: config.json keys -> ModelConfig.

A Ratasun config names its design with ``"architecture": "Ratasun"`` and lists its layers one by one:

* ``vocab``, ``width``, ``norm.eps`` (of every layer norm and of the RMS norms inside the mixers), ``logit_scale``
  (the logits are the head's product times it);
* ``layers[i]``: ``type`` (the mixer: ``latent_attention``, ``channel_delta`` or ``mamba2``), ``mixer`` (its sizes and
  constants) and ``mlp`` (``{"kind": "moe", ...}`` or null for none); layer i's tensors start with ``l<i>.``, its
  mixer's with ``l<i>.mix.``, its feed-forward's with ``l<i>.mlp.``. A layer has one layer norm ``norm1`` (a weight,
  no bias) whose output both sublayers read: x += mixer(norm1 x) + mlp(norm1 x);
* ``latent_attention``: ``heads``, ``dim`` / ``rot_dim`` (unrotated and rotated query/key entries per head), ``vdim``,
  ``kv_rank``, ``scale`` (used as given), ``rot`` (``base``, ``dims``: neighbouring pairs 2i, 2i + 1 among the first
  ``dims`` entries of the rotated part turn by p base^(-2i / dims)); the query comes straight from the input; every
  earlier key is visible;
* ``channel_delta``: a gated delta rule with ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``conv`` (taps of the
  convolutions in front of q, k and v) and one decay per head and key channel; the decay's and the output gate's inputs
  pass a narrow middle whose size is the tensors' (``a1`` / ``a2``, ``g1`` / ``g2``), so it is read from the checkpoint
  when the weights are loaded;
* ``mamba2``: ``heads``, ``vdim``, ``state``, ``groups``, ``norm_groups``, ``conv``;
* ``mlp``: ``router.experts`` / ``router.top`` / ``router.scale`` / ``router.groups.count`` / ``router.groups.keep``
  (no ``groups``: one group), ``expert.ff``;
* ``loop`` (optional): layers ``start`` .. ``stop`` - 1 run ``times`` times in a row with one set of weights and a
  cache or state per pass; before every pass the stream becomes W [x; x0] with the tensor ``loop.in`` [width, 2 width]
  and x0 the embedding output, then row t of ``loop.step`` [times, width] joins it.
"""
from __future__ import annotations

from typing import Any, List, Mapping

from .registry import register_architecture
from .schema import (ConfigError, GatedDeltaSpec, LatentAttentionSpec, LayerNormSpec, LayerSpec, ModelConfig, ModelNames,
                     RopeSpec, RoutedMoeSpec, ScheduleEntry, StateSpaceSpec, StreamMix, StreamVector)

MIXERS = ("latent_attention", "channel_delta", "mamba2")


def _need(m: Any, key: str, where: str):
    if not isinstance(m, Mapping) or key not in m or m[key] is None:
        raise ConfigError(f"config.json: {where} needs '{key}'")
    return m[key]


def _int(m: Any, key: str, where: str, least: int = 1) -> int:
    v = _need(m, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)) or v != int(v) or int(v) < least:
        raise ConfigError(f"config.json: {where}.{key} must be an integer of at least {least}, got {v!r}")
    return int(v)


def _number(m: Any, key: str, where: str) -> float:
    v = _need(m, key, where)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}.{key} must be a number, got {v!r}")
    return float(v)


def _latent(m: Any, w: str, eps: float, positions: List[RopeSpec]) -> LatentAttentionSpec:
    rot_dim = _int(m, "rot_dim", w)
    rot = _need(m, "rot", w)
    dims = _int(rot, "dims", w + ".rot", least=2)
    if dims % 2 or dims > rot_dim:
        raise ConfigError(f"config.json: {w}.rot.dims={dims} must be even and at most rot_dim={rot_dim}")
    rope = RopeSpec(rotary_dim=dims, theta=_number(rot, "base", w + ".rot"), pairing="interleaved")
    if rope not in positions:
        positions.append(rope)
    return LatentAttentionSpec(heads=_int(m, "heads", w), dim=_int(m, "dim", w), rot_dim=rot_dim, vdim=_int(m, "vdim", w),
                               q_rank=0, kv_rank=_int(m, "kv_rank", w), scale=_number(m, "scale", w), eps=eps, window=0,
                               keep=0, position=positions.index(rope), sink=False, out_gate=False)


def _delta(m: Any, w: str, eps: float) -> GatedDeltaSpec:
    heads, kv_heads = _int(m, "heads", w), _int(m, "kv_heads", w)
    if heads % kv_heads:
        raise ConfigError(f"config.json: {w}: {kv_heads} kv_heads do not divide {heads} heads")
    # the narrow middles' sizes are the tensors' own: -1 = taken from the checkpoint at load
    return GatedDeltaSpec(heads=heads, kv_heads=kv_heads, dim=_int(m, "dim", w), vdim=_int(m, "vdim", w),
                          conv=_int(m, "conv", w), eps=eps, decay="channel", decay_rank=-1, gate_rank=-1, gate_fn="sigmoid")


def _state_space(m: Any, w: str, eps: float) -> StateSpaceSpec:
    heads, groups, norm_groups = _int(m, "heads", w), _int(m, "groups", w), _int(m, "norm_groups", w)
    vdim = _int(m, "vdim", w)
    if heads % groups:
        raise ConfigError(f"config.json: {w}: {groups} groups do not divide {heads} heads")
    if (heads * vdim) % norm_groups:
        raise ConfigError(f"config.json: {w}: {norm_groups} norm_groups do not divide heads x vdim = {heads * vdim}")
    return StateSpaceSpec(heads=heads, vdim=vdim, state=_int(m, "state", w), groups=groups, norm_groups=norm_groups,
                          conv=_int(m, "conv", w), eps=eps)


def _moe(mlp: Any, w: str) -> RoutedMoeSpec:
    kind = _need(mlp, "kind", w)
    if kind != "moe":
        raise ConfigError(f"config.json: {w}.kind '{kind}' is not a feed-forward of this design (moe is)")
    router, expert = _need(mlp, "router", w), _need(mlp, "expert", w)
    experts, top = _int(router, "experts", w + ".router"), _int(router, "top", w + ".router")
    groups = router.get("groups")
    count, keep = (_int(groups, "count", w + ".router.groups"), _int(groups, "keep", w + ".router.groups")) \
        if groups is not None else (1, 1)
    if experts % count or keep > count:
        raise ConfigError(f"config.json: {w}.router: {experts} experts in {count} groups, {keep} kept")
    if top > keep * (experts // count):
        raise ConfigError(f"config.json: {w}.router: top={top} of the {keep * (experts // count)} experts of {keep} groups")
    return RoutedMoeSpec(experts=experts, top=top, hidden=_int(expert, "ff", w + ".expert"),
                         scale=_number(router, "scale", w + ".router"), groups=count, keep=keep, correction=True)


def parse_ratasun(c: Mapping[str, Any], model_type: str, architecture: str) -> ModelConfig:
    vocab = _int(c, "vocab", "config")
    width = _int(c, "width", "config")
    eps = _number(_need(c, "norm", "config"), "eps", "norm")
    raw_layers = _need(c, "layers", "config")
    if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
        raise ConfigError("config.json: layers must be a non-empty list")
    norm = LayerNormSpec(eps=eps, bias=False)
    positions: List[RopeSpec] = []
    layers = []
    for i, layer in enumerate(raw_layers):
        where = f"layers[{i}]"
        kind = _need(layer, "type", where)
        m = _need(layer, "mixer", where)
        w = where + ".mixer"
        if kind == "latent_attention":
            mixer, mixer_prefix = _latent(m, w, eps, positions), ""  # its names carry "mix." themselves
        elif kind == "channel_delta":
            mixer, mixer_prefix = _delta(m, w, eps), "mix"
        elif kind == "mamba2":
            mixer, mixer_prefix = _state_space(m, w, eps), "mix"
        else:
            raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design ({', '.join(MIXERS)})")
        mlp = layer.get("mlp")
        ffn = _moe(mlp, where + ".mlp") if mlp is not None else None
        layers.append(LayerSpec(mixer=mixer, ffn=ffn, norm=norm, prefix=f"l{i}", arrangement="parallel",
                                norm_in_name="norm1", name_ending="", mixer_prefix=mixer_prefix))
    n = len(layers)
    loop = c.get("loop")
    if loop is None:
        schedule = [ScheduleEntry(i) for i in range(n)]
        looped = ""
    else:
        start, stop, times = _int(loop, "start", "loop", 0), _int(loop, "stop", "loop", 0), _int(loop, "times", "loop", 0)
        if not start <= stop <= n:
            raise ConfigError(f"config.json: loop runs layers {start} .. {stop} - 1 of {n}")
        schedule = [ScheduleEntry(i) for i in range(start)]
        for t in range(times):
            for i in range(start, stop):
                first = i == start
                schedule.append(ScheduleEntry(i, add_before=StreamVector("loop.step", times, t) if first else None,
                                              mix_before=StreamMix("loop.in") if first else None))
        schedule += [ScheduleEntry(i) for i in range(stop, n)]
        looped = f" loop={start}..{stop - 1}x{times}"
    kinds = [l["type"] for l in raw_layers]
    description = (f"{architecture} width={width} layers={n} runs={len(schedule)} vocab={vocab} "
                   + " ".join(f"{k}={kinds.count(k)}" for k in MIXERS) + looped)
    longest = c.get("max_positions")
    scale = c.get("logit_scale")
    return ModelConfig(
        architecture=architecture, model_type=model_type, hidden=width, vocab=vocab, final_norm=norm,
        layers=tuple(layers), positions=tuple(positions), schedule=tuple(schedule), tie_embeddings=False,
        max_positions=int(longest) if isinstance(longest, int) and longest > 0 else 4096,
        logit_scale=_number(c, "logit_scale", "config") if scale is not None else 1.0,
        description=description, names=ModelNames(embed="embed", final_norm="final.norm", head="head"), raw=dict(c))


register_architecture("ratasun", "Ratasun", parse_ratasun, replace=True)
