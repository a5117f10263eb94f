"""The Pivipel design: config.json keys -> ModelConfig.

A Pivipel config names its design with ``"architecture": "Pivipel"`` and lists its layers one by one:

* ``vocab``, ``width``, ``max_positions`` (rows of the learned position table ``pos``, added to the embedded rows),
  ``norm.eps`` (of the RMS norms inside the mixers; the model's own norm is Dynamic Tanh and has none), ``streams``
  (residual streams per row; without the key there is one stream and the plain residual sum);
* ``layers[i]``: ``type`` (the mixer: ``attention`` or ``attention_2``), ``mixer`` (its sizes and constants), ``mlp``
  (``{"kind": "dense" | "moe", ...}`` or null for none) and optionally ``weights_of``: j, a layer without tensors of
  its own that runs with layer j's (with a cache of its own). Layer i's tensors start with ``l<i>.``, its mixer's with
  ``l<i>.mix.``, its feed-forward's with ``l<i>.mlp.``, its norms are ``norm1`` / ``norm2`` (each with ``.b`` and
  ``.alpha``), its stream weights ``hc1.*`` / ``hc2.*``;
* both mixers: ``heads``, ``kv_heads``, ``dim`` (query/key size per head), ``vdim``, ``scale`` (used as given),
  ``mask.size`` (the sliding window: the query sees itself and the size - 1 keys before it);
* ``attention``: ``rot`` (``base``, ``dims``: the pairs (i, i + dims / 2) among the first ``dims`` entries of every head
  turn by p f_i, f_i = base^(-2i / dims); ``scaling`` with ``factor`` / ``low`` / ``high`` / ``original`` rescales the
  frequencies by wavelength), a learned sink per head in the softmax's denominator, one output gate per head;
* ``attention_2``: RMS norm of every q and k head (gains ``q.norm`` / ``k.norm``), no rotation, ``mask.keep_first`` (that
  many first keys stay visible beside the window), an output gate per channel;
* ``mlp`` dense: ``ff``, ``limit``; moe: ``router.experts`` / ``top`` / ``scale`` / ``groups.count`` / ``groups.keep`` (no
  ``groups``: one group), ``expert.ff`` / ``expert.limit``, ``shared.ff`` / ``shared.limit`` (optional: a shared expert
  with a gate per token).

The head is the embedding table.
"""
from __future__ import annotations

from typing import Any, List, Mapping

from .registry import register_architecture
from .schema import (ConfigError, DynTanhSpec, GatedMlpNames, GatedMlpSpec, LayerSpec, LearnedPositionSpec, ModelConfig,
                     ModelNames, RopeScaling, RopeSpec, RoutedMoeNames, RoutedMoeSpec, ScheduleEntry, WideAttentionNames,
                     WideAttentionSpec)

MIXERS = ("attention", "attention_2")


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


def _rope(rot: Any, w: str, dim: int) -> RopeSpec:
    dims = _int(rot, "dims", w, least=2)
    if dims % 2 or dims > dim:
        raise ConfigError(f"config.json: {w}.dims={dims} must be even and at most dim={dim}")
    sc = rot.get("scaling")
    scaling = RopeScaling()
    if sc is not None:
        scaling = RopeScaling(kind="llama3", factor=_number(sc, "factor", w + ".scaling"),
                              original_max_positions=_int(sc, "original", w + ".scaling"),
                              low_freq_factor=_number(sc, "low", w + ".scaling"),
                              high_freq_factor=_number(sc, "high", w + ".scaling"))
    return RopeSpec(rotary_dim=dims, theta=_number(rot, "base", w), scaling=scaling, pairing="half")


def _mixer(kind: str, m: Any, w: str, eps: float, positions: List[Any]) -> WideAttentionSpec:
    heads, kv_heads = _int(m, "heads", w), _int(m, "kv_heads", w)
    if heads % kv_heads:
        raise ConfigError(f"config.json: {w}: {kv_heads} kv_heads do not divide {heads} heads")
    dim, vdim = _int(m, "dim", w), _int(m, "vdim", w)
    mask = m.get("mask") or {}
    window = _int(mask, "size", w + ".mask") if "size" in mask else 0
    common = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=_number(m, "scale", w), eps=eps, bias=False,
                  out_gate=True, window=window)
    if kind == "attention":
        position = None
        if m.get("rot") is not None:
            rope = _rope(m["rot"], w + ".rot", dim)
            if rope not in positions:
                positions.append(rope)
            position = positions.index(rope)
        return WideAttentionSpec(position=position, sink=True, gate_per_head=True, names=WideAttentionNames(), **common)
    keep = _int(mask, "keep_first", w + ".mask", least=0) if "keep_first" in mask else 0
    return WideAttentionSpec(position=None, qk_norm="head", keep_first=keep if window > 0 else 0, names=WideAttentionNames(),
                             **common)


def _dense(m: Any, w: str, under: str) -> GatedMlpSpec:
    return GatedMlpSpec(hidden=_int(m, "ff", w), activation="swish_clamped", limit=_number(m, "limit", w),
                        names=GatedMlpNames(gate=f"{under}.gate", up=f"{under}.up", down=f"{under}.down", ending=""))


def _ffn(mlp: Any, w: str):
    kind = _need(mlp, "kind", w)
    if kind == "dense":
        return _dense(mlp, w, "mlp")
    if kind != "moe":
        raise ConfigError(f"config.json: {w}.kind '{kind}' is not a feed-forward of this design (dense and moe are)")
    router, expert = _need(mlp, "router", w), _need(mlp, "expert", w)
    experts, top = _int(router, "experts", w + ".router"), _int(router, "top", w + ".router")
    groups = router.get("groups")
    count, keep = (_int(groups, "count", w + ".router.groups"), _int(groups, "keep", w + ".router.groups")) \
        if groups is not None else (1, 1)
    if experts % count or keep > count:
        raise ConfigError(f"config.json: {w}.router: {experts} experts in {count} groups, {keep} kept")
    if top > keep * (experts // count):
        raise ConfigError(f"config.json: {w}.router: top={top} of the {keep * (experts // count)} experts of {keep} groups")
    shared = mlp.get("shared")
    return RoutedMoeSpec(experts=experts, top=top, hidden=_int(expert, "ff", w + ".expert"),
                         scale=_number(router, "scale", w + ".router") if "scale" in router else 1.0, groups=count, keep=keep,
                         correction=False, activation="swish_clamped", limit=_number(expert, "limit", w + ".expert"),
                         score="softmax", group_score="max", normalize=False,
                         shared=_dense(shared, w + ".shared", "mlp.shared") if shared is not None else None,
                         shared_gate=shared is not None, names=RoutedMoeNames())


def parse_pivipel(c: Mapping[str, Any], model_type: str, architecture: str) -> ModelConfig:
    vocab = _int(c, "vocab", "config")
    width = _int(c, "width", "config")
    eps = _number(_need(c, "norm", "config"), "eps", "norm")
    longest = _int(c, "max_positions", "config")
    hyper = c.get("streams") is not None
    streams = _int(c, "streams", "config") if hyper else 1
    raw_layers = _need(c, "layers", "config")
    if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
        raise ConfigError("config.json: layers must be a non-empty list")
    norm = DynTanhSpec()
    positions: List[Any] = [LearnedPositionSpec(name="pos", rows=longest)]
    layers: List[LayerSpec] = []
    # config layer -> index among the layers that have tensors of their own
    index_of = {i: n for n, i in enumerate(i for i, l in enumerate(raw_layers)
                                           if isinstance(l, Mapping) and l.get("weights_of") is None)}
    schedule = []
    for i, layer in enumerate(raw_layers):
        where = f"layers[{i}]"
        kind = _need(layer, "type", where)
        if kind not in MIXERS:
            raise ConfigError(f"config.json: {where}.type '{kind}' is not a mixer of this design ({', '.join(MIXERS)})")
        owner = layer.get("weights_of")
        if owner is not None:
            j = _int(layer, "weights_of", where, least=0)
            if j not in index_of:
                raise ConfigError(f"config.json: {where}.weights_of={j} names no layer with tensors of its own")
            if raw_layers[j].get("type") != kind:
                raise ConfigError(f"config.json: {where} is '{kind}' and borrows the weights of a '{raw_layers[j].get('type')}' layer")
            schedule.append(ScheduleEntry(index_of[j]))  # the same weights, a cache of this run's own
            continue
        mixer = _mixer(kind, _need(layer, "mixer", where), where + ".mixer", eps, positions)
        mlp = layer.get("mlp")
        ffn = _ffn(mlp, where + ".mlp") if mlp is not None else None
        schedule.append(ScheduleEntry(len(layers)))
        layers.append(LayerSpec(mixer=mixer, ffn=ffn, norm=norm, prefix=f"l{i}", arrangement="hyper" if hyper else "prenorm",
                                norm_in_name="norm1", norm_post_name="norm2", name_ending="", mixer_prefix="mix",
                                streams=streams))
    kinds = [l["type"] for l in raw_layers]
    description = (f"{architecture} width={width} layers={len(layers)} runs={len(schedule)} vocab={vocab} streams={streams} "
                   + " ".join(f"{k}={kinds.count(k)}" for k in MIXERS))
    return ModelConfig(
        architecture=architecture, model_type=model_type, hidden=width, vocab=vocab, final_norm=norm, layers=tuple(layers),
        positions=tuple(positions), schedule=tuple(schedule), tie_embeddings=True, max_positions=longest, embed_norm=norm,
        streams=streams, description=description,
        names=ModelNames(embed="embed", final_norm="final.norm", head="head", embed_norm="embed.norm"), raw=dict(c))


register_architecture("pivipel", "Pivipel", parse_pivipel, replace=True)
