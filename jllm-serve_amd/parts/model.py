"""The decoder model assembled from parts: embedding, the layer schedule, final norm, output head.

Skeleton as cpu/CpuBackend.java:936-989 and :821-930: rows of all requests of a step form one activation
matrix; every layer runs over all rows; the final norm and the output head run only over the rows whose
logits are wanted (:895-912). The output head is the head tensor (``lm_head.weight`` for Qwen3) when the checkpoint
has it, else the embedding matrix (model/ModelWeights.java:36-43); the names come from the config's ``names``.

The order in which layers run is the config's ``schedule``: a list of runs, each naming a layer (a layer
may be named twice) and optionally an earlier run whose cache it reads instead of writing its own.
"""
from __future__ import annotations

from typing import List

import torch

from ..cache.manager import CacheEntryPlan
from ..config.schema import ModelConfig
from ..kernels import ops
from ..weights import loader
from ..weights.loader import WeightSpec
from .base import BuildContext, part_factory


class DecoderModel:
    def __init__(self, config: ModelConfig, dtype: torch.dtype, device, max_positions: int):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the engine runs in float32 or bfloat16, not {dtype}")
        self.config = config
        self.dtype = dtype
        self.device = torch.device(device)
        self.build = BuildContext(hidden=config.hidden, dtype=dtype, device=self.device, max_positions=max_positions,
                                  exact=(dtype == torch.float32))
        self.positions = [part_factory("position", p.kind)(p, self.build) for p in config.positions]
        self.layers = [part_factory("arrangement", l.arrangement)(l, l.prefix, self.build, self.positions)
                       for l in config.layers]
        self.final_norm = part_factory("norm", config.final_norm.kind)(config.final_norm, config.hidden,
                                                                      config.names.final_norm, self.build)
        # a norm over the embedding output, and several residual streams per row (all start as the embedding output;
        # the final norm reads their sum): both need a norm part whose forward takes ``read`` / ``copies``
        self.streams = int(getattr(config, "streams", 1))
        self.embed_norm = None
        if getattr(config, "embed_norm", None) is not None:
            self.embed_norm = part_factory("norm", config.embed_norm.kind)(config.embed_norm, config.hidden,
                                                                          config.names.embed_norm, self.build)
        if self.streams > 1 and (self.embed_norm is None or not hasattr(self.final_norm, "vectors")):
            raise ValueError("several residual streams need an embedding norm that writes them and a final norm that reads their sum")
        self.streams_sum = None
        self.embed = None
        self.lm_head = None
        # vectors that join the stream before a run (config: ScheduleEntry.add_before), by tensor name
        self.stream_vector_rows = {}
        for e in config.schedule:
            if e.add_before is not None:
                self.stream_vector_rows[e.add_before.name] = e.add_before.rows
        self.stream_vectors = {}
        # matrices that mix the stream with the embedding output before a run (ScheduleEntry.mix_before), by tensor name
        self.stream_mix_names = sorted({e.mix_before.name for e in config.schedule if e.mix_before is not None})
        self.stream_mixes = {}
        self.watch = None  # a function (run, x) called with the stream after every run (tests, debugging)
        # a part that walks the step's requests on the host sets ``capturable = False``; then decode steps are
        # never recorded as graphs
        self.capturable = all(getattr(l, "capturable", True) for l in self.layers)

    # -------------------------------------------------------------------------------------------- weights

    def weight_specs(self) -> List[WeightSpec]:
        c = self.config
        specs = [WeightSpec(c.names.embed, (c.vocab, c.hidden))]
        for p in self.positions:  # a position encoding may have tensors of its own (a learned table)
            specs += p.weight_specs() if hasattr(p, "weight_specs") else []
        specs += [WeightSpec(name, (rows, c.hidden), init="bias") for name, rows in self.stream_vector_rows.items()]
        specs += [WeightSpec(name, (c.hidden, 2 * c.hidden)) for name in self.stream_mix_names]
        if self.embed_norm is not None:
            specs += self.embed_norm.weight_specs()
        for l in self.layers:
            specs += l.weight_specs()
        specs += self.final_norm.weight_specs()
        specs.append(WeightSpec(c.names.head, (c.vocab, c.hidden), optional=c.tie_embeddings))
        return specs

    def load(self, source) -> None:
        loader.check(self.weight_specs(), source, where=self.config.description)

        def get(name):
            return loader.fetch(source, name, self.dtype, self.device)

        names = self.config.names
        self.embed = get(names.embed)
        for p in self.positions:
            if hasattr(p, "load"):
                p.load(get)
        self.stream_vectors = {name: get(name) for name in self.stream_vector_rows}
        self.stream_mixes = {name: get(name) for name in self.stream_mix_names}
        if self.embed_norm is not None:
            self.embed_norm.load(get)
        if self.streams > 1:
            self.streams_sum = torch.ones(self.streams, dtype=torch.float32, device=self.device)
        for l in self.layers:
            l.load(get)
        self.final_norm.load(get)
        if self.config.logit_scale != 1.0:  # head (s * n) = s * (head n): the scale rides on the final norm's output
            if not hasattr(self.final_norm, "scale_output"):
                raise ValueError(f"a logit scale needs a final norm that can scale its output, '{self.config.final_norm.kind}' cannot")
            self.final_norm.scale_output(self.config.logit_scale)
        self.lm_head = get(names.head) if names.head in set(source.names()) else self.embed

    # -------------------------------------------------------------------------------------------- cache plan

    def cache_plans(self) -> List[CacheEntryPlan]:
        plans = []
        for e in self.config.schedule:
            layer = self.layers[e.layer]
            plans.append(CacheEntryPlan(kv=layer.cache_spec() if e.cache_from is None else None,
                                        cache_from=e.cache_from, state=layer.state_spec()))
        return plans

    def step_planners(self) -> list:
        """What the layers want to know about every batch (engine/step.py runs each distinct planner once per step)."""
        return [pl for l in self.layers for pl in (l.step_planners() if hasattr(l, "step_planners") else [])]

    def _stream_vector(self, v):
        return self.stream_vectors[v.name][v.row]

    # -------------------------------------------------------------------------------------------- forward

    def forward(self, step, slots) -> torch.Tensor:
        """Runs the step's rows through the schedule; returns fp32 logits [len(step.selected), vocab]."""
        x = ops.embed(self.embed, step.token_ids, self.config.embed_scale)
        for p in self.positions:  # an encoding that is added to the embedded rows rather than applied in the mixers
            if hasattr(p, "embed_add"):
                p.embed_add(x, step)
        if self.embed_norm is not None:  # the stream stays fp32; with several streams every one starts as this row
            x = self.embed_norm.forward(x, out_dtype=torch.float32, copies=self.streams) if hasattr(self.embed_norm, "vectors") \
                else self.embed_norm.forward(x).float()
        schedule = self.config.schedule
        x0 = x.clone() if self.stream_mix_names else None  # the embedding output, for the runs that mix it back in
        carry = None  # the next block's input norm, when the block before prepared it (parts/block.py)
        added = False  # this run's vector already joined the stream (the block before added it on its way out)
        for run, e in enumerate(schedule):
            layer = self.layers[e.layer]
            if e.mix_before is not None:
                # x <- W [x; x0] (+ the run's vector, as the product's bias): a new stream tensor
                vec = self._stream_vector(e.add_before) if e.add_before is not None and not added else None
                x = ops.gemm(ops.concat_rows(x, x0, self.build.dtype), self.stream_mixes[e.mix_before.name], bias=vec,
                             out=torch.empty_like(x), exact=self.build.exact)
                added = True
                carry = None
            if e.add_before is not None and not added:
                ops.layernorm_seam(x, 0.0, add_vec=self._stream_vector(e.add_before))
                carry = None
            added = False
            if not getattr(layer, "chains_norms", False):
                layer.forward(x, step, slots[run])
                carry = None
            else:
                nxt_e = schedule[run + 1] if run + 1 < len(schedule) else None
                nxt = self.layers[nxt_e.layer] if nxt_e is not None else None
                next_norm = getattr(nxt, "norm_in", None) if getattr(nxt, "chains_norms", False) else None
                if nxt_e is not None and nxt_e.add_before is not None and nxt_e.mix_before is None and self.watch is None \
                        and getattr(layer, "takes_stream_vector", False):
                    carry = layer.forward(x, step, slots[run], normed_in=carry, next_norm=next_norm,
                                          add_after=self._stream_vector(nxt_e.add_before))
                    added = True
                else:
                    if nxt_e is not None and (nxt_e.add_before is not None or nxt_e.mix_before is not None):
                        next_norm = None  # the stream changes before the next block reads it
                    carry = layer.forward(x, step, slots[run], normed_in=carry, next_norm=next_norm)
            if self.watch is not None:  # (with several streams: their sum)
                self.watch(run, x if self.streams == 1 else x.view(x.shape[0], self.streams, -1).sum(dim=1))
        if step.n_selected == 0:
            return torch.empty((0, self.config.vocab), dtype=torch.float32, device=self.device)
        xs = self.final_norm.forward(x, rows=step.selected) if self.streams == 1 else \
            self.final_norm.forward(x, rows=step.selected, read=self.streams_sum)
        return ops.gemm(xs, self.lm_head, out_dtype=torch.float32, exact=self.build.exact)
