"""A mixture of experts routed by a table: x += (1 / top) * sum over the token's experts of expert(xb) (+ shared(xb)).

Every token id has ``top`` experts in an integer table [vocab, top]; there is no router. An expert is a gated
feed-forward with the clamped gate (``ops.GATE_FUNCTIONS["swish_clamped"]``, the spec's ``limit``); a shared expert, when
the spec has one, is a dense gated feed-forward that runs for every row.

The routing happens on the device from the step's token ids (``ops.moe_route``), the experts' products are grouped
launches over tiles of rows of one expert (``ops.moe_gemm``): gate/up gathers the rows by token and writes hidden rows
in expert order; down writes per assignment (summed into the residual by ``ops.moe_combine``) or, with top = 1, adds
into the residual itself. Steps with many rows per expert use tiles of 128 rows through the tiled matrix-core product. Nothing waits for the GPU, so a decode step with this feed-forward can be captured.
"""
from __future__ import annotations

import torch

from ..config.schema import RoutedMoeSpec, TableMoeSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, pad_rows, part_factory, register_part


class TableMoe(Part):
    def __init__(self, spec: TableMoeSpec, prefix: str, build: BuildContext):
        if not 0 < spec.top <= spec.experts:
            raise ValueError(f"{prefix}: top {spec.top} of {spec.experts} experts")
        self.spec = spec
        self.prefix = prefix
        self.build = build
        self.gate = ops.GATE_FUNCTIONS["swish_clamped"]
        self.shared = part_factory("ffn", spec.shared.kind)(spec.shared, prefix, build) if spec.shared is not None else None
        self.takes_normed_rows = False  # the rows are gathered by the grouped product, not fed to ops.gemm
        self.w_gate = self.w_up = self.w_down = self.table = None

    def _expert(self, e: int, which: str) -> str:
        n = self.spec.names
        return f"{self.prefix}.{n.expert}{e}.{getattr(n, which)}{n.ending}"

    def _table_name(self) -> str:
        return f"{self.prefix}.{self.spec.names.table}{self.spec.names.ending}"

    def weight_specs(self):
        s, d = self.spec, self.build.hidden
        out = []
        for e in range(s.experts):
            out += [WeightSpec(self._expert(e, "gate"), (s.hidden, d)), WeightSpec(self._expert(e, "up"), (s.hidden, d)),
                    WeightSpec(self._expert(e, "down"), (d, s.hidden))]
        from ..weights.loader import EXPERT_COUNTS
        EXPERT_COUNTS[self._table_name()] = s.experts  # for the random-weights mode
        out.append(WeightSpec(self._table_name(), (s.vocab, s.top), init="expert_table"))
        if self.shared is not None:
            out += self.shared.weight_specs()
        return out

    def load(self, get):
        s = self.spec
        stack = lambda which: torch.stack([get(self._expert(e, which)) for e in range(s.experts)]).contiguous()
        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")
        table = get(self._table_name()).to(torch.int32).contiguous()
        lo, hi = int(table.min()), int(table.max())
        if lo < 0 or hi >= s.experts:
            raise ValueError(f"{self._table_name()}: entries {lo}..{hi} for {s.experts} experts")
        self.table = table
        if self.shared is not None:
            self.shared.load(get)

    def forward(self, xb, residual, step, then_norm=None):
        s, exact = self.spec, self.build.exact
        T = xb.shape[0]
        if self.shared is not None:
            self.shared.forward(xb, residual, step)
        # portions of prompts (many rows per expert) go through the tiled matrix-core product, whose K steps are 64 wide
        many_ok = not exact and self.build.dtype == torch.bfloat16 and self.w_gate.dtype == torch.bfloat16 \
            and residual.shape[1] % 64 == 0 and s.hidden % 64 == 0
        routing = ops.moe_route(step.token_ids, self.table, s.experts, many_ok=many_ok)
        A = T * s.top
        hidden = torch.empty((A, s.hidden), dtype=self.build.dtype, device=xb.device)
        ops.moe_gemm(xb, self.w_gate, routing, w2=self.w_up, out=hidden, in_map=1, out_map=0, gate=self.gate,
                     gate_limit=s.limit, exact=exact)
        if routing.many:
            y = torch.empty((A, residual.shape[1]), dtype=torch.float32, device=xb.device)
            ops.moe_gemm(hidden, self.w_down, routing, out=y, in_map=0, out_map=0, exact=exact)
            ops.moe_combine(y, residual, s.top, 1.0 / s.top, place_of=routing.place_of)
        elif s.top == 1:
            ops.moe_gemm(hidden, self.w_down, routing, out=residual, in_map=0, out_map=2, weight=1.0, exact=exact)
        else:
            y = torch.empty((A, residual.shape[1]), dtype=torch.float32, device=xb.device)
            ops.moe_gemm(hidden, self.w_down, routing, out=y, in_map=0, out_map=1, exact=exact)
            ops.moe_combine(y, residual, s.top, 1.0 / s.top)
        return None


register_part("ffn", "table_moe", TableMoe, replace=True)


class RoutedMoe(Part):
    """A mixture of experts chosen by a router: x += sum over the row's chosen experts of weight * expert(xb).

    The router's logits are an fp32 product of the rows with the router's weight (held in fp32); ``ops.moe_router`` turns
    them into the chosen experts and their weights per row (sigmoid or softmax scores, a correction on the choice,
    groups of experts of which only the best are open, weights normalised over the chosen or not). A shared expert
    (``spec.shared``) runs for every row; with ``spec.shared_gate`` its fp32 rows are multiplied by the sigmoid of one
    more logit per row, whose weight rides as a further row of the router's product. From there on the step is the
    table-routed one with the step's own table: ``ops.moe_route`` groups the assignments by expert, the grouped products
    run gate/up and down, ``ops.moe_combine`` takes the weighted sum into the residual. Nothing waits for the GPU, so a
    decode step with this feed-forward can be captured."""

    def __init__(self, spec: RoutedMoeSpec, prefix: str, build: BuildContext):
        if not 0 < spec.top <= spec.experts or spec.experts % spec.groups or not 0 < spec.keep <= spec.groups \
                or spec.top > spec.keep * (spec.experts // spec.groups):
            raise ValueError(f"{prefix}: top {spec.top} of {spec.experts} experts in {spec.groups} groups, {spec.keep} kept")
        if spec.activation not in ops.GATE_FUNCTIONS:
            raise ValueError(f"{prefix}: gate function '{spec.activation}' is not built ({sorted(ops.GATE_FUNCTIONS)} are)")
        if spec.shared_gate and spec.shared is None:
            raise ValueError(f"{prefix}: a gate for a shared expert that the feed-forward does not have")
        self.spec = spec
        self.prefix = prefix
        self.build = build
        self.gate = ops.GATE_FUNCTIONS[spec.activation]
        self.limit = float(getattr(spec, "limit", 0.0))
        self.takes_normed_rows = False
        self.shared = part_factory("ffn", spec.shared.kind)(spec.shared, prefix, build) if spec.shared is not None else None
        self.w_gate = self.w_up = self.w_down = self.w_router = self.correction = None

    def _expert(self, e: int, which: str) -> str:
        n = self.spec.names
        return f"{self.prefix}.{n.expert}{e}.{getattr(n, which)}{n.ending}"

    def _own(self, which: str) -> str:
        return f"{self.prefix}.{getattr(self.spec.names, which)}{self.spec.names.ending}"

    def weight_specs(self):
        s, d = self.spec, self.build.hidden
        out = []
        for e in range(s.experts):
            out += [WeightSpec(self._expert(e, "gate"), (s.hidden, d)), WeightSpec(self._expert(e, "up"), (s.hidden, d)),
                    WeightSpec(self._expert(e, "down"), (d, s.hidden))]
        out.append(WeightSpec(self._own("router"), (s.experts, d)))
        if s.correction:
            out.append(WeightSpec(self._own("correction"), (s.experts,), init="bias"))
        if self.shared is not None:
            out += self.shared.weight_specs()
        if s.shared_gate:
            out.append(WeightSpec(self._own("shared_gate"), (1, d)))
        return out

    def load(self, get):
        s = self.spec
        stack = lambda which: torch.stack([get(self._expert(e, which)) for e in range(s.experts)]).contiguous()
        self.w_gate, self.w_up, self.w_down = stack("gate"), stack("up"), stack("down")
        # The routing is computed in fp32. A router stored in bf16 stays bf16 in a bf16 run: the product of two bf16
        # numbers is exact in fp32 and the product kernels sum in fp32, so the logits are the fp32 ones (up to the
        # order of the sums) and the product runs on the matrix cores; its rows are filled up to a group of 16.
        w = get(self._own("router"))
        if s.shared_gate:  # the shared expert's gate logit is one more row of the router's product
            w = torch.cat([w, get(self._own("shared_gate")).to(w.dtype)], dim=0).contiguous()
        if self.shared is not None:
            self.shared.load(get)
        fast = w.dtype == torch.bfloat16 and self.build.dtype == torch.bfloat16 and not self.build.exact
        self.w_router = pad_rows(w) if fast else w.float().contiguous()
        self.correction = get(self._own("correction")).float().contiguous() if s.correction else None

    def forward(self, xb, residual, step, then_norm=None):
        self._run(xb, residual, step, overwrite=False)
        return None

    def output(self, xb, step):
        """The feed-forward's output as fp32 rows of its own, for an arrangement that does not add it into the stream
        as it is."""
        out = torch.empty((xb.shape[0], self.build.hidden), dtype=torch.float32, device=xb.device)
        self._run(xb, out, step, overwrite=True)
        return out

    def _run(self, xb, residual, step, overwrite):
        s, exact = self.spec, self.build.exact
        T = xb.shape[0]
        # fp32 logits: plain FMAs for an fp32 router, the matrix cores' exact products for a bf16 one
        zz = ops.gemm(xb, self.w_router, out_dtype=torch.float32, exact=self.w_router.dtype == torch.float32)
        z = zz[:, :s.experts]
        shared_rows = self.shared.output(xb, step) if self.shared is not None else None
        shared_gate = zz[:, s.experts] if s.shared_gate else None
        chosen, weights = ops.moe_router(z, self.correction, s.groups, s.keep, s.top, s.scale, score=s.score,
                                         group_score=s.group_score, normalize=s.normalize)
        many_ok = not exact and self.build.dtype == torch.bfloat16 and self.w_gate.dtype == torch.bfloat16 \
            and residual.shape[1] % 64 == 0 and s.hidden % 64 == 0
        routing = ops.moe_route(None, chosen, s.experts, many_ok=many_ok)
        A = T * s.top
        hidden = torch.empty((A, s.hidden), dtype=self.build.dtype, device=xb.device)
        ops.moe_gemm(xb, self.w_gate, routing, w2=self.w_up, out=hidden, in_map=1, out_map=0, gate=self.gate,
                     gate_limit=self.limit, exact=exact)
        y = torch.empty((A, residual.shape[1]), dtype=torch.float32, device=xb.device)
        if routing.many:
            ops.moe_gemm(hidden, self.w_down, routing, out=y, in_map=0, out_map=0, exact=exact)
            ops.moe_combine(y, residual, s.top, 1.0, place_of=routing.place_of, weights=weights, shared=shared_rows,
                            shared_gate=shared_gate, overwrite=overwrite)
        else:
            ops.moe_gemm(hidden, self.w_down, routing, out=y, in_map=0, out_map=1, exact=exact)
            ops.moe_combine(y, residual, s.top, 1.0, weights=weights, shared=shared_rows, shared_gate=shared_gate,
                            overwrite=overwrite)


register_part("ffn", "routed_moe", RoutedMoe, replace=True)
