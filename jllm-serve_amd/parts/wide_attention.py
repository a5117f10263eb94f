"""Causal grouped-query attention over the paged cache with key and value sizes of their own, and what several designs
put around the softmax (config/schema.py: WideAttentionSpec): two score maps per head whose outputs are subtracted
(differential attention), a norm with gains over the whole q and k projections or over every head alone, rotation of
neighbouring pairs or of the two halves of a head's rotated part, capped scores, a query scale that grows with the
position, a sliding window that may keep the first keys, a learned sink in the softmax's denominator, an output gate per
channel or per head.

A step is
  1. one product with the stacked weight [W_q | W_k | W_v | W_g] and the stacked bias (zeros for the gate's rows),
  2. one launch that norms, rotates and scales q in place and stores k and v at the rows' places in the pages
     (``ops.qkv_prepare``),
  3. the attention over the pages, every map of every head alone (``ops.attention_dv``), fp32 out,
  4. one launch that subtracts the maps, norms each head and multiplies by sigmoid(gate) (``ops.heads_finish``),
  5. the output product.
The cache holds, per position, the keys of every map [kv_heads x maps, dim] and the values [kv_heads, vdim].
"""
from __future__ import annotations


import torch

from ..cache.manager import CacheRow, PageSpec
from ..config.schema import WideAttentionSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, pad_rows, register_part


class WideStepPlanner:
    """What the matrix-core attention kernel wants to know about a batch, once per step for all such layers: every
    request's rows cut into tiles of at most ``ops.WIDE_TILE_ROWS`` rows as (request, first row, rows, first position),
    the tiles with the most keys first. A step of fixed size (every request one row) gets one tile per row in row order
    with position -1: the kernel then reads the row's position on the device."""

    key = ("wide_attention", ops.WIDE_TILE_ROWS)

    def plan(self, batch):
        from ..engine.step import StepPlan
        R = ops.WIDE_TILE_ROWS
        if batch.padded:
            runs = [(r, r, 1, -1) for r in range(batch.rows)]
        else:
            runs = [(s.index, s.row0 + r, min(R, s.n - r), s.pos0 + r) for s in batch.segments for r in range(0, s.n, R)]
            runs.sort(key=lambda t: -(t[3] + t[2]))
        single = batch.padded or all(s.n == 1 for s in batch.segments)
        return StepPlan({"tiles": [v for t in runs for v in t]}, {"n_tiles": len(runs), "single_rows": single})


class WideAttention(Part):
    def __init__(self, spec: WideAttentionSpec, prefix: str, build: BuildContext, positions):
        if spec.maps not in (1, 2):
            raise ValueError(f"{prefix}: {spec.maps} score maps per head (one or two are built)")
        if spec.qk_norm not in (None, "whole", "head"):
            raise ValueError(f"{prefix}: q/k norm '{spec.qk_norm}' is not built for this mixer ('whole' and 'head' are)")
        if spec.sink and spec.maps != 1:
            raise ValueError(f"{prefix}: a sink with {spec.maps} score maps per head")
        if spec.keep_first and not spec.window:
            raise ValueError(f"{prefix}: first keys are kept beside a window, and this mixer has none")
        self.spec = spec
        self.prefix = prefix
        self.build = build
        self.position = positions[spec.position] if spec.position is not None else None
        rot = self.position.rotary() if self.position is not None else None
        self.pairing = getattr(self.position, "pairing", "half") if rot is not None else "interleaved"
        self.rot = rot
        try:
            ops.check_attention_dv_shape(spec.heads, spec.kv_heads, spec.maps, spec.dim, spec.vdim, rot[2] if rot else 0)
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.q_dim = spec.heads * spec.maps * spec.dim
        self.k_dim = spec.kv_heads * spec.maps * spec.dim
        self.v_dim = spec.kv_heads * spec.vdim
        self.o_dim = spec.heads * spec.vdim
        self.gate_dim = spec.heads if spec.gate_per_head else self.o_dim  # rows of W_g: one per head, or one per channel
        self.sinks = None
        self.w_in = self.b_in = self.w_o = self.g_q = self.g_k = None
        self.lam = 0.0

    def _name(self, which: str, suffix: str = "") -> str:
        return f"{self.prefix}.{getattr(self.spec.names, which)}{suffix}"

    def weight_specs(self):
        s, d, nm = self.spec, self.build.hidden, self.spec.names
        out = [WeightSpec(self._name("q"), (self.q_dim, d)), WeightSpec(self._name("k"), (self.k_dim, d)),
               WeightSpec(self._name("v"), (self.v_dim, d))]
        if s.bias:
            out += [WeightSpec(self._name(n, nm.bias_suffix), (w,), init="bias")
                    for n, w in (("q", self.q_dim), ("k", self.k_dim), ("v", self.v_dim))]
        if s.qk_norm == "whole":
            out += [WeightSpec(self._name("q", nm.norm_suffix), (self.q_dim,), init="gain"),
                    WeightSpec(self._name("k", nm.norm_suffix), (self.k_dim,), init="gain")]
        if s.qk_norm == "head":  # one gain vector for all q heads, one for all k heads
            out += [WeightSpec(self._name("q", nm.norm_suffix), (s.dim,), init="gain"),
                    WeightSpec(self._name("k", nm.norm_suffix), (s.dim,), init="gain")]
        if s.sink:
            out.append(WeightSpec(self._name("sink"), (s.heads,), init="bias"))
        if s.maps == 2:
            out += [WeightSpec(f"{self.prefix}.{n}", (s.dim,), init="bias") for n in nm.lambda_q + nm.lambda_k]
        if s.out_gate:
            out.append(WeightSpec(self._name("gate"), (self.gate_dim, d)))
        out.append(WeightSpec(self._name("o"), (d, self.o_dim)))
        return out

    def load(self, get):
        s, nm = self.spec, self.spec.names
        stack = [get(self._name(n)) for n in "qkv"]
        if s.out_gate:
            stack.append(get(self._name("gate")))
        dt = stack[0].dtype if all(t.dtype == stack[0].dtype for t in stack) else torch.float32
        self.w_in = pad_rows(torch.cat([t.to(dt) for t in stack], dim=0).contiguous())  # [q | k | v | g] rows
        del stack
        if s.bias:
            b = [get(self._name(n, nm.bias_suffix)).to(torch.float32) for n in "qkv"]
            if s.out_gate:
                b.append(torch.zeros(self.gate_dim, dtype=torch.float32, device=b[0].device))
            self.b_in = pad_rows(torch.cat(b).contiguous())
        if s.sink:
            self.sinks = get(self._name("sink")).float().contiguous()
        if s.qk_norm in ("whole", "head"):
            self.g_q, self.g_k = get(self._name("q", nm.norm_suffix)), get(self._name("k", nm.norm_suffix))
            if self.g_q.dtype != self.g_k.dtype:
                self.g_q, self.g_k = self.g_q.float(), self.g_k.float()
        if s.maps == 2:
            # one number for the layer, from four vectors of the checkpoint: computed once, in fp32
            v = [get(f"{self.prefix}.{n}").to(torch.float32) for n in nm.lambda_q + nm.lambda_k]
            self.lam = float(torch.exp((v[0] * v[2]).sum()) - torch.exp((v[1] * v[3]).sum())) + float(s.diff)
        self.w_o = get(self._name("o"))

    def cache_spec(self):
        s = self.spec
        return PageSpec((CacheRow("k", (s.kv_heads * s.maps, s.dim), 1), CacheRow("v", (s.kv_heads, s.vdim), 1)), s.window,
                        s.keep_first if s.window else 0)

    def step_planners(self):
        return [WideStepPlanner()]

    @staticmethod
    def _batch_facts(step):
        meta = {"max_context": step.max_context, "requests": step.n_requests, "rows": step.n_tokens}
        plan = step.plans.get(WideStepPlanner.key)
        if plan is not None:
            tiles = plan.arrays.get("tiles")
            meta["n_tiles"] = plan.facts["n_tiles"]
            meta["single_rows"] = plan.facts["single_rows"]
            meta["tiles_dev"] = tiles if tiles is not None and tiles.numel() else None
        return meta

    # a mixer that runs beside others on the same input may have its input product and its output product stacked
    # with theirs (parts/parallel.py): it says what they are, and works from its columns of the stacked result
    def input_projection(self):
        return self.w_in, self.b_in

    def output_weight(self):
        return self.w_o

    @property
    def heads_width(self):
        return self.o_dim

    def heads_rows(self, xb, step, slot):
        """The input of the output product, [rows, heads x vdim] in the run's type."""
        y = ops.gemm(xb, self.w_in, bias=self.b_in, out_dtype=self.build.dtype, exact=self.build.exact)
        return self.heads_rows_from(y, step, slot)

    def heads_rows_from(self, y, step, slot, out=None, out_mul=1.0):
        """The same from the input product's result ``y`` (a view with any row stride); ``out``: where to write."""
        s, exact = self.spec, self.build.exact
        g = step.groups[slot.group]
        k_cache, v_cache = slot.rows["k"], slot.rows["v"]
        cos, sin, rdims = self.rot if self.rot is not None else (None, None, 0)
        ops.qkv_prepare(y, step.positions, g.slots if slot.writes else None, s.heads, s.kv_heads, s.maps, s.dim, s.vdim,
                        k_cache, v_cache, gq=self.g_q, gk=self.g_k, eps=s.eps, cos=cos, sin=sin, rot_dims=rdims,
                        temp_coef=s.q_temp_coef, temp_every=s.q_temp_every, norm_per_head=s.qk_norm == "head",
                        pairing=self.pairing)
        meta = self._batch_facts(step)
        att = ops.attention_dv(y[:, :self.q_dim], k_cache, v_cache, g.block_table, step.row_req, step.positions, s.heads,
                               s.kv_heads, s.maps, s.dim, s.vdim, s.scale, softcap=s.softcap, window=s.window,
                               out_dtype=torch.float32, meta=meta, exact=exact, defer_merge=True, keep_first=s.keep_first,
                               sinks=self.sinks)
        gate_at = self.q_dim + self.k_dim + self.v_dim
        gate = y[:, gate_at:gate_at + self.gate_dim] if s.out_gate else None
        return ops.heads_finish(att, s.heads, s.maps, s.vdim, self.build.dtype, lam=self.lam, normed=s.maps == 2,
                                eps=s.eps, norm_mul=1.0 - s.diff, gate=gate, out=out, out_mul=out_mul,
                                gate_per_head=bool(s.out_gate and s.gate_per_head))

    def output(self, xb, step, slot):
        """The mixer's output as fp32 rows of its own (for arrangements that norm or weigh it before the add)."""
        return ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out_dtype=torch.float32, exact=self.build.exact)

    def forward(self, xb, residual, step, slot):
        ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)


register_part("mixer", "wide_attention", WideAttention, replace=True)
