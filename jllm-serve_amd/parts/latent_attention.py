"""Latent attention over the paged cache: queries, keys and values all pass through low-rank latents.

Per position a layer caches one row: the RMS-normed latent c (kv_rank numbers) and one rotated key part (rot_dim
numbers) shared by all heads. Head h's unrotated key is W_uk[h] c, its value W_uv[h] c; a query head has ``dim``
unrotated and ``rot_dim`` rotated entries and comes from a normed latent of q_rank. The score of key j for the row at
p is (q_plain . k_plain + q_rot . k_rot) * scale over the keys p + 1 - window .. p, the softmax's denominator also holds
exp(sink_h), the concatenated heads are multiplied by sigmoid(W_g h) and go through W_o.

Here the per-head key and value products are moved to the query's side, so that nothing but the cached rows is ever
read per key: with qa[h] = [W_uk[h]^T q_plain[h] | q_rot[h]] a score is qa[h] . row, and a head's output is
W_uv[h] (sum_j p_j c_j). A step is

  1. one product with the stacked weight [W_dq | W_dkv | W_g] (a run that reads another run's cache has no W_dkv),
  2. one launch that norms the query latent and norms / rotates / stores the row of the cache (``ops.latent_prepare``),
  3. the product with W_uq,
  4. one launch for all heads' W_uk[h]^T products and the rotation of the queries' rotated parts (``ops.latent_heads``),
  5. the attention over the cached rows (``ops.latent_attention``),
  6. one launch for all heads' W_uv[h] products, multiplied by the gate (``ops.latent_heads`` with ``gate``),
  7. the output product, added into the residual.
"""
from __future__ import annotations

import torch

from ..cache.manager import CacheRow, PageSpec
from ..config.schema import LatentAttentionSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, register_part

TILE_ROWS = 16  # rows of one request that a workgroup of the matrix-core attention kernel takes


class LatentStepPlanner:
    """What the latent-attention kernels want to know about a batch, once per step for all such layers: the requests'
    rows cut into runs of at most TILE_ROWS rows as (request, first row, rows, first position), the runs with the most
    keys first. A captured step (fixed size, every request one row) gets one run per row in row order."""

    key = ("latent_attention", TILE_ROWS)

    def plan(self, batch):
        from ..engine.step import StepPlan
        if batch.padded:
            runs = [(r, r, 1, 0) for r in range(batch.rows)]  # positions are read on the device
        else:
            runs = [(s.index, s.row0 + r, min(TILE_ROWS, s.n - r), s.pos0 + r) for s in batch.segments
                    for r in range(0, s.n, TILE_ROWS)]
            runs.sort(key=lambda t: -(t[3] + t[2]))
        single = batch.padded or all(s.n == 1 for s in batch.segments)
        return StepPlan({"tiles": [v for t in runs for v in t]}, {"n_tiles": len(runs), "single_rows": single})


class LatentAttention(Part):
    takes_normed_rows = True    # the input goes into ops.gemm and nowhere else
    prepares_next_norm = True   # forward(then_norm=...) ends with then_norm.after_add and returns its promise

    def __init__(self, spec: LatentAttentionSpec, prefix: str, build: BuildContext, positions):
        self.spec = spec
        self.prefix = prefix
        self.build = build
        self.position = positions[spec.position] if spec.position is not None else None
        rot = self.position.rotary() if self.position is not None else None
        self.rot_dims = rot[2] if rot is not None else 0
        # The kernels rotate the pairs (i, i + rotary_dim / 2). A checkpoint whose pairs are neighbours (2i, 2i + 1)
        # runs on the same kernels with the rows of its rotated projections reordered at load (evens first, then
        # odds): a score is a dot product of a rotated query part and a rotated key part, and reordering both the same
        # way changes no dot product. The angles of pair i are the same in both layouts.
        self.reorder = None
        if getattr(self.position, "pairing", "half") == "interleaved" and self.rot_dims:
            self.reorder = list(range(0, self.rot_dims, 2)) + list(range(1, self.rot_dims, 2)) + list(range(self.rot_dims, spec.rot_dim))
        try:
            ops.check_latent_shape(spec.heads, spec.kv_rank, spec.rot_dim, self.rot_dims)
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.w_in = self.w_uq = self.w_ukt = self.w_uv = self.w_o = self.g_q = self.g_kv = self.sink = None

    def _name(self, which: str) -> str:
        return f"{self.prefix}.{getattr(self.spec.names, which)}{self.spec.names.ending}"

    @property
    def kv_width(self) -> int:
        return self.spec.kv_rank + self.spec.rot_dim

    def weight_specs(self):
        s, d = self.spec, self.build.hidden
        if s.q_rank > 0:
            out = [WeightSpec(self._name("dq"), (s.q_rank, d)), WeightSpec(self._name("dq_norm"), (s.q_rank,), init="gain"),
                   WeightSpec(self._name("uq"), (s.heads * (s.dim + s.rot_dim), s.q_rank))]
        else:  # the query comes straight from the input
            out = [WeightSpec(self._name("q"), (s.heads * (s.dim + s.rot_dim), d))]
        if s.owns_cache:
            out += [WeightSpec(self._name("dkv"), (self.kv_width, d)),
                    WeightSpec(self._name("dkv_norm"), (s.kv_rank,), init="gain")]
        out += [WeightSpec(self._name("uk"), (s.heads * s.dim, s.kv_rank)),
                WeightSpec(self._name("uv"), (s.heads * s.vdim, s.kv_rank))]
        if s.sink:
            out.append(WeightSpec(self._name("sink"), (s.heads,), init="bias"))
        if s.out_gate:
            out.append(WeightSpec(self._name("gate"), (s.heads * s.vdim, d)))
        out.append(WeightSpec(self._name("o"), (d, s.heads * s.vdim)))
        return out

    def load(self, get):
        s = self.spec

        def reordered(w, first, per, count):
            """Rows first + j * per + reorder[i] of w in place of first + j * per + i, for j < count."""
            if self.reorder is None:
                return w
            w = w.clone()
            idx = torch.tensor(self.reorder, device=w.device)
            for j in range(count):
                at = first + j * per
                w[at:at + len(self.reorder)] = w[at + idx]
            return w

        q_name = "uq" if s.q_rank > 0 else "q"
        w_q = reordered(get(self._name(q_name)), s.dim, s.dim + s.rot_dim, s.heads)
        stack = [get(self._name("dq"))] if s.q_rank > 0 else [w_q]
        if s.owns_cache:
            stack.append(reordered(get(self._name("dkv")), s.kv_rank, 0, 1))
            self.g_kv = get(self._name("dkv_norm"))
        if s.out_gate:
            stack.append(get(self._name("gate")))
        dt = stack[0].dtype if all(t.dtype == stack[0].dtype for t in stack) else torch.float32
        self.w_in = torch.cat([t.to(dt) for t in stack], dim=0).contiguous()  # [dq | dkv | g] rows
        del stack
        self.g_q = get(self._name("dq_norm")) if s.q_rank > 0 else None
        if self.g_kv is not None and self.g_q is not None and self.g_kv.dtype != self.g_q.dtype:
            self.g_q, self.g_kv = self.g_q.float(), self.g_kv.float()
        self.w_uq = w_q if s.q_rank > 0 else None
        self.q_width = s.heads * (s.dim + s.rot_dim)
        # W_uk[h] is [dim, kv_rank]; the query side needs its transpose as a weight [N = kv_rank, K = dim] per head
        self.w_ukt = get(self._name("uk")).view(s.heads, s.dim, s.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = get(self._name("uv")).view(s.heads, s.vdim, s.kv_rank).contiguous()
        self.sink = get(self._name("sink")).to(torch.float32).contiguous() if s.sink else None
        self.w_o = get(self._name("o"))

    def cache_spec(self):
        # one row per position: [latent | rotated key part]; the pages honour the widest window that reads them
        return PageSpec((CacheRow("ckr", (self.kv_width,), 0),), self.spec.keep)

    def step_planners(self):
        return [LatentStepPlanner()]

    @staticmethod
    def _batch_facts(step):
        plan = step.plans.get(LatentStepPlanner.key)
        meta = {"max_context": step.max_context, "requests": step.n_requests, "rows": step.n_tokens}
        if plan is not None:
            meta.update(plan.facts)
            tiles = plan.arrays.get("tiles")
            meta["tiles_dev"] = tiles if tiles is not None and tiles.numel() else None
        return meta

    def forward(self, xb, residual, step, slot, then_norm=None):
        s, exact = self.spec, self.build.exact
        g = step.groups[slot.group]
        cache = slot.rows["ckr"]
        rot = self.position.rotary() if self.position is not None else None
        cos, sin, rdims = rot if rot is not None else (None, None, 0)
        y = ops.gemm(xb, self.w_in, out_dtype=self.build.dtype, exact=exact)
        kv_off = s.q_rank if s.q_rank > 0 else self.q_width
        gate_off = kv_off + (self.kv_width if s.owns_cache else 0)
        cq = None
        if s.owns_cache and slot.writes:
            cq = ops.latent_prepare(y, s.q_rank, self.g_q, s.eps, kv_off=kv_off, kv_rank=s.kv_rank, rot_dim=s.rot_dim,
                                    rot_dims=rdims, gkv=self.g_kv, positions=step.positions, slots=g.slots, cos=cos,
                                    sin=sin, cache=cache)
        elif s.q_rank > 0:
            cq = ops.latent_prepare(y, s.q_rank, self.g_q, s.eps)
        q = ops.gemm(cq, self.w_uq, out_dtype=self.build.dtype, exact=exact) if s.q_rank > 0 else y[:, :self.q_width]
        qa = ops.latent_heads(q, self.w_ukt, tail=s.rot_dim, rot_dims=rdims, positions=step.positions, cos=cos, sin=sin,
                              exact=exact)
        lat = ops.latent_attention(qa, cache, g.block_table, step.row_req, step.positions, s.heads, s.kv_rank, s.window,
                                   s.scale, self.sink, meta=self._batch_facts(step), exact=exact)
        if s.out_gate:
            att = ops.latent_heads(lat, self.w_uv, gate=y[:, gate_off:gate_off + s.heads * s.vdim], exact=exact)
        else:
            att = ops.latent_heads(lat, self.w_uv, exact=exact)
        if then_norm is not None:
            return then_norm.after_add(att, self.w_o, residual, exact=exact)
        ops.gemm(att, self.w_o, out=residual, epilogue=ops.EPI_ADD, exact=exact)
        return None


register_part("mixer", "latent_attention", LatentAttention, replace=True)
