"""A gated delta rule with short convolutions: a recurrent mixer whose per-request state has a fixed size.

Per head the state is a matrix S [dim, vdim] in fp32 (kept column by column, [vdim, dim]); per token it decays, is corrected along the token's key towards
the token's value (the delta rule) and is read with the token's query. Beside it the state holds the last conv - 1
inputs of the convolutions in front of q, k and v. Both live in the cache manager's state slots (one row per live
request), so nothing grows with the context and nothing is paged.

A step is
  1. one product with the stacked weight [W_q | W_k | W_v | W_g | W_a | W_b],
  2. the convolutions with silu over the first columns, reading and advancing their state (``ops.short_conv``),
  3. the recurrence over each request's rows in order, with unit norms, decay and write strength inside
     (``ops.gated_delta``; its value columns are spread over workgroups, so its read-out comes back raw),
  4. the heads' norm, gain and silu gate (``ops.heads_finish``, the kernel that ends attention heads too),
  5. the output product.
With one decay per head and key channel (``spec.decay == "channel"``) the decay's input is a product of its own behind
the stacked one (through a narrow middle, W_up (W_down h), whose first half rides in the stack), in fp32; the gate's
input may pass such a middle too. The same launches serve portions of prompts and single rows: the recurrence visits a request's rows one after the
other either way, so its result does not depend on how a prompt was cut.
"""
from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..config.schema import GatedDeltaSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, pad_rows, register_part


class GatedDelta(Part):
    def __init__(self, spec: GatedDeltaSpec, prefix: str, build: BuildContext, positions):
        self.spec = spec
        self.prefix = prefix
        self.build = build
        try:
            ops.check_gated_delta_shape(spec.heads, spec.kv_heads, spec.dim, spec.vdim, spec.conv)
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        if spec.decay not in ("head", "channel"):
            raise ValueError(f"{prefix}: a decay per '{spec.decay}' is not built ('head' and 'channel' are)")
        if spec.decay == "channel" and spec.decay_rank == 0:
            raise ValueError(f"{prefix}: a decay per key channel takes its input through a narrow middle (decay_rank)")
        if spec.gate_fn not in ops.HEAD_GATES:
            raise ValueError(f"{prefix}: gate function '{spec.gate_fn}' ({sorted(ops.HEAD_GATES)} are built)")
        self.qk_dim = spec.kv_heads * spec.dim
        self.v_dim = spec.heads * spec.vdim
        self.channels = 2 * self.qk_dim + self.v_dim  # what passes the convolutions: q | k | v
        self.decay_dim = spec.heads * spec.dim if spec.decay == "channel" else spec.heads
        self.gate_at = self.channels
        # the stacked product's columns behind q | k | v: gate (or its middle) | decay (or its middle) | b; a middle
        # whose size the checkpoint chooses (-1) is known once the weights are loaded
        self.gate_cols = self.a_at = self.a_cols = self.b_at = None
        if spec.gate_rank >= 0 and spec.decay_rank >= 0:
            self._offsets(spec.gate_rank, spec.decay_rank)
        self.w_in = self.taps = self.a_log = self.dt_bias = self.gain = self.w_o = self.w_gate_up = self.w_decay_up = None

    def _offsets(self, gate_rank: int, decay_rank: int) -> None:
        self.gate_cols = gate_rank if gate_rank else self.v_dim
        self.a_at = self.gate_at + self.gate_cols
        self.a_cols = decay_rank if decay_rank else self.decay_dim
        self.b_at = self.a_at + self.a_cols

    def _name(self, which: str, suffix: str = "") -> str:
        return f"{self.prefix}.{getattr(self.spec.names, which)}{suffix}"

    def weight_specs(self):
        s, d, nm = self.spec, self.build.hidden, self.spec.names
        sizes = (("q", self.qk_dim), ("k", self.qk_dim), ("v", self.v_dim))
        out = [WeightSpec(self._name(n), (w, d)) for n, w in sizes]
        out += [WeightSpec(self._name(n, nm.conv_suffix), (w, s.conv)) for n, w in sizes]
        out.append(WeightSpec(self._name("beta"), (s.heads, d)))
        if s.decay_rank:
            out += [WeightSpec(self._name("decay_down"), (s.decay_rank, d)),
                    WeightSpec(self._name("decay_up"), (self.decay_dim, s.decay_rank))]
        else:
            out.append(WeightSpec(self._name("decay"), (self.decay_dim, d)))
        if s.gate_rank:
            out += [WeightSpec(self._name("gate_down"), (s.gate_rank, d)), WeightSpec(self._name("gate_up"), (self.v_dim, s.gate_rank))]
        else:
            out.append(WeightSpec(self._name("gate"), (self.v_dim, d)))
        out += [WeightSpec(self._name("a_log"), (s.heads,), init="bias"), WeightSpec(self._name("dt_bias"), (self.decay_dim,), init="bias"),
                WeightSpec(self._name("norm"), (s.vdim,), init="gain"), WeightSpec(self._name("o"), (d, self.v_dim))]
        return out

    def load(self, get):
        s, nm = self.spec, self.spec.names
        gate_in = get(self._name("gate_down" if s.gate_rank else "gate"))
        decay_in = get(self._name("decay_down" if s.decay_rank else "decay"))
        self.w_gate_up = get(self._name("gate_up")) if s.gate_rank else None
        self.w_decay_up = get(self._name("decay_up")) if s.decay_rank else None
        for up, down, what in ((self.w_gate_up, gate_in, "gate"), (self.w_decay_up, decay_in, "decay")):
            if up is not None and up.shape[1] != down.shape[0]:
                raise ValueError(f"{self.prefix}: the two halves of the {what}'s input disagree about their middle: "
                                 f"{down.shape[0]} and {up.shape[1]}")
        self._offsets(gate_in.shape[0] if s.gate_rank else 0, decay_in.shape[0] if s.decay_rank else 0)
        stack = [get(self._name(n)) for n in ("q", "k", "v")] + [gate_in, decay_in, get(self._name("beta"))]
        dt = stack[0].dtype if all(t.dtype == stack[0].dtype for t in stack) else torch.float32
        self.w_in = pad_rows(torch.cat([t.to(dt) for t in stack], dim=0).contiguous())
        del stack
        taps = [get(self._name(n, nm.conv_suffix)) for n in "qkv"]
        dt = taps[0].dtype if all(t.dtype == taps[0].dtype for t in taps) else torch.float32
        self.taps = torch.cat([t.to(dt) for t in taps], dim=0).contiguous()
        small = [get(self._name(n)) for n in ("a_log", "dt_bias")]
        if small[0].dtype != small[1].dtype:
            small = [t.float() for t in small]
        self.a_log, self.dt_bias = small
        self.gain = get(self._name("norm"))
        self.w_o = get(self._name("o"))

    def state_spec(self):
        s = self.spec
        return (StateSpec((s.heads, s.vdim, s.dim), torch.float32),
                StateSpec((max(s.conv - 1, 1), self.channels), torch.float32))

    def input_projection(self):
        return self.w_in, None

    def output_weight(self):
        return self.w_o

    @property
    def heads_width(self):
        return self.v_dim

    def heads_rows(self, xb, step, slot):
        """The input of the output product, [rows, heads x vdim] in the run's type."""
        y = ops.gemm(xb, self.w_in, out_dtype=self.build.dtype, exact=self.build.exact)
        return self.heads_rows_from(y, step, slot)

    def heads_rows_from(self, y, step, slot, out=None, out_mul=1.0):
        """The same from the input product's result ``y`` (a view with any row stride); ``out``: where to write."""
        s = self.spec
        matrix, tail = slot.state
        qkv = ops.short_conv(y, self.taps, tail, step.row_req, step.state_slots, step.n_requests)
        exact = self.build.exact
        decay_rows = None
        if s.decay == "channel":  # what enters the recurrence besides the projections is fp32: the decay's input too
            decay_rows = ops.gemm(y[:, self.a_at:self.a_at + self.a_cols], self.w_decay_up, out_dtype=torch.float32, exact=exact)
            a_at = 0
        elif s.decay_rank:
            raise NotImplementedError("a decay per head through a narrow middle")
        else:
            a_at = self.a_at
        o = ops.gated_delta(qkv, y, a_at, self.b_at, self.a_log, self.dt_bias, matrix, step.row_req, step.state_slots,
                            step.n_requests, s.heads, s.kv_heads, s.dim, s.vdim, decay_rows=decay_rows)
        gate = y[:, self.gate_at:self.gate_at + self.gate_cols]
        if s.gate_rank:
            gate = ops.gemm(gate, self.w_gate_up, out_dtype=self.build.dtype, exact=exact)
        return ops.heads_finish(o, s.heads, 1, s.vdim, self.build.dtype, normed=True, eps=s.eps, gain=self.gain,
                                gate=gate, gate_fn=s.gate_fn, out=out, out_mul=out_mul)

    def output(self, xb, step, slot):
        return ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out_dtype=torch.float32, exact=self.build.exact)

    def forward(self, xb, residual, step, slot):
        ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)


register_part("mixer", "gated_delta", GatedDelta, replace=True)
