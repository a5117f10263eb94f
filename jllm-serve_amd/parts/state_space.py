"""A selective state-space mixer (the Mamba-2 form): a recurrent mixer whose per-request state has a fixed size.

Per head the state is a matrix S [state, vdim] in fp32 (kept column by column, [vdim, state]); per token it decays by one number, takes in the outer product of
the token's B and x scaled by the step size, and is read with the token's C. Beside it the state holds the last conv - 1
inputs of the convolution in front of x, B and C. Both live in the cache manager's state slots (one row per live
request), so nothing grows with the context and nothing is paged.

A step is
  1. one product with the input weight, whose rows are laid out [z | x | B | C | dt],
  2. the convolution with bias and silu over the x | B | C columns, reading and advancing its state (``ops.short_conv``),
  3. the recurrence over each request's rows in order, with the step sizes' softplus and the decay inside
     (``ops.ssm_scan``; its value columns are spread over workgroups, so its read-out comes back raw, in fp32),
  4. the gate silu(z), then the RMS norm in equal parts of the row, then the weight (``ops.gated_group_norm``),
  5. the output product.
The same launches serve portions of prompts and single rows: the recurrence visits a request's rows one after the
other either way, so its result does not depend on how a prompt was cut.
"""
from __future__ import annotations

import torch

from ..cache.manager import StateSpec
from ..config.schema import StateSpaceSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, pad_rows, register_part


class StateSpace(Part):
    def __init__(self, spec: StateSpaceSpec, prefix: str, build: BuildContext, positions):
        self.spec = spec
        self.prefix = prefix
        self.build = build
        try:
            ops.check_ssm_shape(spec.heads, spec.groups, spec.state, spec.vdim, spec.conv)
        except ops.KernelError as e:
            raise ValueError(f"{prefix}: {e}") from None
        self.inner = spec.heads * spec.vdim
        if self.inner % spec.norm_groups:
            raise ValueError(f"{prefix}: {spec.norm_groups} norm groups do not divide heads x vdim = {self.inner}")
        self.channels = self.inner + 2 * spec.groups * spec.state  # what passes the convolution: x | B | C
        self.x_at = self.inner                   # z comes first
        self.dt_at = self.inner + self.channels
        self.width = self.dt_at + spec.heads
        self.w_in = self.taps = self.conv_bias = self.a_log = self.dt_bias = self.skip = self.gain = self.w_o = None

    def _name(self, which: str) -> str:
        return f"{self.prefix}.{getattr(self.spec.names, which)}"

    def weight_specs(self):
        s, d = self.spec, self.build.hidden
        return [WeightSpec(self._name("in_proj"), (self.width, d)), WeightSpec(self._name("conv"), (self.channels, s.conv)),
                WeightSpec(self._name("conv_bias"), (self.channels,), init="bias"),
                WeightSpec(self._name("dt_bias"), (s.heads,), init="bias"), WeightSpec(self._name("a_log"), (s.heads,), init="bias"),
                WeightSpec(self._name("skip"), (s.heads,), init="gain"), WeightSpec(self._name("norm"), (self.inner,), init="gain"),
                WeightSpec(self._name("o"), (d, self.inner))]

    def load(self, get):
        self.w_in = pad_rows(get(self._name("in_proj")))
        taps, bias = get(self._name("conv")), get(self._name("conv_bias"))
        if taps.dtype != bias.dtype:
            taps, bias = taps.float(), bias.float()
        self.taps, self.conv_bias = taps, bias
        small = [get(self._name(n)) for n in ("a_log", "dt_bias", "skip")]
        if any(t.dtype != small[0].dtype for t in small):
            small = [t.float() for t in small]
        self.a_log, self.dt_bias, self.skip = small
        self.gain = get(self._name("norm"))
        self.w_o = get(self._name("o"))

    def state_spec(self):
        s = self.spec
        return (StateSpec((s.heads, s.vdim, s.state), torch.float32),
                StateSpec((max(s.conv - 1, 1), self.channels), torch.float32))

    def heads_rows(self, xb, step, slot):
        """The input of the output product, [rows, heads x vdim] in the run's type."""
        s = self.spec
        y = ops.gemm(xb, self.w_in, out_dtype=self.build.dtype, exact=self.build.exact)
        matrix, tail = slot.state
        xbc = ops.short_conv(y[:, self.x_at:self.x_at + self.channels], self.taps, tail, step.row_req, step.state_slots,
                             step.n_requests, bias=self.conv_bias)
        o = ops.ssm_scan(xbc, y, self.dt_at, self.a_log, self.dt_bias, self.skip, matrix, step.row_req, step.state_slots,
                         step.n_requests, s.heads, s.groups, s.state, s.vdim)
        return ops.gated_group_norm(o, y[:, :self.inner], self.gain, s.eps, s.norm_groups, self.build.dtype)

    def output(self, xb, step, slot):
        return ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out_dtype=torch.float32, exact=self.build.exact)

    def forward(self, xb, residual, step, slot):
        ops.gemm(self.heads_rows(xb, step, slot), self.w_o, out=residual, epilogue=ops.EPI_ADD, exact=self.build.exact)


register_part("mixer", "state_space", StateSpace, replace=True)
