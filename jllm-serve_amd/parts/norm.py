"""RMSNorm: y = (x * rsqrt(mean(x^2) + eps)) * g over fp32 rows (cpu/VectorKernels.java:630-634), layer norm with a
weight and a bias: y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b, and Dynamic Tanh, which takes no statistics
of the row: y = tanh(alpha x) w + b."""
from __future__ import annotations

import torch

from ..config.schema import DynTanhSpec, LayerNormSpec, NormSpec
from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import BuildContext, Part, register_part


class RMSNorm(Part):
    def __init__(self, spec: NormSpec, dim: int, weight_name: str, build: BuildContext):
        self.eps = float(spec.eps)
        self.dim = dim
        self.weight_name = weight_name
        self.out_dtype = build.dtype
        self.gain = None

    def weight_specs(self):
        return [WeightSpec(self.weight_name, (self.dim,), init="gain")]

    def load(self, get):
        self.gain = get(self.weight_name)

    def forward(self, x, rows=None):
        return ops.rmsnorm(x, self.gain, self.eps, self.out_dtype, rows)

    def defer(self, x):
        """The normalised rows as a promise, for consumers that feed them to ``ops.gemm`` only."""
        return ops.NormedRows(x, self.gain, self.eps, self.out_dtype)

    def scale_output(self, factor: float) -> None:
        """From now on the norm's output is ``factor`` times what it was (the gain in fp32)."""
        if factor != 1.0:
            self.gain = (self.gain.float() * factor).contiguous()

    def after_add(self, a, w, residual, bias=None, exact=False):
        """residual += a @ w.T (+ bias), and this norm of the result as a promise: the product that makes the new
        residual rows can prepare their norm on its way out (``ops.gemm_add_then_norm``)."""
        return ops.gemm_add_then_norm(a, w, residual, self.gain, self.eps, self.out_dtype, bias=bias, exact=exact)


register_part("norm", "rmsnorm", RMSNorm, replace=True)


class LayerNorm(Part):
    """Mean and variance in fp32 over fp32 rows. Beside ``forward`` it offers the seam between two sublayers as one
    launch (``seam``): the norm of a sublayer's output added into the stream, a vector added to the stream, and the
    next sublayer's input norm, each optional."""

    def __init__(self, spec: LayerNormSpec, dim: int, weight_name: str, build: BuildContext):
        self.eps = float(spec.eps)
        self.dim = dim
        self.weight_name = weight_name
        self.has_bias = bool(getattr(spec, "bias", True))
        self.bias_name = weight_name + spec.bias_suffix
        self.out_dtype = build.dtype
        self.gain = self.bias = None

    def weight_specs(self):
        out = [WeightSpec(self.weight_name, (self.dim,), init="gain")]
        if self.has_bias:
            out.append(WeightSpec(self.bias_name, (self.dim,), init="bias"))
        return out

    def load(self, get):
        self.gain = get(self.weight_name)
        # a norm without a bias runs the same kernel with zeros in its place
        self.bias = get(self.bias_name) if self.has_bias else torch.zeros_like(self.gain)
        if self.gain.dtype != self.bias.dtype:
            self.gain, self.bias = self.gain.float(), self.bias.float()

    def scale_output(self, factor: float) -> None:
        """From now on the norm's output is ``factor`` times what it was (weight and bias in fp32): for a product
        behind it whose result is scaled by a constant."""
        if factor != 1.0:
            self.gain = (self.gain.float() * factor).contiguous()
            self.bias = (self.bias.float() * factor).contiguous()

    def forward(self, x, rows=None):
        return ops.layernorm_seam(x, self.eps, nxt=(self.gain, self.bias), out_dtype=self.out_dtype, rows=rows)

    def seam(self, residual, branches, scales, add_vec=None, then=None):
        """``residual += this norm of (sum_i scales[i] * branches[i])`` (one or two branches, [rows, width] each);
        then ``residual += add_vec``; returns ``then``'s norm of the new rows (``then``: a LayerNorm part or None)."""
        if not 1 <= len(branches) <= 2 or len(scales) != len(branches):
            raise ValueError("the seam takes one or two branches with a scale each")
        a2 = branches[1] if len(branches) == 2 else None
        s2 = scales[1] if len(branches) == 2 else 0.0
        vecs = [self.gain, self.bias]
        nxt = None
        if then is not None:
            if then.eps != self.eps:
                raise ValueError("the norms of one seam share their eps")
            nxt = (then.gain, then.bias)
            vecs += list(nxt)
        if add_vec is not None:
            vecs.append(add_vec)
        if any(v.dtype != self.gain.dtype for v in vecs):  # one launch takes one type for all of them
            out = ops.layernorm_seam(residual, self.eps, a=branches[0], a2=a2, s1=scales[0], s2=s2, post=(self.gain, self.bias))
            if add_vec is not None:
                ops.layernorm_seam(residual, self.eps, add_vec=add_vec)
            return then.forward(residual) if then is not None else None
        return ops.layernorm_seam(residual, self.eps, a=branches[0], a2=a2, s1=scales[0], s2=s2, post=(self.gain, self.bias),
                                  add_vec=add_vec, nxt=nxt, out_dtype=then.out_dtype if then is not None else None)


register_part("norm", "layernorm", LayerNorm, replace=True)


class DynTanh(Part):
    """tanh(alpha * x) * w + b element by element in fp32 (weight, bias and slope are held in fp32 whatever the run's
    type): no mean, no variance, no eps. ``forward`` also reads several residual streams as one weighted sum first
    (``read`` fp32 [streams], ``x`` [rows, streams x width]) and can write its result several times side by side."""

    def __init__(self, spec: DynTanhSpec, dim: int, weight_name: str, build: BuildContext):
        self.dim = dim
        self.weight_name = weight_name
        self.bias_name = weight_name + spec.bias_suffix
        self.alpha_name = weight_name + spec.alpha_suffix
        self.out_dtype = build.dtype
        self.gain = self.bias = self.alpha = None

    def weight_specs(self):
        return [WeightSpec(self.weight_name, (self.dim,), init="gain"), WeightSpec(self.bias_name, (self.dim,), init="bias"),
                WeightSpec(self.alpha_name, (), init="gain")]

    def load(self, get):
        self.gain = get(self.weight_name).float().contiguous()
        self.bias = get(self.bias_name).float().contiguous()
        self.alpha = get(self.alpha_name).float().reshape(1).contiguous()

    def vectors(self):
        """(weight, bias, alpha) as the stream kernels take them."""
        return self.gain, self.bias, self.alpha

    def forward(self, x, rows=None, read=None, out_dtype=None, copies=1):
        streams = read.numel() if read is not None else 1
        return ops.dyntanh(x, self.gain, self.bias, self.alpha, out_dtype or self.out_dtype, streams=streams, read=read,
                           rows=rows, copies=copies)


register_part("norm", "dyntanh", DynTanh, replace=True)
