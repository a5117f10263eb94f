"""How the parts of one layer are arranged.

"prenorm" (model/LayerSpec.java:18-19; cpu/CpuBackend.java:959-969): xb = norm_in(x); x += mixer(xb);
xb = norm_post(x); x += ffn(xb). The residual stream x is fp32 and is never normalised itself.

Norms between two products need no launch of their own when both sides agree (optional, by attributes of the
parts; a part that knows nothing of this works as before):
* a mixer / feed-forward with ``takes_normed_rows = True`` only feeds its input to ``ops.gemm`` and so may get the
  norm as a promise (``norm.defer`` / ``ops.NormedRows``) instead of a tensor;
* one with ``prepares_next_norm = True`` takes ``then_norm=<norm part>`` in ``forward``, ends with
  ``then_norm.after_add(...)`` instead of the add into the residual, and returns that promise.
"""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import WeightSpec
from .base import Part, part_factory, register_part


class PreNormBlock(Part):
    def __init__(self, spec, prefix, build, positions):
        ending = getattr(spec, "name_ending", ".weight")
        self.norm_in = part_factory("norm", spec.norm.kind)(spec.norm, build.hidden, f"{prefix}.{spec.norm_in_name}{ending}", build)
        mixer_prefix = f"{prefix}.{spec.mixer_prefix}" if getattr(spec, "mixer_prefix", "") else prefix
        self.mixer = part_factory("mixer", spec.mixer.kind)(spec.mixer, mixer_prefix, build, positions)
        if spec.ffn is None:  # a layer of a mixer alone: no second norm, no feed-forward
            self.norm_post = self.ffn = None
            self.parts = (self.norm_in, self.mixer)
        else:
            self.norm_post = part_factory("norm", spec.norm.kind)(spec.norm, build.hidden,
                                                                f"{prefix}.{spec.norm_post_name}{ending}", build)
            self.ffn = part_factory("ffn", spec.ffn.kind)(spec.ffn, prefix, build)
            self.parts = (self.norm_in, self.mixer, self.norm_post, self.ffn)
        self.capturable = all(getattr(p, "capturable", True) for p in self.parts)

    def weight_specs(self):
        return [w for p in self.parts for w in p.weight_specs()]

    def load(self, get):
        for p in self.parts:
            p.load(get)

    def cache_spec(self):
        return self.mixer.cache_spec()

    def state_spec(self):
        return self.mixer.state_spec()

    def step_planners(self):
        return [pl for p in self.parts for pl in (p.step_planners() if hasattr(p, "step_planners") else [])]

    chains_norms = True  # forward takes normed_in / next_norm and returns the next block's input promise

    @staticmethod
    def _input(norm, consumer, x, promise):
        if getattr(consumer, "takes_normed_rows", False) and hasattr(norm, "defer"):
            if promise is not None and getattr(promise, "x", None) is x and promise.gain is getattr(norm, "gain", None):
                return promise
            return norm.defer(x)
        return norm.forward(x)

    def forward(self, x, step, slot, normed_in=None, next_norm=None):
        """``normed_in``: norm_in of x, prepared by whoever wrote x last (or None); ``next_norm``: the norm part that
        will read x next. Returns that norm of the new x as a promise when the feed-forward prepared it."""
        xb = self._input(self.norm_in, self.mixer, x, normed_in)
        if self.ffn is None:
            if next_norm is not None and getattr(self.mixer, "prepares_next_norm", False) and hasattr(next_norm, "after_add"):
                return self.mixer.forward(xb, x, step, slot, then_norm=next_norm)
            self.mixer.forward(xb, x, step, slot)
            return None
        if getattr(self.mixer, "prepares_next_norm", False) and hasattr(self.norm_post, "after_add"):
            mid = self.mixer.forward(xb, x, step, slot, then_norm=self.norm_post)
        else:
            self.mixer.forward(xb, x, step, slot)
            mid = None
        xb = self._input(self.norm_post, self.ffn, x, mid)
        if next_norm is not None and getattr(self.ffn, "prepares_next_norm", False) and hasattr(next_norm, "after_add"):
            return self.ffn.forward(xb, x, step, then_norm=next_norm)
        self.ffn.forward(xb, x, step)
        return None


register_part("arrangement", "prenorm", PreNormBlock, replace=True)


def sublayer_output(part, xb, step, slot, width):
    """A mixer's or feed-forward's output as fp32 rows of its own, [rows, width]: its ``output`` method where it has
    one, else what it adds into a cleared tensor."""
    args = (step,) if slot is None else (step, slot)
    if hasattr(part, "output"):
        return part.output(xb, *args)
    out = torch.empty((step.n_tokens, width), dtype=torch.float32, device=xb.device).zero_()
    part.forward(xb, out, *args)
    return out


class SandwichBlock(Part):
    """A norm in front of and behind each sublayer: x += norm_mixer_out(mixer(norm_in(x))); x += norm_ffn_out(ffn(
    norm_post(x))). Where the norm part offers a ``seam`` (parts/norm.py: LayerNorm), the norm of a sublayer's output,
    its add into the stream, a vector that joins the stream before the next layer, and the next sublayer's input norm
    are one launch, handed on as the next block's input."""

    chains_norms = True
    takes_stream_vector = True  # forward(..., add_after=) adds that vector to the stream as its last act

    def __init__(self, spec, prefix, build, positions):
        ending = getattr(spec, "name_ending", ".weight")
        make = part_factory("norm", spec.norm.kind)

        def norm(name):
            if not name:
                raise ValueError(f"{prefix}: the sandwich arrangement names four norms")
            return make(spec.norm, build.hidden, f"{prefix}.{name}{ending}", build)

        self.width = build.hidden
        self.norm_in = norm(spec.norm_in_name)
        self.norm_mixer_out = norm(spec.norm_mixer_out_name)
        mixer_prefix = f"{prefix}.{spec.mixer_prefix}" if getattr(spec, "mixer_prefix", "") else prefix
        self.mixer = part_factory("mixer", spec.mixer.kind)(spec.mixer, mixer_prefix, build, positions)
        if spec.ffn is None:
            self.norm_post = self.norm_ffn_out = self.ffn = None
            self.parts = (self.norm_in, self.mixer, self.norm_mixer_out)
        else:
            self.norm_post = norm(spec.norm_post_name)
            self.norm_ffn_out = norm(spec.norm_ffn_out_name)
            self.ffn = part_factory("ffn", spec.ffn.kind)(spec.ffn, prefix, build)
            self.parts = (self.norm_in, self.mixer, self.norm_mixer_out, self.norm_post, self.ffn, self.norm_ffn_out)
        self.capturable = all(getattr(p, "capturable", True) for p in self.parts)

    def weight_specs(self):
        return [w for p in self.parts for w in p.weight_specs()]

    def load(self, get):
        for p in self.parts:
            p.load(get)

    def cache_spec(self):
        return self.mixer.cache_spec()

    def state_spec(self):
        return self.mixer.state_spec()

    def step_planners(self):
        return [pl for p in self.parts for pl in (p.step_planners() if hasattr(p, "step_planners") else [])]

    @staticmethod
    def _join(norm, x, branch, add_vec, then):
        """x += norm(branch) (+ add_vec); returns then's norm of the new x, or None when nobody prepared it."""
        if hasattr(norm, "seam") and (then is None or hasattr(then, "seam")):
            return norm.seam(x, [branch], [1.0], add_vec=add_vec, then=then)
        x += norm.forward(branch).float()
        if add_vec is not None:
            x += add_vec.float()
        return None

    def forward(self, x, step, slot, normed_in=None, next_norm=None, add_after=None):
        """``normed_in``: norm_in of x as the block before left it (a tensor) or None; ``next_norm``: the norm part that
        reads x next; ``add_after``: a vector that joins the stream behind this layer. Returns ``next_norm`` of the new
        x when the last seam prepared it."""
        xb = normed_in if isinstance(normed_in, torch.Tensor) else self.norm_in.forward(x)
        then, vec = (next_norm, add_after) if self.ffn is None else (self.norm_post, None)
        scales = getattr(getattr(self.mixer, "spec", None), "scales", ())
        if hasattr(self.mixer, "outputs") and not getattr(self.mixer, "fused", False) and len(scales) == 2 \
                and hasattr(self.norm_mixer_out, "seam") \
                and (then is None or hasattr(then, "seam")):
            # two weighted branches: their sum is taken inside the seam's launch
            xb = self.norm_mixer_out.seam(x, self.mixer.outputs(xb, step, slot), list(scales), add_vec=vec, then=then)
        else:
            xb = self._join(self.norm_mixer_out, x, sublayer_output(self.mixer, xb, step, slot, self.width), vec, then)
        if self.ffn is None:
            return xb
        if xb is None:
            xb = self.norm_post.forward(x)
        branch = sublayer_output(self.ffn, xb, step, None, self.width)
        return self._join(self.norm_ffn_out, x, branch, add_after, next_norm)


register_part("arrangement", "sandwich", SandwichBlock, replace=True)


class ParallelBlock(Part):
    """One norm, two readers: with h = norm_in(x), x += mixer(h) + ffn(h). Both sublayers add their output into the
    fp32 stream themselves (the mixer first, then the feed-forward), so the sum is taken in the stream."""

    chains_norms = False

    def __init__(self, spec, prefix, build, positions):
        ending = getattr(spec, "name_ending", ".weight")
        self.norm_in = part_factory("norm", spec.norm.kind)(spec.norm, build.hidden, f"{prefix}.{spec.norm_in_name}{ending}", build)
        mixer_prefix = f"{prefix}.{spec.mixer_prefix}" if getattr(spec, "mixer_prefix", "") else prefix
        self.mixer = part_factory("mixer", spec.mixer.kind)(spec.mixer, mixer_prefix, build, positions)
        self.ffn = part_factory("ffn", spec.ffn.kind)(spec.ffn, prefix, build) if spec.ffn is not None else None
        self.parts = tuple(p for p in (self.norm_in, self.mixer, self.ffn) if p is not None)
        self.capturable = all(getattr(p, "capturable", True) for p in self.parts)

    def weight_specs(self):
        return [w for p in self.parts for w in p.weight_specs()]

    def load(self, get):
        for p in self.parts:
            p.load(get)

    def cache_spec(self):
        return self.mixer.cache_spec()

    def state_spec(self):
        return self.mixer.state_spec()

    def step_planners(self):
        return [pl for p in self.parts for pl in (p.step_planners() if hasattr(p, "step_planners") else [])]

    def forward(self, x, step, slot):
        h = self.norm_in.forward(x)  # a tensor: both readers need the same rows
        self.mixer.forward(h, x, step, slot)
        if self.ffn is not None:
            self.ffn.forward(h, x, step)


register_part("arrangement", "parallel", ParallelBlock, replace=True)


class StreamReader:
    """How a sublayer of a hyper-connected layer gets its input: the weighted sum of the row's streams, then the norm.
    The block before may have made it already, in the launch that wrote the streams (``HyperBlock.forward(next_norm=)``)."""

    def __init__(self, read_name: str, norm):
        self.read_name = read_name
        self.norm = norm
        self.read = None  # fp32 [streams]

    def vectors(self):
        return (self.read,) + tuple(self.norm.vectors())

    def forward(self, x):
        return self.norm.forward(x, read=self.read)


class HyperBlock(Part):
    """Hyper-connections: a row has ``streams`` copies x_1 .. x_s of the residual (fp32, side by side). Sublayer q (the
    mixer, then the feed-forward) reads u = sum_s in_q[s] x_s, computes y = sublayer(norm_q(u)), and every stream is
    rewritten from the previous ones together: x_t <- sum_s mix_q[s, t] x_s + out_q[t] * y. The weights are the tensors
    ``<prefix>.<name>.in`` [streams], ``.out`` [streams] and ``.mix`` [streams, streams] (row: the stream read, column: the stream written), held in
    fp32. Writing the streams and reading the next sublayer's input from them is one launch (``ops.streams_write``), so
    a layer costs two such launches beside its sublayers; the norm must be one that takes no statistics of the row
    (``vectors()``: Dynamic Tanh)."""

    chains_norms = True

    def __init__(self, spec, prefix, build, positions):
        ending = getattr(spec, "name_ending", ".weight")
        self.streams = int(spec.streams)
        if not 1 <= self.streams <= ops.MAX_STREAMS:
            raise ValueError(f"{prefix}: {self.streams} residual streams (1..{ops.MAX_STREAMS} are built)")
        self.width = build.hidden
        self.dtype = build.dtype
        make = part_factory("norm", spec.norm.kind)
        norm1 = make(spec.norm, build.hidden, f"{prefix}.{spec.norm_in_name}{ending}", build)
        if not hasattr(norm1, "vectors"):
            raise ValueError(f"{prefix}: the hyper arrangement reads its streams inside the norm's launch; norm '{spec.norm.kind}' does not offer that")
        self.names = [f"{prefix}.{n}" for n in spec.hyper_names]
        self.norm_in = StreamReader(self.names[0] + ".in", norm1)
        mixer_prefix = f"{prefix}.{spec.mixer_prefix}" if getattr(spec, "mixer_prefix", "") else prefix
        self.mixer = part_factory("mixer", spec.mixer.kind)(spec.mixer, mixer_prefix, build, positions)
        if spec.ffn is None:
            self.norm_post = self.ffn = None
            self.parts = (norm1, self.mixer)
        else:
            norm2 = make(spec.norm, build.hidden, f"{prefix}.{spec.norm_post_name}{ending}", build)
            self.norm_post = StreamReader(self.names[1] + ".in", norm2)
            self.ffn = part_factory("ffn", spec.ffn.kind)(spec.ffn, prefix, build)
            self.parts = (norm1, self.mixer, norm2, self.ffn)
        self.capturable = all(getattr(p, "capturable", True) for p in self.parts)
        self.mix = [None, None]
        self.out = [None, None]

    def _sublayers(self):
        return 1 if self.ffn is None else 2

    def weight_specs(self):
        s = self.streams
        out = [w for p in self.parts for w in p.weight_specs()]
        for n in self.names[:self._sublayers()]:
            out += [WeightSpec(n + ".in", (s,), init="gain"), WeightSpec(n + ".out", (s,), init="gain"),
                    WeightSpec(n + ".mix", (s, s), init="eye")]
        if self.ffn is None:  # a checkpoint may still carry the second sublayer's (unused) stream weights
            n = self.names[1]
            out += [WeightSpec(n + ".in", (s,), optional=True), WeightSpec(n + ".out", (s,), optional=True),
                    WeightSpec(n + ".mix", (s, s), optional=True)]
        return out

    def load(self, get):
        for p in self.parts:
            p.load(get)
        readers = (self.norm_in, self.norm_post)
        for q in range(self._sublayers()):
            readers[q].read = get(self.names[q] + ".in").float().contiguous()
            self.out[q] = get(self.names[q] + ".out").float().contiguous()
            self.mix[q] = get(self.names[q] + ".mix").float().contiguous()

    def cache_spec(self):
        return self.mixer.cache_spec()

    def state_spec(self):
        return self.mixer.state_spec()

    def step_planners(self):
        return [pl for p in self.parts for pl in (p.step_planners() if hasattr(p, "step_planners") else [])]

    def _write(self, q, x, y, then):
        """The streams' update behind sublayer q; returns ``then``'s input from the new streams (or None)."""
        nxt = then.vectors() if isinstance(then, StreamReader) else None
        return ops.streams_write(x, y, self.mix[q], self.out[q], nxt=nxt, out_dtype=self.dtype)

    def forward(self, x, step, slot, normed_in=None, next_norm=None):
        """``x``: fp32 [rows, streams x width]. ``normed_in``: this block's first input as the block before left it (a
        tensor) or None; ``next_norm``: the ``StreamReader`` of the block that runs next. Returns its input when the
        last write made it."""
        xb = normed_in if isinstance(normed_in, torch.Tensor) else self.norm_in.forward(x)
        y = sublayer_output(self.mixer, xb, step, slot, self.width)
        if self.ffn is None:
            return self._write(0, x, y, next_norm)
        xb = self._write(0, x, y, self.norm_post)
        y = sublayer_output(self.ffn, xb, step, None, self.width)
        return self._write(1, x, y, next_norm)


register_part("arrangement", "hyper", HyperBlock, replace=True)
