"""Arrangements of parts in a block.  Post-norm: the branches read the stream itself and are normed on their way out,
``x += post(mixer(x)); x += post(feed_forward(x))``.  Parallel: one norm feeds both branches, ``x += mixer(norm(x)) + feed_forward(norm(x))``.
Multi-stream: pre-norm over several residual streams, a branch reading ``sum_s in[s] x_s`` and written back as
``x_t = sum_s mix[s, t] x_s + out[t] y``.  Sandwich: a norm before and one after each branch,
``x += post(mixer(pre(x))); x += post(feed_forward(pre(x)))``.  Pre-norm (``crates/mach-model/src/batched.rs:3180-3200,
4031, 4050, 4453``): ``x += mixer(norm(x)); x += feed_forward(norm(x))``."""
from __future__ import annotations

from .base import Block, MultiStream, Part, TensorDecl
from .registry import FEED_FORWARDS, MIXERS, NORMS, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """Reads ``mixer``, ``feed_forward`` (may be None, then its norm too), ``mixer_norm`` and ``feed_forward_norm`` of its
    layer's spec."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer = MIXERS.build(spec.mixer, rt)
        self.mixer_norm = NORMS.build(spec.mixer_norm, rt)
        self.feed_forward = self.feed_forward_norm = None
        if spec.feed_forward is not None:
            self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, rt)
            self.feed_forward_norm = NORMS.build(spec.feed_forward_norm, rt)

    def parts(self):
        return [self.mixer_norm, self.mixer] + ([self.feed_forward_norm, self.feed_forward] if self.feed_forward is not None else [])

    def forward(self, stream, ctx):
        self.mixer.forward(self._input(self.mixer_norm, self.mixer, stream), stream, ctx)
        if self.feed_forward is not None:
            self.feed_forward.forward(self._input(self.feed_forward_norm, self.feed_forward, stream), stream, ctx)

    @staticmethod
    def _input(norm, reader, stream):
        """The reader's normalised input: a tensor, or for a reader that starts with a product over it
        the norm left pending, so that the product's kernel can apply it."""
        if reader.takes_pending_norm:
            pending = norm.pending(stream)
            if pending is not None:
                return pending
        return norm.forward(stream)


@register_block("parallel")
class ParallelBlock(Block):
    """One norm for both branches, ``h = norm(x); x += mixer(h) + feed_forward(h)``.  Reads ``mixer``, ``feed_forward``
    (may be None) and ``norm`` of its layer's spec.  Both branches end in a product that adds into the 32-bit stream."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer = MIXERS.build(spec.mixer, rt)
        self.norm = NORMS.build(spec.norm, rt)
        self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, rt) if spec.feed_forward is not None else None

    def parts(self):
        return [self.norm, self.mixer] + ([self.feed_forward] if self.feed_forward is not None else [])

    def forward(self, stream, ctx):
        h = self.norm.forward(stream)  # a tensor: two readers share it
        self.mixer.forward(h, stream, ctx)
        if self.feed_forward is not None:
            self.feed_forward.forward(h, stream, ctx)


class _Branch:
    """What a branch of a sandwich block writes to in the stream's place: it keeps the branch's output, as the
    operands of its last product or as a finished tensor, for the norm that follows."""

    def __init__(self, ops):
        self.ops = ops
        self.product = None
        self.bias = None
        self.tensor = None
        self.branches = None
        self.scaled = None

    def add_linear(self, a, w, bias=None) -> None:
        self.product, self.bias = (a, w), bias

    def add_normed_mean(self, branches, eps) -> None:
        self.branches = (list(branches), eps)

    def add(self, y) -> None:
        self.tensor = y

    def add_rows_scaled(self, h, weights, first, count) -> None:
        self.scaled = (h, weights, first, count)


class StreamMix(Part):
    """The three small tensors with which one branch reads and writes several streams."""

    def tensor_decls(self):
        n = self.spec.streams
        return [TensorDecl("in", (n,), "vector"), TensorDecl("out", (n,), "vector"), TensorDecl("mix", (n, n), "vector")]

    def load(self, t):
        self.w_in, self.w_out, self.w_mix = t["in"], t["out"], t["mix"]


@register_block("multistream")
class MultiStreamBlock(Block):
    """Pre-norm over several residual streams (``base.MultiStream``).  Reads ``mixer``, ``feed_forward`` (may be None),
    ``mixer_norm``, ``feed_forward_norm``, ``mixer_streams`` and ``feed_forward_streams`` of its layer's spec.  A branch's
    input is the norm of ``sum_s in[s] x_s`` (one kernel for the sum and an RMS norm, which also writes what the branch before
    left); what it leaves (the operands of a
    last product, a bias, a finished tensor, rows of its input to be added with weights) is written into all streams by
    one kernel that also adds the product's partial sums up."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer = MIXERS.build(spec.mixer, rt)
        self.mixer_norm = NORMS.build(spec.mixer_norm, rt)
        self.mixer_streams = StreamMix(spec.mixer_streams, rt)
        self.feed_forward = self.feed_forward_norm = self.feed_forward_streams = None
        if spec.feed_forward is not None:
            self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, rt)
            self.feed_forward_norm = NORMS.build(spec.feed_forward_norm, rt)
            self.feed_forward_streams = StreamMix(spec.feed_forward_streams, rt)

    def parts(self):
        out = [self.mixer_norm, self.mixer, self.mixer_streams]
        if self.feed_forward is not None:
            out += [self.feed_forward_norm, self.feed_forward, self.feed_forward_streams]
        return out

    def forward(self, stream, ctx):
        if not isinstance(stream, MultiStream):
            raise TypeError("a multi-stream block in a model of one residual stream: the model's spec names no streams")
        self._branch(self.mixer_norm, self.mixer, self.mixer_streams, stream, ctx)
        if self.feed_forward is not None:
            self._branch(self.feed_forward_norm, self.feed_forward, self.feed_forward_streams, stream, ctx)

    def _branch(self, norm, part, mix, stream, ctx):
        ops = self.rt.ops
        if type(norm).__name__ == "RMSNorm" and hasattr(ops, "streams_read_norm"):
            h = stream.read_norm(mix.w_in, norm.weight, norm.spec.eps)  # one kernel with the write before it, if one is pending
        else:
            h = norm.forward(stream.read(mix.w_in))
        out = _Branch(ops)
        part.forward(h, out, ctx)
        if out.product is not None:
            sums = ops.linear_split(*out.product)
        elif out.tensor is not None:
            sums = out.tensor.float().contiguous().unsqueeze(0)
        else:
            raise ValueError(f"{type(part).__name__} left neither a last product nor a finished tensor")
        if out.scaled is not None:  # into the first of the sums, which nobody else holds
            ops.add_scaled_rows(sums[0], *out.scaled)
        stream.write(sums, out.bias, mix.w_mix, mix.w_out)


@register_block("sandwich")
class SandwichBlock(Block):
    """Reads ``mixer``, ``feed_forward`` (may be None), ``mixer_norm``, ``mixer_post_norm``, ``feed_forward_norm`` and
    ``feed_forward_post_norm`` of its layer's spec.  A post norm is a norm with ``add_normed``."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer = MIXERS.build(spec.mixer, rt)
        self.mixer_norm = NORMS.build(spec.mixer_norm, rt)
        self.mixer_post_norm = NORMS.build(spec.mixer_post_norm, rt)
        self.feed_forward = self.feed_forward_norm = self.feed_forward_post_norm = None
        if spec.feed_forward is not None:
            self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, rt)
            self.feed_forward_norm = NORMS.build(spec.feed_forward_norm, rt)
            self.feed_forward_post_norm = NORMS.build(spec.feed_forward_post_norm, rt)

    def parts(self):
        out = [self.mixer_norm, self.mixer, self.mixer_post_norm]
        if self.feed_forward is not None:
            out += [self.feed_forward_norm, self.feed_forward, self.feed_forward_post_norm]
        return out

    def forward(self, stream, ctx):
        self._branch(self.mixer_norm, self.mixer, self.mixer_post_norm, stream, ctx)
        if self.feed_forward is not None:
            self._branch(self.feed_forward_norm, self.feed_forward, self.feed_forward_post_norm, stream, ctx)

    def _branch(self, pre, part, post, stream, ctx):
        out = _Branch(self.rt.ops)
        part.forward(PreNormBlock._input(pre, part, stream), out, ctx)
        stream.flush()  # a norm left pending has added what was pending by now; nothing else may be
        if out.product is not None:
            post.add_normed(stream, *out.product)
        else:
            post.add_normed_tensor(stream, out.tensor)


@register_block("postnorm")
class PostNormBlock(Block):
    """Reads ``mixer``, ``feed_forward`` (may be None), ``mixer_post_norm`` and ``feed_forward_post_norm`` of its layer's
    spec.  A branch gets the stream's rows in the element type, or, if it says ``reads_stream``, the 32-bit rows
    themselves; what it leaves (a last product with or without bias, branches side by side, a finished tensor) is
    normed and added by the post norm's own kernel."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        self.mixer = MIXERS.build(spec.mixer, rt)
        self.mixer_post_norm = NORMS.build(spec.mixer_post_norm, rt)
        self.feed_forward = self.feed_forward_post_norm = None
        if spec.feed_forward is not None:
            self.feed_forward = FEED_FORWARDS.build(spec.feed_forward, rt)
            self.feed_forward_post_norm = NORMS.build(spec.feed_forward_post_norm, rt)

    def parts(self):
        out = [self.mixer, self.mixer_post_norm]
        if self.feed_forward is not None:
            out += [self.feed_forward, self.feed_forward_post_norm]
        return out

    def forward(self, stream, ctx):
        self._branch(self.mixer, self.mixer_post_norm, stream, ctx)
        if self.feed_forward is not None:
            self._branch(self.feed_forward, self.feed_forward_post_norm, stream, ctx)

    def _branch(self, part, post, stream, ctx):
        out = _Branch(self.rt.ops)
        x = stream.value()
        part.forward(x if getattr(part, "reads_stream", False) else self.rt.ops.round_rows(x), out, ctx)
        if out.branches is not None:
            post.add_normed_mean(stream, *out.branches)
        elif out.product is not None:
            post.add_normed(stream, *out.product, bias=out.bias)
        else:
            post.add_normed_tensor(stream, out.tensor)
