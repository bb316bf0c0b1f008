"""A recurrent block around a real-gated linear recurrent unit, as a mixer with state of fixed size.

Per step: the gate branch ``y = W_y h`` in the element type and the recurrent branch ``W_x h`` as 32-bit sums; a causal
convolution per channel over the recurrent branch (its last ``taps - 1`` inputs are state; the projection's bias enters
before it, the convolution's own after it); per block of channels the two gates from square maps of the convolved
input, the decay ``a = exp(-c r softplus(lam))`` and the drive ``sqrt(1 - a^2) i u``; the recurrence ``S <- a S + drive``
token after token from the request's slot (long portions in segments side by side, see ``ops.lru_scan``), times
``gelu_tanh(y + b_y)``; the output projection.  Gates, decays, the
state and the convolution are 32-bit in every build.
"""
from __future__ import annotations

from .base import Mixer, StateRequest, TensorDecl, require_kernel_sizes
from .registry import register_mixer


@register_mixer("gated_recurrence")
class GatedRecurrence(Mixer):
    graph_safe = True  # reads the requests' rows and slots from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.blocks < 1 or s.width % s.blocks:
            raise ValueError(f"gated_recurrence: {s.width} channels are not a multiple of {s.blocks} blocks")
        if s.conv_taps < 1:
            raise ValueError(f"gated_recurrence: {s.conv_taps} taps; a convolution has at least one")
        require_kernel_sizes(rt, "gated_recurrence", [("hidden size", s.hidden), ("recurrent width", s.width)])
        limits = getattr(rt.ops, "linrec_limits", None)
        if limits is not None and s.conv_taps > limits()["taps"]:
            raise ValueError(f"gated_recurrence: {s.conv_taps} taps; the convolution takes up to {limits()['taps']}")
        self.bw = s.width // s.blocks
        if limits is not None and self.bw > limits().get("lru_block", self.bw):
            raise ValueError(f"gated_recurrence: blocks of {self.bw} channels; the gates' kernel takes up to {limits()['lru_block']}")
        self.state = None

    def tensor_decls(self):
        s, c, bw = self.spec, self.spec.width, self.bw
        return [TensorDecl("y.weight", (c, s.hidden)), TensorDecl("y.bias", (c,), "vector"),
                TensorDecl("x.weight", (c, s.hidden)), TensorDecl("x.bias", (c,), "vector"),
                TensorDecl("conv.weight", (c, s.conv_taps), "vector"), TensorDecl("conv.bias", (c,), "vector"),
                TensorDecl("ra.weight", (s.blocks, bw, bw)), TensorDecl("ra.bias", (s.blocks, bw), "vector"),
                TensorDecl("ri.weight", (s.blocks, bw, bw)), TensorDecl("ri.bias", (s.blocks, bw), "vector"),
                TensorDecl("lam", (c,), "vector"), TensorDecl("o.weight", (s.hidden, c))]

    def load(self, t):
        self.w_y, self.b_y, self.w_x, self.b_x = t["y.weight"], t["y.bias"], t["x.weight"], t["x.bias"]
        self.conv_w, self.conv_b = t["conv.weight"], t["conv.bias"]
        # [block, in, out]: the gate kernel's threads are outputs and read neighbouring numbers
        self.wa_t, self.wi_t = t["ra.weight"].transpose(1, 2).contiguous(), t["ri.weight"].transpose(1, 2).contiguous()
        self.ba, self.bi = t["ra.bias"].reshape(-1).contiguous(), t["ri.bias"].reshape(-1).contiguous()
        self.lam, self.w_o = t["lam"], t["o.weight"]

    def cache_request(self):
        shapes = {"lru": (self.spec.width,)}
        if self.spec.conv_taps > 1:
            shapes["conv"] = (self.spec.conv_taps - 1, self.spec.width)
        return StateRequest(shapes)

    def bind_cache(self, binding):
        self.state = binding.tensors

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        y = ops.linear(h, self.w_y)
        u = ops.conv_sums(ops.linear_split(h, self.w_x), 0, s.width, self.b_x, self.conv_w, self.conv_b, self.state.get("conv"),
                          ctx.seq_q_start, ctx.seq_q_len, ctx.seq_slot)
        a, drive = ops.lru_gates(u, self.wa_t, self.wi_t, self.ba, self.bi, self.lam, float(s.decay_factor))
        out = ops.lru_scan(a, drive, y, 0, self.b_y, self.state["lru"], ctx.seq_q_start, ctx.seq_q_len, ctx.seq_slot)
        stream.add_linear(out, self.w_o)
