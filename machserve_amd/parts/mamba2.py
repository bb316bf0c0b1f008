"""The second Mamba layer (state-space duality) as a mixer with state of fixed size.

Per step: the input projection to ``[z | x | B | C | dt]`` as 32-bit sums; a causal convolution per channel of x, B and C
with bias, whose last ``taps - 1`` inputs of every request are state; the recurrence per head, token after token in
32-bit, ``S <- exp(-exp(A_log) dt) S + dt B x^T``, ``y = S^T C + D x`` with ``dt = softplus(. + dt_bias)`` one number a head and
token and B and C shared by the heads of a group, the ``[heads, states, head size]`` state carried in the request's slot
(SiLU on x, B and C is applied where the recurrence reads them); the gate ``y silu(z)``, RMS-normed in equal parts with a
weight per channel; the output projection.
"""
from __future__ import annotations

import torch

from .base import Mixer, StateRequest, TensorDecl, require_kernel_sizes
from .registry import register_mixer


@register_mixer("mamba2")
class StateSpaceDual(Mixer):
    graph_safe = True  # reads the requests' rows and slots from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.heads % s.groups:
            raise ValueError(f"mamba2: {s.heads} heads are not a multiple of {s.groups} groups")
        self.inner = s.heads * s.head_dim
        if self.inner % s.norm_groups:
            raise ValueError(f"mamba2: {s.norm_groups} parts of the norm do not divide {self.inner} channels")
        self.conv_channels = self.inner + 2 * s.groups * s.states
        self.out_cols = -(-self.inner // 8) * 8  # the output projection sums over a multiple of 8
        require_kernel_sizes(rt, "mamba2", [("hidden size", s.hidden)])
        limits = getattr(rt.ops, "ssd_limits", None)
        if limits is not None:
            lim = limits()
            if s.states > lim["states"] or s.head_dim > lim["head_dim"]:
                raise ValueError(f"mamba2: {s.states} states and heads of {s.head_dim}; the kernels take up to {lim['states']} and {lim['head_dim']}")
        limits = getattr(rt.ops, "linrec_limits", None)
        if limits is not None and s.conv_taps > limits()["taps"]:
            raise ValueError(f"mamba2: {s.conv_taps} taps; the convolution takes up to {limits()['taps']}")
        self.state = None

    def tensor_decls(self):
        s = self.spec
        return [TensorDecl("in.weight", (2 * self.inner + 2 * s.groups * s.states + s.heads, s.hidden)),
                TensorDecl("conv.weight", (self.conv_channels, s.conv_taps), "vector"), TensorDecl("conv.bias", (self.conv_channels,), "vector"),
                TensorDecl("dt_bias", (s.heads,), "vector"), TensorDecl("A_log", (s.heads,), "vector"), TensorDecl("D", (s.heads,), "vector"),
                TensorDecl("norm", (self.inner,), "vector"), TensorDecl("o.weight", (s.hidden, self.inner))]

    def load(self, t):
        self.w_in = t["in.weight"]
        self.conv_w, self.conv_b = t["conv.weight"], t["conv.bias"]
        self.dt_bias, self.a_log, self.d_skip, self.norm_w = t["dt_bias"], t["A_log"], t["D"], t["norm"]
        self.w_o = torch.nn.functional.pad(t["o.weight"], (0, self.out_cols - self.inner)).contiguous()

    def cache_request(self):
        s = self.spec
        return StateRequest({"conv": (max(s.conv_taps - 1, 1), self.conv_channels), "ssm": (s.heads, s.states, s.head_dim)})

    def bind_cache(self, binding):
        self.state = binding.tensors

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        seqs = (ctx.seq_q_start, ctx.seq_q_len, ctx.seq_slot)
        proj = ops.linear(h, self.w_in, None, out_f32=True)
        xbc = ops.conv_sums(proj, self.inner, self.conv_channels, None, self.conv_w, self.conv_b, self.state["conv"], *seqs)
        y = ops.ssd_scan(xbc, proj, self.inner + self.conv_channels, self.dt_bias, self.a_log, self.d_skip, self.state["ssm"], *seqs,
                         s.heads, s.head_dim, s.states, s.groups)
        yn = ops.gated_group_norm(y, proj, 0, self.norm_w, s.norm_eps, s.norm_groups, self.out_cols)
        stream.add_linear(yn, self.w_o)
