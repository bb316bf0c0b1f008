"""A feed-forward of many small experts ``W_down act(W_up h)`` of which a token uses a few, with an optional expert that
every token uses.

The router's logits are 32-bit sums over 32-bit weights; a row's ``top`` largest choose its experts and the softmax
over the chosen logits alone weighs them.  All experts' up projections are one matrix and their down projections one
matrix: the up product runs for every expert, one kernel applies the activation and the row's weight for the expert
(an exact zero for an expert the row did not choose, one for the expert that every row uses), and the down product
sums the chosen experts' outputs.  A row's result depends on its own logits alone.
"""
from __future__ import annotations

import torch

from .base import FeedForward, TensorDecl, require_kernel_sizes
from .registry import register_feed_forward


@register_feed_forward("routed_mlp")
class RoutedMlp(FeedForward):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if not 1 <= s.top <= s.experts:
            raise ValueError(f"routed_mlp: {s.top} of {s.experts} experts a token")
        require_kernel_sizes(rt, "routed_mlp", [("hidden size", s.hidden)])
        limits = getattr(rt.ops, "route_limits", None)
        if limits is not None and (s.experts > limits()["experts"] or s.top > limits()["top"]):
            raise ValueError(f"routed_mlp: {s.top} of {s.experts} experts; the router takes up to {limits()['top']} of {limits()['experts']}")
        if s.activation not in getattr(rt.ops, "EXPERT_ACTIVATIONS", {s.activation: 0}):
            raise ValueError(f"routed_mlp: activation {s.activation!r} is not built")
        self.columns = s.experts * s.intermediate + s.shared

    def tensor_decls(self):
        s = self.spec
        decls = [TensorDecl("router.weight", (s.experts, s.hidden), "vector")]
        if s.router_bias:
            decls.append(TensorDecl("router.bias", (s.experts,), "vector"))
        for e in range(s.experts):
            decls += [TensorDecl(f"e{e}.up", (s.intermediate, s.hidden)), TensorDecl(f"e{e}.down", (s.hidden, s.intermediate))]
        if s.shared:
            decls += [TensorDecl("shared.up", (s.shared, s.hidden)), TensorDecl("shared.down", (s.hidden, s.shared))]
        return decls

    def load(self, t):
        s = self.spec
        self.w_router, self.b_router = t["router.weight"], t.get("router.bias")
        ups, downs = [t[f"e{e}.up"] for e in range(s.experts)], [t[f"e{e}.down"] for e in range(s.experts)]
        if s.shared:
            ups.append(t["shared.up"])
            downs.append(t["shared.down"])
        fill = -self.columns % 8  # the down product sums over a multiple of 8: columns of zeros
        if fill:
            ups.append(ups[0].new_zeros((fill, s.hidden)))
            downs.append(downs[0].new_zeros((s.hidden, fill)))
        self.w_up, self.w_down = torch.cat(ups, dim=0).contiguous(), torch.cat(downs, dim=1).contiguous()

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        gates = ops.route(h, self.w_router, self.b_router, s.top)
        up = ops.linear(h, self.w_up, None, out_f32=True)
        stream.add_linear(ops.expert_act(up, gates, s.intermediate, s.activation), self.w_down)
