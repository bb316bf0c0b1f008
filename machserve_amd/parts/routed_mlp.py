"""A feed-forward of many small experts ``W_down act(W_up h)`` of which a token uses a few, with an optional expert that
every token uses.

The router's logits are 32-bit sums over 32-bit weights; a row's ``top`` largest choose its experts and the softmax
over the chosen logits alone weighs them.  All experts' up projections are one matrix and their down projections one
matrix: the up product runs for every expert, one kernel applies the activation and the row's weight for the expert
(an exact zero for an expert the row did not choose, one for the expert that every row uses), and the down product
sums the chosen experts' outputs.  A row's result depends on its own logits alone.

Variants that the spec names: experts with a gate, ``W_down (act(W_gate h) * (W_up h))`` (all gates are the first half of
the one up matrix); scores that are the softmax over every router output, a correction added for the choice only, and
weights that are the chosen scores over their sum; and router outputs beyond the experts that stand for experts without
tensors which return their input (the rows of the input are added with those weights).
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
        if not 1 <= s.top <= s.experts + int(getattr(s, "identity", 0)):
            raise ValueError(f"routed_mlp: {s.top} of {s.experts} experts a token")
        require_kernel_sizes(rt, "routed_mlp", [("hidden size", s.hidden)])
        limits = getattr(rt.ops, "route_limits", None)
        if limits is not None and (s.experts > limits()["experts"] or s.top > limits()["top"]):
            raise ValueError(f"routed_mlp: {s.top} of {s.experts} experts; the router takes up to {limits()['top']} of {limits()['experts']}")
        if s.activation not in getattr(rt.ops, "EXPERT_ACTIVATIONS", {s.activation: 0}):
            raise ValueError(f"routed_mlp: activation {s.activation!r} is not built")
        self.columns = s.experts * s.intermediate + s.shared
        self.gated, self.identity = bool(getattr(s, "gated", False)), int(getattr(s, "identity", 0))
        self.scoring, self.correction = getattr(s, "scoring", "softmax_chosen"), bool(getattr(s, "correction", False))
        if self.scoring not in ("softmax_chosen", "softmax_all"):
            raise ValueError(f"routed_mlp: scoring {self.scoring!r} (softmax_chosen, softmax_all)")
        if self.gated and s.shared:
            raise ValueError("routed_mlp: an expert that every token uses beside gated experts is not built")
        if self.correction and self.scoring != "softmax_all":
            raise ValueError("routed_mlp: a correction of the choice goes with scores over all router outputs")
        if s.top > s.experts + self.identity:
            raise ValueError(f"routed_mlp: {s.top} of {s.experts + self.identity} router outputs a token")

    def tensor_decls(self):
        s = self.spec
        outputs = s.experts + self.identity
        decls = [TensorDecl("router.weight", (outputs, s.hidden), "vector")]
        if s.router_bias:
            decls.append(TensorDecl("router.bias", (outputs,), "vector"))
        if self.correction:
            decls.append(TensorDecl("correction", (outputs,), "vector"))
        for e in range(s.experts):
            decls += [TensorDecl(f"e{e}.up", (s.intermediate, s.hidden)), TensorDecl(f"e{e}.down", (s.hidden, s.intermediate))]
            if self.gated:
                decls.append(TensorDecl(f"e{e}.gate", (s.intermediate, s.hidden)))
        if s.shared:
            decls += [TensorDecl("shared.up", (s.shared, s.hidden)), TensorDecl("shared.down", (s.hidden, s.shared))]
        return decls

    def load(self, t):
        s = self.spec
        self.w_router, self.b_router, self.w_correction = t["router.weight"], t.get("router.bias"), t.get("correction")
        ups, downs = [t[f"e{e}.up"] for e in range(s.experts)], [t[f"e{e}.down"] for e in range(s.experts)]
        if s.shared:
            ups.append(t["shared.up"])
            downs.append(t["shared.down"])
        fill = -self.columns % 8  # the down product sums over a multiple of 8: columns of zeros
        if fill:
            ups.append(ups[0].new_zeros((fill, s.hidden)))
            downs.append(downs[0].new_zeros((s.hidden, fill)))
        if self.gated:  # every expert's gate, then every expert's up projection
            gates = [t[f"e{e}.gate"] for e in range(s.experts)] + ([ups[0].new_zeros((fill, s.hidden))] if fill else [])
            ups = gates + ups
        self.w_up, self.w_down = torch.cat(ups, dim=0).contiguous(), torch.cat(downs, dim=1).contiguous()

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        if self.scoring == "softmax_all":
            gates = ops.route(h, self.w_router, self.b_router, s.top, correction=self.w_correction, softmax_all=True)
        else:
            gates = ops.route(h, self.w_router, self.b_router, s.top)
        up = ops.linear(h, self.w_up, None, out_f32=True)
        if self.gated or self.identity:
            a = ops.expert_act(up, gates, s.intermediate, s.activation, experts=s.experts, gated=self.gated)
        else:
            a = ops.expert_act(up, gates, s.intermediate, s.activation)
        stream.add_linear(a, self.w_down)
        if self.identity:
            stream.add_rows_scaled(h, gates, s.experts, self.identity)
