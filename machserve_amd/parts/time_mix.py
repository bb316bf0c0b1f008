"""Time mixing with a decay per key channel that depends on the token, as a mixer with state of fixed size.

Per step: each of r, k, v, the gate and the decay reads its own mix of a token's input with the one before it
(``x + (x' - x) mu``, worked out from the 32-bit stream; the previous token's input is state); four products for r, k, v
and the gate; the decay's bottleneck (product, tanh, product, left as 32-bit sums); one kernel that walks a request's
tokens per head with the ``[dim, dim]`` state in registers (``o = (S + diag(u) k v^T)^T r``, ``S <- diag(w) S + k v^T`` with
``w = exp(-exp(z + w0))``; long portions in segments side by side, see ``ops.wkv``), divides a head's output by its root mean square, and applies the weight and the gate's SiLU;
the output projection.  The decay, the state and the unit norm are 32-bit in every build.
"""
from __future__ import annotations

import torch

from .base import Mixer, StateRequest, TensorDecl, require_kernel_sizes
from .registry import register_mixer


@register_mixer("time_mix")
class TimeMix(Mixer):
    graph_safe = True   # reads the requests' rows and slots from device memory only
    reads_stream = True  # a block that can gives it the 32-bit rows: the mixes are worked out from them

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        self.n = s.heads * s.head_dim
        require_kernel_sizes(rt, "time_mix", [("hidden size", s.hidden), ("heads x head size", self.n)])
        limits = getattr(rt.ops, "linrec_limits", None)
        if limits is not None and s.head_dim > limits()["wkv_dim"]:
            raise ValueError(f"time_mix: heads of {s.head_dim}; the kernel takes up to {limits()['wkv_dim']}")
        self.rank = s.decay_rank
        self.state = None

    def tensor_decls(self):
        s, n = self.spec, self.n
        decls = [TensorDecl(f"mu.{m}", (s.hidden,), "vector") for m in "rkvgw"]
        decls += [TensorDecl(f"{m}.weight", (n, s.hidden)) for m in "rkvg"]
        rank = self.rank
        decls += [TensorDecl("w1.weight", (rank, s.hidden) if rank else None), TensorDecl("w2.weight", (n, rank) if rank else None),
                  TensorDecl("w0", (n,), "vector"), TensorDecl("u", (s.heads, s.head_dim), "vector"),
                  TensorDecl("norm", (n,), "vector"), TensorDecl("o.weight", (s.hidden, n))]
        return decls

    def load(self, t):
        self.mu = torch.stack([t[f"mu.{m}"] for m in "rkvgw"]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (t[f"{m}.weight"] for m in "rkvg")
        w1, w2 = t["w1.weight"], t["w2.weight"]
        if w1.shape[0] != w2.shape[1] or w1.shape[1] != self.spec.hidden or w2.shape[0] != self.n:
            raise ValueError(f"time_mix: the decay's bottleneck {tuple(w1.shape)} and {tuple(w2.shape)} does not fit")
        fill = -w1.shape[0] % 8  # the products sum over multiples of 8: rows of zeros, columns of zeros
        if fill:
            w1 = torch.cat([w1, w1.new_zeros((fill, w1.shape[1]))], dim=0)
            w2 = torch.cat([w2, w2.new_zeros((w2.shape[0], fill))], dim=1)
        self.w_1, self.w_2 = w1.contiguous(), w2.contiguous()
        self.w0, self.u, self.norm_w, self.w_o = t["w0"], t["u"].reshape(-1).contiguous(), t["norm"], t["o.weight"]

    def cache_request(self):
        s = self.spec
        return StateRequest({"prev": (s.hidden,), "wkv": (s.heads, s.head_dim, s.head_dim)})

    def bind_cache(self, binding):
        self.state = binding.tensors

    def forward(self, x, stream, ctx):
        s, ops = self.spec, self.rt.ops
        if x.dtype != torch.float32:  # a block that norms its input first: the mixes are of the normed rows
            x = x.float()
        mix = ops.shift_mix(x, self.state["prev"], self.mu, ctx.seq_q_start, ctx.seq_q_len, ctx.seq_slot)
        r, k, v, g = (ops.linear(mix[i], w) for i, w in enumerate((self.w_r, self.w_k, self.w_v, self.w_g)))
        z = ops.linear(ops.tanh_rows(ops.linear(mix[4], self.w_1, None, out_f32=True)), self.w_2, None, out_f32=True)
        out = ops.wkv(r, k, v, g, z, self.w0, self.u, self.norm_w, s.norm_eps, self.state["wkv"], ctx.seq_q_start, ctx.seq_q_len,
                      ctx.seq_slot, s.heads, s.head_dim)
        stream.add_linear(out, self.w_o)
