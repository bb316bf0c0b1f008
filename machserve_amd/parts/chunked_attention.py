"""Grouped-query attention with values of a width of their own, behind a short convolution on q, k and v, whose rows
see the keys of their own chunk of positions only and whose scores are capped by a tanh, over the paged cache.

Per step: q, k and v as one product that leaves 32-bit sums; a causal convolution over time on every channel of the
three (its last ``taps - 1`` inputs are state of fixed size, the bias of the projection is added before it); one kernel
that finishes a row (an RMS norm over the whole of q and one over the whole of k, the rotation of the first numbers of
every head, the write of k and v into their pages); the framework's paged attention kernels with the chunk and the
cap as parameters; the output projection.  Keys and values share pools whose heads are as wide as the wider of the
two, filled with zeros up to the attention tile's size.  The convolution, both norms, the angles and the scores are
32-bit in every build.
"""
from __future__ import annotations

import torch

from .base import Mixer, PagedKVRequest, StateRequest, TensorDecl, attention_head_size, require_kernel_sizes
from .registry import POSITION_ENCODINGS, register_mixer


@register_mixer("chunked_attention")
class ChunkedAttention(Mixer):
    graph_safe = True  # reads positions, rows, slots and addresses from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.heads % s.kv_heads:
            raise ValueError(f"chunked_attention: {s.heads} heads are not a multiple of {s.kv_heads} key/value heads")
        self.nq, self.nk, self.nv = s.heads * s.head_dim, s.kv_heads * s.head_dim, s.kv_heads * s.v_head_dim
        self.n = self.nq + self.nk + self.nv
        self.taps = s.conv_taps or 0
        self.hd = attention_head_size(rt, max(s.head_dim, s.v_head_dim))  # of the pools and of the attention kernels
        require_kernel_sizes(rt, "chunked_attention", [("hidden size", s.hidden)], self.hd)
        self.position = POSITION_ENCODINGS.build(s.position, rt) if s.position is not None else None
        self.rot, self.neighbours = 0, False
        if self.position is not None:
            if self.position.rotary_inv_freq() is None or self.position.score_factor() != 1.0:
                raise ValueError("chunked_attention: the position encoding must be a plain rotation")
            self.rot = self.position.rotary_dim
            self.neighbours = getattr(s.position, "pairing", "halves") == "neighbours"
        limits = getattr(rt.ops, "conv_rows_limits", None)
        if limits is not None and self.n + self.rot > limits()["row"]:
            raise ValueError(f"chunked_attention: a row of q, k and v of {self.n} numbers; the kernels take up to {limits()['row'] - self.rot}")
        limits = getattr(rt.ops, "linrec_limits", None)
        if limits is not None and self.taps > limits()["taps"]:
            raise ValueError(f"chunked_attention: {self.taps} taps; the convolution takes up to {limits()['taps']}")
        self.group = self.kpool = self.vpool = self.state = None

    def sub_parts(self):
        return [self.position] if self.position is not None else []

    def tensor_decls(self):
        s = self.spec
        decls = []
        for name, n in (("q", self.nq), ("k", self.nk), ("v", self.nv)):
            decls.append(TensorDecl(f"{name}.weight", (n, s.hidden)))
            if s.bias:
                decls.append(TensorDecl(f"{name}.bias", (n,), "vector"))
            if self.taps:
                decls.append(TensorDecl(f"{name}.conv", (n, self.taps), "vector"))
        if s.qk_norm:
            decls += [TensorDecl("q.norm", (self.nq,), "vector"), TensorDecl("k.norm", (self.nk,), "vector")]
        decls.append(TensorDecl("o.weight", (s.hidden, s.heads * s.v_head_dim)))
        return decls

    def load(self, t):
        s = self.spec
        names = ("q", "k", "v")
        self.w_qkv = torch.cat([t[n + ".weight"] for n in names], dim=0).contiguous()
        self.b_qkv = torch.cat([t[n + ".bias"] for n in names]).contiguous() if s.bias else None
        self.conv_w = torch.cat([t[n + ".conv"] for n in names], dim=0).contiguous() if self.taps else None
        self.q_norm, self.k_norm = (t["q.norm"], t["k.norm"]) if s.qk_norm else (None, None)
        w_o = t["o.weight"]
        if self.hd != s.v_head_dim:  # the attention's output has the pools' head size: columns of zeros in between
            w_o = torch.nn.functional.pad(w_o.view(s.hidden, s.heads, s.v_head_dim), (0, self.hd - s.v_head_dim)).reshape(s.hidden, -1)
        self.w_o = w_o.contiguous()

    def cache_request(self):
        pages = PagedKVRequest(self.spec.kv_heads, self.hd, self.spec.window)
        if self.taps < 2:
            return pages
        return [pages, StateRequest({"conv": (self.taps - 1, self.n)})]

    def bind_cache(self, binding):
        pages = binding[0] if self.taps > 1 else binding
        self.group, self.kpool, self.vpool = pages.group, pages.kpool, pages.vpool
        self.state = binding[1].tensors["conv"] if self.taps > 1 else None

    def attention_rows_per_token(self):
        return self.spec.heads // self.spec.kv_heads

    def attention_rows_per_block(self):
        return self.rt.ops.attention_rows_per_block(self.hd)

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        view = ctx.groups[self.group]
        g = self.attention_rows_per_token()
        if self.taps:
            rows = ops.conv_sums(ops.linear_split(h, self.w_qkv), 0, self.n, self.b_qkv, self.conv_w, None, self.state,
                                 ctx.seq_q_start, ctx.seq_q_len, ctx.seq_slot)
        else:
            rows = ops.linear(h, self.w_qkv, self.b_qkv, out_f32=True)
        inv_freq = self.position.rotary_inv_freq() if self.position is not None else None
        q = ops.finish_rows(rows, self.q_norm, self.k_norm, s.norm_eps, ctx.position_axis(0), inv_freq, self.rot, self.neighbours,
                            view.slot_map, self.kpool, self.vpool, s.heads, s.kv_heads, s.head_dim, s.v_head_dim, view.page_size)
        chunk, cap = int(s.chunk or 0), float(s.softcap or 0.0)
        if ctx.decode_only and g <= ops.DECODE_MAX_GROUP:
            o = ops.decode_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_pos0, s.heads, s.kv_heads, self.hd,
                                     view.page_size, s.window, float(s.scale), chunk=chunk, softcap=cap)
        else:
            o = ops.paged_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_q_start, ctx.seq_q_len, ctx.seq_pos0,
                                    ctx.attention_work[g], s.heads, s.kv_heads, self.hd, view.page_size, s.window, float(s.scale),
                                    chunk=chunk, softcap=cap)
        stream.add_linear(o, self.w_o)
