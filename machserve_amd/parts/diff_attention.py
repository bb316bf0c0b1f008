"""Differential grouped-query attention behind a short convolution on q, k and v, over the paged cache.

Every head has two softmax maps over the same values, each with queries and keys of its own; the head's result is the
first map's minus ``lambda`` times the second's, divided by its root mean square and multiplied by ``1 - diff``; the heads
side by side are multiplied by ``sigmoid(W_g h)`` and projected.

On the framework's paged attention kernels a map is a head: the cache holds ``2 x kv_heads`` key heads and the values
once per map (a value head's rows of ``W_v`` are used twice), and the queries' maps are ordered so that the maps of a
key/value head's group lie side by side, ``(group, map, head in the group)``, which is a permutation of ``W_q``'s rows made
when the weights are loaded.  Per step: q, k and v as one product that leaves 32-bit sums; the convolution over time on
every channel (its last ``taps - 1`` inputs are state of fixed size; the projection's bias is added before it); one
kernel that rotates every map of q and k and writes k and v into their pages; attention; one kernel that combines a
head's two maps, norms, scales and gates; the output projection with its bias.  A layer that reads another layer's keys
and values has only its queries to project, convolve and rotate.
"""
from __future__ import annotations

import math

import torch

from .base import Mixer, PagedKVRequest, SharedKVRequest, StateRequest, TensorDecl, attention_head_size, require_kernel_sizes
from .registry import POSITION_ENCODINGS, register_mixer


@register_mixer("diff_attention")
class DiffAttention(Mixer):
    graph_safe = True  # reads positions, rows, slots and addresses from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.heads % s.kv_heads:
            raise ValueError(f"diff_attention: {s.heads} heads are not a multiple of {s.kv_heads} key/value heads")
        self.writes_cache = s.kv_source is None
        self.maps, self.kv_maps = 2 * s.heads, 2 * s.kv_heads
        self.nq = self.maps * s.head_dim
        self.nk = self.kv_maps * s.head_dim if self.writes_cache else 0
        self.nv = self.kv_maps * s.v_head_dim if self.writes_cache else 0
        self.n = self.nq + self.nk + self.nv
        self.taps = s.conv_taps or 0
        self.hd = attention_head_size(rt, max(s.head_dim, s.v_head_dim))  # of the pools and of the attention kernels
        self.out_cols = -(-s.heads * s.v_head_dim // 8) * 8  # the output projection sums over a multiple of 8
        require_kernel_sizes(rt, "diff_attention", [("hidden size", s.hidden)], self.hd)
        self.position = POSITION_ENCODINGS.build(s.position, rt) if s.position is not None else None
        self.rot, self.neighbours = 0, False
        if self.position is not None:
            if self.position.rotary_inv_freq() is None or self.position.score_factor() != 1.0:
                raise ValueError("diff_attention: the position encoding must be a plain rotation")
            self.rot = self.position.rotary_dim
            self.neighbours = getattr(s.position, "pairing", "halves") == "neighbours"
        limits = getattr(rt.ops, "conv_rows_limits", None)
        if limits is not None and self.n + self.rot > limits()["row"]:
            raise ValueError(f"diff_attention: a row of q, k and v of {self.n} numbers; the kernels take up to {limits()['row'] - self.rot}")
        limits = getattr(rt.ops, "linrec_limits", None)
        if limits is not None and self.taps > limits()["taps"]:
            raise ValueError(f"diff_attention: {self.taps} taps; the convolution takes up to {limits()['taps']}")
        self.group = self.kpool = self.vpool = self.state = None

    def sub_parts(self):
        return [self.position] if self.position is not None else []

    def _own(self):
        s = self.spec
        own = [("q", 2 * s.heads * s.head_dim)]
        if self.writes_cache:
            own += [("k", 2 * s.kv_heads * s.head_dim), ("v", s.kv_heads * s.v_head_dim)]
        return own

    def tensor_decls(self):
        s = self.spec
        decls = []
        for name, n in self._own():
            decls.append(TensorDecl(f"{name}.weight", (n, s.hidden)))
            if s.bias:
                decls.append(TensorDecl(f"{name}.bias", (n,), "vector"))
            if self.taps:
                decls.append(TensorDecl(f"{name}.conv", (n, self.taps), "vector"))
        decls += [TensorDecl(n, (s.head_dim,), "vector") for n in ("lq1", "lk1", "lq2", "lk2")]
        decls += [TensorDecl("g.weight", (s.heads * s.v_head_dim, s.hidden)), TensorDecl("o.weight", (s.hidden, s.heads * s.v_head_dim))]
        if s.bias:
            decls.append(TensorDecl("o.bias", (s.hidden,), "vector"))
        return decls

    def load(self, t):
        s = self.spec
        dev = t["q.weight"].device
        per_group, d, dv = s.heads // s.kv_heads, s.head_dim, s.v_head_dim
        # rows of q in the order (key/value head, map, head of the group): a map's queries then lie in the group of the
        # key head of that map
        head = torch.arange(s.heads, device=dev).view(s.kv_heads, 1, per_group)
        maps = (head * 2 + torch.arange(2, device=dev).view(1, 2, 1)).reshape(-1)
        rows = {"q": (maps[:, None] * d + torch.arange(d, device=dev)[None, :]).reshape(-1)}
        if self.writes_cache:
            rows["k"] = torch.arange(self.nk, device=dev)
            # a value head once per map
            rows["v"] = (torch.arange(s.kv_heads, device=dev).repeat_interleave(2)[:, None] * dv + torch.arange(dv, device=dev)[None, :]).reshape(-1)
        names = [n for n, _ in self._own()]
        self.w_qkv = torch.cat([t[n + ".weight"][rows[n]] for n in names], dim=0).contiguous()
        self.b_qkv = torch.cat([t[n + ".bias"][rows[n]] for n in names]).contiguous() if s.bias else None
        self.conv_w = torch.cat([t[n + ".conv"][rows[n]] for n in names], dim=0).contiguous() if self.taps else None
        f = lambda n: t[n].double()
        self.lam = float(torch.exp((f("lq1") * f("lk1")).sum()) - torch.exp((f("lq2") * f("lk2")).sum())) + float(s.diff)
        self.w_g = t["g.weight"]
        self.w_o = torch.nn.functional.pad(t["o.weight"], (0, self.out_cols - s.heads * dv)).contiguous()
        self.b_o = t.get("o.bias")

    def cache_request(self):
        pages = PagedKVRequest(self.kv_maps, self.hd) if self.writes_cache else SharedKVRequest(self.spec.kv_source)
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
        q = ops.finish_rows(rows, None, None, s.norm_eps, ctx.position_axis(0), inv_freq, self.rot, self.neighbours, view.slot_map,
                            self.kpool, self.vpool, self.maps, self.kv_maps, s.head_dim, s.v_head_dim, view.page_size,
                            queries_only=not self.writes_cache)
        if ctx.decode_only and g <= ops.DECODE_MAX_GROUP:
            o = ops.decode_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_pos0, self.maps, self.kv_maps, self.hd,
                                     view.page_size, None, float(s.scale))
        else:
            o = ops.paged_attention(q, self.kpool, self.vpool, view.block_table, ctx.seq_q_start, ctx.seq_q_len, ctx.seq_pos0,
                                    ctx.attention_work[g], self.maps, self.kv_maps, self.hd, view.page_size, None, float(s.scale))
        gate = ops.linear(h, self.w_g, None, out_f32=True)
        y = ops.diff_combine(o, gate, self.lam, s.norm_eps, 1.0 - float(s.diff), s.heads, s.kv_heads, self.hd, s.v_head_dim, self.out_cols)
        stream.add_linear(y, self.w_o, self.b_o)
