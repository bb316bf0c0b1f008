"""Attention through a latent over the paged cache.

The cache keeps per token the normed latent ``c`` and one rotated key part, as ONE key/value head of width
``kv_rank + rot_dim`` (filled with zeros up to the attention tile's size); every query head is in that head's group.
Per step: the down projections of queries and (unless the layer reads another layer's cache) latent and key part as
one product that leaves 32-bit sums; one kernel that finishes a row (two RMS norms with weights, rotation of the key
part, write into the page); the queries' up projection; the heads' plain parts carried into the latent's space by a
product per head with ``W_uk^T``, the rotated parts written behind them; the framework's paged attention kernels with
a sink per head; the result carried out of the latent's space by a product per head with ``W_uv``; the output
projection.  A head's keys and values are never materialised.  Without a bottleneck of the queries (``q_rank`` 0) the
heads' queries are one projection of the input; the rotated parts turn neighbouring pairs or half against half, as the
rotation's spec says; a window and a gate per head (the sigmoid of one more projection of the input, applied to the
attention's output in the latent's space, which the per-head product carries out unchanged) are the attention kernels'
own parameters.
"""
from __future__ import annotations

import torch

from .base import Mixer, PagedKVRequest, SharedKVRequest, TensorDecl, attention_head_size, require_kernel_sizes
from .registry import POSITION_ENCODINGS, register_mixer


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True  # reads positions and addresses from device memory only

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        s = spec
        if s.rot_dim % 2:
            raise ValueError(f"latent_attention: a rotated part of {s.rot_dim} numbers cannot be rotated in pairs")
        self.position = POSITION_ENCODINGS.build(s.position, rt) if s.position is not None and s.rot_dim else None
        if s.rot_dim and self.position is None:
            raise ValueError("latent_attention: a rotated part needs a rotation")
        self.halves = self.position is not None and getattr(s.position, "pairing", "neighbours") == "halves"
        self.window = getattr(s, "window", None)
        self.head_gate = bool(getattr(s, "head_gate", False))
        self.hd = attention_head_size(rt, s.kv_rank + s.rot_dim)  # of the pools and of the attention kernels
        self.rank8 = -(-s.kv_rank // 8) * 8
        # the value size as the output projection sums over it: filled up where heads x value size is no multiple of 8
        self.vd = s.v_head_dim if (s.heads * s.v_head_dim) % 8 == 0 else -(-s.v_head_dim // 8) * 8
        require_kernel_sizes(rt, "latent_attention", [("hidden size", s.hidden)], self.hd)
        limits = getattr(rt.ops, "latent_limits", None)
        if s.q_rank == 0 and s.kv_source is not None:
            raise ValueError("latent_attention: queries without a bottleneck beside another layer's cache are not built")
        if limits is not None and s.q_rank + s.kv_rank + s.rot_dim > limits()["row"]:
            raise ValueError(f"latent_attention: a row of {s.q_rank + s.kv_rank + s.rot_dim} numbers exceeds the kernels' {limits()['row']}")
        self.writes_cache = s.kv_source is None
        self.group = self.kpool = self.vpool = None

    def sub_parts(self):
        return [self.position] if self.position is not None else []

    def tensor_decls(self):
        s = self.spec
        if s.q_rank:
            decls = [TensorDecl("dq.weight", (s.q_rank, s.hidden)), TensorDecl("dq.norm", (s.q_rank,), "vector"),
                     TensorDecl("uq.weight", (s.heads * (s.head_dim + s.rot_dim), s.q_rank))]
        else:
            decls = [TensorDecl("q.weight", (s.heads * (s.head_dim + s.rot_dim), s.hidden))]
        if self.head_gate:
            decls.append(TensorDecl("g.weight", (s.heads, s.hidden)))
        decls += [TensorDecl("uk.weight", (s.heads * s.head_dim, s.kv_rank)), TensorDecl("uv.weight", (s.heads * s.v_head_dim, s.kv_rank)),
                 TensorDecl("o.weight", (s.hidden, s.heads * s.v_head_dim))]
        if self.writes_cache:
            decls += [TensorDecl("dkv.weight", (s.kv_rank + s.rot_dim, s.hidden)), TensorDecl("dkv.norm", (s.kv_rank,), "vector")]
        if s.sink:
            decls.append(TensorDecl("sink", (s.heads,), "vector"))
        return decls

    def load(self, t):
        s = self.spec
        pad = torch.nn.functional.pad
        if s.q_rank:
            self.w_down = torch.cat([t["dq.weight"], t["dkv.weight"]], dim=0).contiguous() if self.writes_cache else t["dq.weight"]
            self.w_uq = pad(t["uq.weight"], (0, -s.q_rank % 8)).contiguous()  # the query latent comes filled up to a multiple of 8
        else:
            self.w_down, self.w_q = t.get("dkv.weight"), t["q.weight"]
        self.q_norm, self.c_norm = t.get("dq.norm"), t.get("dkv.norm")
        self.w_g = t.get("g.weight")
        d8 = -(-s.head_dim // 8) * 8
        # W_uk^T per head, [heads, kv_rank, head_dim (up to a multiple of 8)]: carries a plain query into the latent's space
        self.w_ukT = pad(t["uk.weight"].view(s.heads, s.head_dim, s.kv_rank).transpose(1, 2), (0, d8 - s.head_dim)).contiguous()
        # W_uv per head over the attention's head size, [heads, v_head_dim, hd]: zeros beside the latent's columns
        self.w_uv = pad(t["uv.weight"].view(s.heads, s.v_head_dim, s.kv_rank), (0, self.hd - s.kv_rank)).contiguous()
        self.w_o = pad(t["o.weight"].view(s.hidden, s.heads, s.v_head_dim), (0, self.vd - s.v_head_dim)).reshape(s.hidden, -1).contiguous()
        self.sink = t.get("sink")

    def cache_request(self):
        if not self.writes_cache:
            return SharedKVRequest(self.spec.kv_source)
        return PagedKVRequest(1, self.hd, self.window)

    def bind_cache(self, binding):
        self.group, self.kpool, self.vpool = binding.group, binding.kpool, binding.vpool

    def attention_rows_per_token(self):
        return self.spec.heads

    def attention_rows_per_block(self):
        return self.rt.ops.attention_rows_per_block(self.hd)

    def forward(self, h, stream, ctx):
        s, ops = self.spec, self.rt.ops
        view = ctx.groups[self.group]
        pos = ctx.position_axis(0)
        inv_freq = self.position.inv_freq if self.position is not None else None
        factor = float(self.position.factor) if self.position is not None else 1.0
        pairing = {"halves": True} if self.halves else {}
        cq = None
        if self.writes_cache:
            cq = ops.latent_rows(ops.linear_split(h, self.w_down), self.q_norm, self.c_norm, s.norm_eps, pos, inv_freq, factor, view.slot_map,
                                 self.kpool, self.vpool, s.q_rank, s.kv_rank, s.rot_dim, view.page_size, **pairing)
        elif s.q_rank:
            cq = ops.latent_rows(ops.linear_split(h, self.w_down), self.q_norm, None, s.norm_eps, pos, None, 1.0, None, None, None, s.q_rank,
                                 s.kv_rank, s.rot_dim, view.page_size)
        q = ops.linear(cq, self.w_uq, None, out_f32=True) if s.q_rank else ops.linear(h, self.w_q, None, out_f32=True)
        plain, att = ops.latent_query(q, pos, inv_freq, factor, s.heads, s.head_dim, s.rot_dim, s.kv_rank, self.hd, **pairing)
        ops.heads_linear(plain, self.w_ukT, att)
        gate = ops.sigmoid_rows(ops.linear(h, self.w_g, None, out_f32=True)) if self.head_gate else None
        if ctx.decode_only and s.heads <= ops.DECODE_MAX_GROUP:
            o = ops.decode_attention(att.view(att.shape[0], -1), self.kpool, self.vpool, view.block_table, ctx.seq_pos0, s.heads, 1, self.hd,
                                     view.page_size, self.window, float(s.scale), self.sink, gate)
        else:
            o = ops.paged_attention(att.view(att.shape[0], -1), self.kpool, self.vpool, view.block_table, ctx.seq_q_start, ctx.seq_q_len,
                                    ctx.seq_pos0, ctx.attention_work[s.heads], s.heads, 1, self.hd, view.page_size, self.window, float(s.scale),
                                    sinks=self.sink, out_gate=gate)
        y = o.new_zeros((o.shape[0], s.heads, self.vd)) if self.vd != s.v_head_dim else None
        y = ops.heads_linear(o.view(o.shape[0], s.heads, self.hd), self.w_uv, y)
        stream.add_linear(y.view(y.shape[0], -1), self.w_o)
