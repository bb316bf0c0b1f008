"""Several mixers side by side: all read the same input, each one's output is RMS-normed over the model's width with a
weight of its own, and the result is their mean.  The branches are mixers of any registered kind; each keeps the cache
or state it asks for, and what the branches ask for is handed on as one flat list.  A branch must end in a product
(``add_linear``): the norms read its 32-bit sums."""
from __future__ import annotations

from .base import Mixer, TensorDecl
from .registry import MIXERS, register_mixer


class _Last:
    """What a branch writes to in the stream's place: the operands of its last product."""

    def __init__(self):
        self.product = None

    def add_linear(self, a, w, bias=None):
        if bias is not None:
            raise ValueError("side_by_side: a branch whose last product has a bias")
        self.product = (a, w)

    def add(self, y):
        raise ValueError("side_by_side: a branch must end in a product")


@register_mixer("side_by_side")
class SideBySide(Mixer):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        if len(spec.branches) < 2:
            raise ValueError("side_by_side: fewer than two branches")
        self.branches = [MIXERS.build(b, rt) for b in spec.branches]
        if any(getattr(b, "reads_stream", False) for b in self.branches):
            raise ValueError("side_by_side: a branch that reads the 32-bit stream itself")
        self.norms = None

    @property
    def graph_safe(self):
        return all(getattr(b, "graph_safe", False) for b in self.branches)

    def sub_parts(self):
        out = []
        for b in self.branches:
            out.append(b)
            out.extend(getattr(b, "sub_parts", lambda: [])())
        return out

    def tensor_decls(self):
        return [TensorDecl(f"norm.{i}", (self.spec.hidden,), "vector") for i in range(len(self.branches))]

    def load(self, t):
        self.norms = [t[f"norm.{i}"] for i in range(len(self.branches))]

    # ------------------------------------------------------------------ caches: every branch's own, as one flat list
    def _requests(self):
        out = []
        for b in self.branches:
            r = b.cache_request()
            out.append(list(r) if isinstance(r, (list, tuple)) else [r])
        return out

    def cache_request(self):
        return [r for rs in self._requests() for r in rs]

    def bind_cache(self, binding):
        at = 0
        for b, rs in zip(self.branches, self._requests()):
            several = isinstance(b.cache_request(), (list, tuple))
            mine = binding[at:at + len(rs)]
            at += len(rs)
            if several:
                b.bind_cache(mine)
            elif mine[0] is not None:
                b.bind_cache(mine[0])

    def _one(self, what):
        values = {v for b in self.branches for v in [getattr(b, what)()] if v}
        if len(values) > 1:
            raise ValueError(f"side_by_side: branches with different {what}: {sorted(values)}")
        return next(iter(values)) if values else None

    def attention_rows_per_token(self):
        return self._one("attention_rows_per_token")

    def attention_rows_per_block(self):
        return self._one("attention_rows_per_block")

    def forward(self, h, stream, ctx):
        lasts = []
        for b in self.branches:
            last = _Last()
            b.forward(h, last, ctx)
            lasts.append(last.product)
        stream.add_normed_mean(list(zip(lasts, self.norms)), self.spec.norm_eps)
