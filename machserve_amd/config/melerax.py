"""Typed configuration of the Melerax decoder, read from config.json's own keys.

A Melerax model is a list of layers whose branches read the stream itself and are normed on their way out:
``x += ls1 * norm1(mixer(x))``, then ``x += ls2 * norm2(ff(x))``, the norms RMS norms whose weight is stored around zero
(``1 + w`` is applied) and ``ls`` a layer's scale per coordinate.  The mixer is ``parallel`` (chunked attention behind a
convolution on q, k and v beside a gated linear recurrence, each RMS-normed, half their sum), ``rglru`` (the recurrence
alone) or ``wkv`` (time mixing with a decay per key channel and token).  The feed-forward is dense and gated with
biases (the tanh form of GELU), or routed experts with an optional expert that every token uses (the exact GELU), or
absent.  The embedding adds a row of a second table chosen by the token and the one before it.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``embedding.bigram.{buckets, mul_prev, mul_cur}``, and
``layers``, a list of ``{"type", "mixer": {...}, "mlp": {"kind": "dense", "ff"} | {"kind": "moe", "expert": {"ff"},
"router": {"experts", "top"}, "shared": {"ff"}} | null}``.  Every size and constant comes from there; a missing or
ill-typed key is an error that names it.  The decay's bottleneck of a ``wkv`` layer is as wide as the checkpoint's
tensors are (``mixer.rank`` names it for the random-weights mode).  Tensor names: ``embed``, ``bigram``, ``head``,
``final.norm``, and per layer ``l<i>.norm1 | norm2 | ls1 | ls2``, ``l<i>.mix.*`` and ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .renanex import _get, _int, _num
from .specs import (ChunkedAttentionSpec, ConfigError, GatedMlpSpec, GatedRecurrenceSpec, HeadSpec, ModelSpec, NormSpec,
                    PairEmbeddingSpec, EmbeddingSpec, PostNormLayerSpec, RotarySpec, RoutedMlpSpec, SideBySideSpec, TimeMixSpec)

ARCHITECTURE = "Melerax"
# the configuration names no longest sequence: positions are 32-bit integers, and the pools bound a request
MAX_POSITIONS = 1 << 30
# the factor in the exponent of the recurrence's decay, which the design fixes
DECAY_FACTOR = 8.0
# the decay's bottleneck of a wkv layer in the random-weights mode when the configuration names none
DEFAULT_DECAY_RANK = 16


@dataclass(frozen=True)
class ChunkedAttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int                          # taps of the convolution on q, k and v; 0: none
    rot: Optional[Tuple[float, int]]   # (base, dims) or None
    softcap: float                     # 0: scores are not capped
    chunk: Optional[int]               # the mask's chunk size; None: plain causal


@dataclass(frozen=True)
class RecurrenceLayer:
    width: int
    blocks: int
    conv: int
    type: str = "rglru"


@dataclass(frozen=True)
class ParallelLayer:
    left: ChunkedAttentionLayer
    right: RecurrenceLayer
    type: str = "parallel"


@dataclass(frozen=True)
class TimeMixLayer:
    heads: int
    dim: int
    rank: Optional[int]
    type: str = "wkv"


@dataclass(frozen=True)
class DenseMlp:
    ff: int
    kind: str = "dense"


@dataclass(frozen=True)
class RoutedMlp:
    experts: int
    top: int
    ff: int
    shared: int  # 0: no expert that every token uses
    kind: str = "moe"


def _attention_of(m: dict, where: str) -> ChunkedAttentionLayer:
    heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv:
        raise ConfigError(f"config.json: '{where}heads' {heads} is not a multiple of '{where}kv_heads' {kv}")
    dim = _int(m, "dim", where)
    rot = None
    if m.get("rot") is not None:
        r = m["rot"]
        dims = _int(r, "dims", where + "rot.", 2)
        if dims % 2 or dims > dim:
            raise ConfigError(f"config.json: '{where}rot.dims' {dims} must be even and at most '{where}dim' {dim}")
        rot = (_num(r, "base", where + "rot."), dims)
    chunk = None
    if m.get("mask") is not None:
        chunk = _int(m["mask"], "size", where + "mask.")
    return ChunkedAttentionLayer(heads, kv, dim, _int(m, "vdim", where), _num(m, "scale", where),
                                 _int(m, "conv", where) if m.get("conv") is not None else 0, rot,
                                 _num(m, "softcap", where) if m.get("softcap") is not None else 0.0, chunk)


def _recurrence_of(m: dict, where: str) -> RecurrenceLayer:
    width, blocks = _int(m, "width", where), _int(m, "blocks", where)
    if width % blocks:
        raise ConfigError(f"config.json: '{where}width' {width} is not a multiple of '{where}blocks' {blocks}")
    return RecurrenceLayer(width, blocks, _int(m, "conv", where))


def _mixer_of(kind, m: dict, where: str):
    if kind == "parallel":
        return ParallelLayer(_attention_of(_get(m, "left", where), where + "left."), _recurrence_of(_get(m, "right", where), where + "right."))
    if kind == "rglru":
        return _recurrence_of(m, where)
    if kind == "wkv":
        return TimeMixLayer(_int(m, "heads", where), _int(m, "dim", where), _int(m, "rank", where) if m.get("rank") is not None else None)
    raise ConfigError(f"config.json: '{where[:-6]}type' {kind!r} is not a mixer of this architecture (parallel, rglru, wkv)")


def _mlp_of(mlp, where: str):
    if mlp is None:
        return None
    if not isinstance(mlp, dict):
        raise ConfigError(f"config.json: '{where[:-1]}' must be an object or null")
    kind = _get(mlp, "kind", where)
    if kind == "dense":
        return DenseMlp(_int(mlp, "ff", where))
    if kind == "moe":
        router = _get(mlp, "router", where)
        experts, top = _int(router, "experts", where + "router."), _int(router, "top", where + "router.")
        if top > experts:
            raise ConfigError(f"config.json: '{where}router.top' {top} exceeds '{where}router.experts' {experts}")
        shared = mlp.get("shared")
        return RoutedMlp(experts, top, _int(_get(mlp, "expert", where), "ff", where + "expert."),
                         _int(shared, "ff", where + "shared.") if shared is not None else 0)
    raise ConfigError(f"config.json: '{where}kind' {kind!r} is not a feed-forward of this architecture (dense, moe)")


@dataclass(frozen=True)
class MeleraxConfig:
    vocab: int
    width: int
    norm_eps: float
    bigram: Optional[Tuple[int, int, int]]  # (buckets, mul_prev, mul_cur) or None
    mixers: tuple
    mlps: tuple

    @classmethod
    def from_dict(cls, raw: dict) -> "MeleraxConfig":
        layers = _get(raw, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        mixers, mlps = [], []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json: 'layers[{i}]' must be an object")
            mixers.append(_mixer_of(_get(layer, "type", where), _get(layer, "mixer", where), where + "mixer."))
            mlps.append(_mlp_of(layer.get("mlp"), where + "mlp."))
        bigram = None
        bg = (raw.get("embedding") or {}).get("bigram")
        if bg is not None:
            w = "embedding.bigram."
            bigram = (_int(bg, "buckets", w), _int(bg, "mul_prev", w, 0), _int(bg, "mul_cur", w, 0))
        return cls(vocab=_int(raw, "vocab", ""), width=_int(raw, "width", ""), norm_eps=_num(_get(raw, "norm", ""), "eps", "norm."),
                   bigram=bigram, mixers=tuple(mixers), mlps=tuple(mlps))

    # ------------------------------------------------------------------ back to config.json
    @staticmethod
    def _attention_dict(m: ChunkedAttentionLayer) -> dict:
        d = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale}
        if m.conv:
            d["conv"] = m.conv
        if m.rot is not None:
            d["rot"] = {"base": m.rot[0], "dims": m.rot[1]}
        if m.softcap:
            d["softcap"] = m.softcap
        if m.chunk is not None:
            d["mask"] = {"size": m.chunk}
        return d

    def to_dict(self) -> dict:
        layers = []
        for m, mlp in zip(self.mixers, self.mlps):
            rec = lambda r: {"width": r.width, "blocks": r.blocks, "conv": r.conv}
            if isinstance(m, ParallelLayer):
                mixer = {"left": self._attention_dict(m.left), "right": rec(m.right)}
            elif isinstance(m, RecurrenceLayer):
                mixer = rec(m)
            else:
                mixer = {"heads": m.heads, "dim": m.dim}
                if m.rank is not None:
                    mixer["rank"] = m.rank
            if mlp is None:
                ff = None
            elif isinstance(mlp, DenseMlp):
                ff = {"kind": "dense", "ff": mlp.ff}
            else:
                ff = {"kind": "moe", "expert": {"ff": mlp.ff}, "router": {"experts": mlp.experts, "top": mlp.top}}
                if mlp.shared:
                    ff["shared"] = {"ff": mlp.shared}
            layers.append({"type": m.type, "mixer": mixer, "mlp": ff})
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.bigram is not None:
            out["embedding"] = {"bigram": {"buckets": self.bigram[0], "mul_prev": self.bigram[1], "mul_cur": self.bigram[2]}}
        return out

    # ------------------------------------------------------------------ the model as data
    def _attention_spec(self, m: ChunkedAttentionLayer, p: str) -> ChunkedAttentionSpec:
        rotary = None
        if m.rot is not None:
            rotary = RotarySpec("rotary", m.dim, m.rot[0], rotary_dim=m.rot[1], table_precision="float64", pairing="neighbours")
        names = {"q.weight": p + "q", "k.weight": p + "k", "v.weight": p + "v", "q.bias": p + "q.b", "k.bias": p + "k.b", "v.bias": p + "v.b",
                 "q.conv": p + "q.conv", "k.conv": p + "k.conv", "v.conv": p + "v.conv", "q.norm": p + "q.norm", "k.norm": p + "k.norm",
                 "o.weight": p + "o"}
        return ChunkedAttentionSpec("chunked_attention", self.width, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, rotary, conv_taps=m.conv,
                                    bias=True, qk_norm=True, norm_eps=self.norm_eps, softcap=m.softcap, chunk=m.chunk, tensors=names)

    def _recurrence_spec(self, m: RecurrenceLayer, p: str) -> GatedRecurrenceSpec:
        names = {"y.weight": p + "y", "y.bias": p + "y.b", "x.weight": p + "x", "x.bias": p + "x.b", "conv.weight": p + "conv",
                 "conv.bias": p + "conv.b", "ra.weight": p + "ra", "ra.bias": p + "ra.b", "ri.weight": p + "ri", "ri.bias": p + "ri.b",
                 "lam": p + "lam", "o.weight": p + "o"}
        return GatedRecurrenceSpec("gated_recurrence", self.width, m.width, m.blocks, m.conv, DECAY_FACTOR, names)

    def to_spec(self) -> ModelSpec:
        layers = []
        for i, (m, mlp) in enumerate(zip(self.mixers, self.mlps)):
            p = f"l{i}.mix."
            if isinstance(m, ParallelLayer):
                mixer = SideBySideSpec("side_by_side", self.width,
                                       (self._attention_spec(m.left, p + "left."), self._recurrence_spec(m.right, p + "right.")),
                                       self.norm_eps, {"norm.0": p + "left.out", "norm.1": p + "right.out"})
            elif isinstance(m, RecurrenceLayer):
                mixer = self._recurrence_spec(m, p)
            else:
                names = {f"mu.{s}": p + f"mu.{s}" for s in "rkvgw"}
                names.update({f"{s}.weight": p + s for s in ("r", "k", "v", "g", "w1", "w2", "o")})
                names.update({"w0": p + "w0", "u": p + "u", "norm": p + "norm"})
                mixer = TimeMixSpec("time_mix", self.width, m.heads, m.dim, m.rank, self.norm_eps, names)
            feed = post2 = None
            q = f"l{i}.mlp."
            if isinstance(mlp, DenseMlp):
                feed = GatedMlpSpec("gated_mlp", self.width, mlp.ff, "gelu_tanh", bias=True,
                                    tensors={"gate.weight": q + "gate", "up.weight": q + "up", "down.weight": q + "down",
                                             "gate.bias": q + "gate.b", "up.bias": q + "up.b", "down.bias": q + "down.b"})
            elif isinstance(mlp, RoutedMlp):
                names = {"router.weight": q + "router", "router.bias": q + "router.b", "shared.up": q + "shared.up", "shared.down": q + "shared.down"}
                for e in range(mlp.experts):
                    names[f"e{e}.up"], names[f"e{e}.down"] = q + f"e{e}.up", q + f"e{e}.down"
                feed = RoutedMlpSpec("routed_mlp", self.width, mlp.experts, mlp.top, mlp.ff, "gelu", mlp.shared, True, names)
            if feed is not None:
                post2 = self._norm(f"l{i}.norm2", f"l{i}.ls2")
            layers.append(PostNormLayerSpec("postnorm", mixer, feed, self._norm(f"l{i}.norm1", f"l{i}.ls1"), post2))
        if self.bigram is not None:
            embedding = PairEmbeddingSpec(self.vocab, self.width, self.bigram[0], self.bigram[1], self.bigram[2],
                                          {"weight": "embed", "pairs": "bigram"})
        else:
            embedding = EmbeddingSpec(self.vocab, self.width, {"weight": "embed"})
        spec = ModelSpec(architecture=ARCHITECTURE, embedding=embedding, layers=tuple(layers), order=tuple(range(len(layers))),
                         final_norm=self._norm("final.norm"), head=HeadSpec(self.vocab, self.width, False, {"weight": "head"}),
                         max_positions=MAX_POSITIONS)
        spec.validate()
        return spec

    def _norm(self, name: str, scale: Optional[str] = None) -> NormSpec:
        tensors = {"weight": name}
        if scale is not None:
            tensors["scale"] = scale
        return NormSpec("rmsnorm", self.width, self.norm_eps, tensors, offset=1.0, scaled=scale is not None)

    # ------------------------------------------------------------------ random weights
    def random_tensor_plan(self):
        """(name, shape, law) of every tensor of a random checkpoint; the laws are those of ``weights.random_init``."""
        w = self.width
        plan = [("embed", (self.vocab, w), "matrix")]
        if self.bigram is not None:
            plan.append(("bigram", (self.bigram[0] + 1, w), "matrix"))

        def attention(m, p):
            nq, nk, nv = m.heads * m.dim, m.kv_heads * m.dim, m.kv_heads * m.vdim
            out = []
            for s, n in (("q", nq), ("k", nk), ("v", nv)):
                out += [(p + s, (n, w), "matrix"), (p + s + ".b", (n,), "bias")]
            out += [(p + "q.norm", (nq,), "norm"), (p + "k.norm", (nk,), "norm")]
            if m.conv:
                out += [(p + f"{s}.conv", (n, m.conv), "filter") for s, n in (("q", nq), ("k", nk), ("v", nv))]
            return out + [(p + "o", (w, m.heads * m.vdim), "matrix")]

        def recurrence(m, p):
            bw = m.width // m.blocks
            return [(p + "y", (m.width, w), "matrix"), (p + "y.b", (m.width,), "bias"), (p + "x", (m.width, w), "matrix"),
                    (p + "x.b", (m.width,), "bias"), (p + "conv", (m.width, m.conv), "filter"), (p + "conv.b", (m.width,), "bias"),
                    (p + "ra", (m.blocks, bw, bw), "filter"), (p + "ra.b", (m.blocks, bw), "bias"), (p + "ri", (m.blocks, bw, bw), "filter"),
                    (p + "ri.b", (m.blocks, bw), "bias"), (p + "lam", (m.width,), "filter"), (p + "o", (w, m.width), "matrix")]

        for i, (m, mlp) in enumerate(zip(self.mixers, self.mlps)):
            plan += [(f"l{i}.norm1", (w,), "bias")]
            if mlp is not None:
                plan += [(f"l{i}.norm2", (w,), "bias")]
            p = f"l{i}.mix."
            if isinstance(m, ParallelLayer):
                plan += attention(m.left, p + "left.") + recurrence(m.right, p + "right.")
                plan += [(p + "left.out", (w,), "norm"), (p + "right.out", (w,), "norm")]
            elif isinstance(m, RecurrenceLayer):
                plan += recurrence(m, p)
            else:
                n, rank = m.heads * m.dim, m.rank or DEFAULT_DECAY_RANK
                plan += [(p + f"mu.{s}", (w,), "blend") for s in "rkvgw"]
                plan += [(p + s, (n, w), "matrix") for s in ("r", "k", "v", "g")]
                plan += [(p + "w1", (rank, w), "matrix"), (p + "w2", (n, rank), "filter"), (p + "w0", (n,), "filter"),
                         (p + "u", (m.heads, m.dim), "filter"), (p + "norm", (n,), "norm"), (p + "o", (w, n), "matrix")]
            q = f"l{i}.mlp."
            if isinstance(mlp, DenseMlp):
                for s, shape in (("gate", (mlp.ff, w)), ("up", (mlp.ff, w)), ("down", (w, mlp.ff))):
                    plan += [(q + s, shape, "matrix"), (q + s + ".b", (shape[0],), "bias")]
            elif isinstance(mlp, RoutedMlp):
                for e in range(mlp.experts):
                    plan += [(q + f"e{e}.up", (mlp.ff, w), "matrix"), (q + f"e{e}.down", (w, mlp.ff), "matrix")]
                plan += [(q + "router", (mlp.experts, w), "filter"), (q + "router.b", (mlp.experts,), "bias")]
                if mlp.shared:
                    plan += [(q + "shared.up", (mlp.shared, w), "matrix"), (q + "shared.down", (w, mlp.shared), "matrix")]
            plan += [(f"l{i}.ls1", (w,), "norm")]
            if mlp is not None:
                plan += [(f"l{i}.ls2", (w,), "norm")]
        plan += [("final.norm", (w,), "bias"), ("head", (self.vocab, w), "matrix")]
        return plan
