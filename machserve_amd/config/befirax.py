"""Typed configuration of the Befirax decoder, read from config.json's own keys.

A Befirax model is a list of pre-norm layers, ``x += mixer(norm1(x))``, then ``x += ff(norm2(x))``, over one residual
stream or, with ``streams``, over several: a branch then reads ``sum_s in[s] x_s`` through its norm and is written back as
``x_t = sum_s mix[s, t] x_s + out[t] y``; the streams all start as the embedding and are summed before the last norm.  The
mixer is ``attention`` (differential grouped-query attention behind a short convolution on q, k and v, rotation of
neighbouring pairs on part of every map, an output gate; ``kv_from`` names an earlier layer whose keys and values it
reads), ``latent_attention`` (one normed latent and one rotated key part a token for all heads, rotation of half against
half, a sliding window, a gate per head) or ``mamba2`` (state-space duality: a decay and a step size per head and token, B
and C per group, a gated norm in groups).  The feed-forward is a mixture of gated experts without biases, chosen by the
softmax of the router plus a correction, among them experts without tensors that return their input; or absent.  The
head is the embedding table.

Keys: ``architecture``, ``vocab``, ``width``, ``norm.eps``, ``streams`` (absent: one stream and the plain sum), and
``layers``, a list of ``{"type", "mixer": {...}, "mlp": {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top",
"identity"}} | null}``.  Every size and constant comes from there; a missing or ill-typed key is an error that names it.
Tensor names: ``embed``, ``final.norm``, and per layer ``l<i>.norm1 | norm2``, ``l<i>.hc1.* | hc2.*``, ``l<i>.mix.*`` and
``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

from .renanex import _get, _int, _num
from .specs import (ConfigError, DiffAttentionSpec, EmbeddingSpec, HeadSpec, LatentAttentionSpec, LayerSpec, ModelSpec,
                    MultiStreamLayerSpec, NormSpec, RotarySpec, RoutedMlpSpec, StateSpaceDualSpec, StreamMixSpec)

ARCHITECTURE = "Befirax"
# the configuration names no longest sequence: positions are 32-bit integers, and the pools bound a request
MAX_POSITIONS = 1 << 30


@dataclass(frozen=True)
class DiffAttentionLayer:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    conv: int                          # taps of the convolution on q, k and v; 0: none
    rot: Optional[Tuple[float, int]]   # (base, dims) or None
    kv_from: Optional[int]             # the layer whose keys and values this one reads
    type: str = "attention"


@dataclass(frozen=True)
class LatentLayer:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    base: float
    window: Optional[int]
    type: str = "latent_attention"


@dataclass(frozen=True)
class StateSpaceLayer:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int
    type: str = "mamba2"


@dataclass(frozen=True)
class ExpertsMlp:
    experts: int
    top: int
    identity: int
    ff: int
    kind: str = "moe"


def _rot_of(m: dict, where: str, most: int) -> Optional[Tuple[float, int]]:
    if m.get("rot") is None:
        return None
    r = m["rot"]
    dims = _int(r, "dims", where + "rot.", 2)
    if dims % 2 or dims > most:
        raise ConfigError(f"config.json: '{where}rot.dims' {dims} must be even and at most {most}")
    return _num(r, "base", where + "rot."), dims


def _mixer_of(kind, m: dict, where: str, index: int):
    if kind == "attention":
        heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
        if heads % kv:
            raise ConfigError(f"config.json: '{where}heads' {heads} is not a multiple of '{where}kv_heads' {kv}")
        dim = _int(m, "dim", where)
        src = m.get("kv_from")
        if src is not None and (isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < index):
            raise ConfigError(f"config.json: '{where}kv_from' must name an earlier layer, got {src!r}")
        diff = _num(m, "diff", where, positive=False)
        if not 0.0 <= diff < 1.0:
            raise ConfigError(f"config.json: '{where}diff' must lie in [0, 1), got {diff!r}")
        return DiffAttentionLayer(heads, kv, dim, _int(m, "vdim", where), _num(m, "scale", where), diff,
                                  _int(m, "conv", where, 0) if m.get("conv") is not None else 0, _rot_of(m, where, dim), src)
    if kind == "latent_attention":
        rot_dim = _int(m, "rot_dim", where, 2)
        rot = _rot_of(m, where, rot_dim)
        if rot is None or rot[1] != rot_dim:
            raise ConfigError(f"config.json: '{where}rot.dims' must equal '{where}rot_dim' {rot_dim}: the whole part is rotated")
        window = _int(m["mask"], "size", where + "mask.") if m.get("mask") is not None else None
        return LatentLayer(_int(m, "heads", where), _int(m, "dim", where), rot_dim, _int(m, "vdim", where), _int(m, "kv_rank", where),
                           _num(m, "scale", where), rot[0], window)
    if kind == "mamba2":
        heads, groups, parts = _int(m, "heads", where), _int(m, "groups", where), _int(m, "norm_groups", where)
        vdim = _int(m, "vdim", where)
        if heads % groups:
            raise ConfigError(f"config.json: '{where}heads' {heads} is not a multiple of '{where}groups' {groups}")
        if (heads * vdim) % parts:
            raise ConfigError(f"config.json: '{where}norm_groups' {parts} does not divide heads x vdim = {heads * vdim}")
        return StateSpaceLayer(heads, vdim, _int(m, "state", where), groups, _int(m, "conv", where), parts)
    raise ConfigError(f"config.json: '{where[:-6]}type' {kind!r} is not a mixer of this architecture (attention, latent_attention, mamba2)")


def _mlp_of(mlp, where: str) -> Optional[ExpertsMlp]:
    if mlp is None:
        return None
    if not isinstance(mlp, dict):
        raise ConfigError(f"config.json: '{where[:-1]}' must be an object or null")
    kind = _get(mlp, "kind", where)
    if kind != "moe":
        raise ConfigError(f"config.json: '{where}kind' {kind!r} is not a feed-forward of this architecture (moe)")
    router = _get(mlp, "router", where)
    experts, top = _int(router, "experts", where + "router."), _int(router, "top", where + "router.")
    identity = _int(router, "identity", where + "router.", 0) if router.get("identity") is not None else 0
    if top > experts + identity:
        raise ConfigError(f"config.json: '{where}router.top' {top} exceeds the {experts + identity} router outputs")
    return ExpertsMlp(experts, top, identity, _int(_get(mlp, "expert", where), "ff", where + "expert."))


@dataclass(frozen=True)
class BefiraxConfig:
    vocab: int
    width: int
    norm_eps: float
    streams: Optional[int]
    mixers: tuple
    mlps: tuple

    @classmethod
    def from_dict(cls, raw: dict) -> "BefiraxConfig":
        layers = _get(raw, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: 'layers' must be a list of at least one layer")
        mixers, mlps = [], []
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json: 'layers[{i}]' must be an object")
            mixers.append(_mixer_of(_get(layer, "type", where), _get(layer, "mixer", where), where + "mixer.", i))
            mlps.append(_mlp_of(layer.get("mlp"), where + "mlp."))
        for i, m in enumerate(mixers):
            if isinstance(m, DiffAttentionLayer) and m.kv_from is not None:
                src = mixers[m.kv_from]
                where = f"layers[{i}].mixer.kv_from"
                if not isinstance(src, DiffAttentionLayer) or src.kv_from is not None:
                    raise ConfigError(f"config.json: '{where}' {m.kv_from} is not an attention layer with keys and values of its own")
                if (src.kv_heads, src.dim, src.vdim, src.rot) != (m.kv_heads, m.dim, m.vdim, m.rot):
                    raise ConfigError(f"config.json: '{where}' {m.kv_from}: the two layers' key/value heads, sizes and rotation differ")
        streams = _int(raw, "streams", "") if raw.get("streams") is not None else None
        return cls(vocab=_int(raw, "vocab", ""), width=_int(raw, "width", ""), norm_eps=_num(_get(raw, "norm", ""), "eps", "norm."),
                   streams=streams, mixers=tuple(mixers), mlps=tuple(mlps))

    # ------------------------------------------------------------------ back to config.json
    def to_dict(self) -> dict:
        layers = []
        for m, mlp in zip(self.mixers, self.mlps):
            if isinstance(m, DiffAttentionLayer):
                mixer = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale, "diff": m.diff}
                if m.conv:
                    mixer["conv"] = m.conv
                if m.rot is not None:
                    mixer["rot"] = {"base": m.rot[0], "dims": m.rot[1]}
                if m.kv_from is not None:
                    mixer["kv_from"] = m.kv_from
            elif isinstance(m, LatentLayer):
                mixer = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale,
                         "rot": {"base": m.base, "dims": m.rot_dim}}
                if m.window is not None:
                    mixer["mask"] = {"size": m.window}
            else:
                mixer = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "conv": m.conv, "norm_groups": m.norm_groups}
            ff = None
            if mlp is not None:
                ff = {"kind": "moe", "expert": {"ff": mlp.ff}, "router": {"experts": mlp.experts, "top": mlp.top, "identity": mlp.identity}}
            layers.append({"type": m.type, "mixer": mixer, "mlp": ff})
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps}, "layers": layers}
        if self.streams is not None:
            out["streams"] = self.streams
        return out

    # ------------------------------------------------------------------ the model as data
    def _mixer_spec(self, m, p: str):
        if isinstance(m, DiffAttentionLayer):
            rotary = None
            if m.rot is not None:
                rotary = RotarySpec("rotary", m.dim, m.rot[0], rotary_dim=m.rot[1], table_precision="float64", pairing="neighbours")
            names = {"q.weight": p + "q", "k.weight": p + "k", "v.weight": p + "v", "q.bias": p + "q.b", "k.bias": p + "k.b", "v.bias": p + "v.b",
                     "q.conv": p + "q.conv", "k.conv": p + "k.conv", "v.conv": p + "v.conv", "g.weight": p + "g", "o.weight": p + "o",
                     "o.bias": p + "o.b", "lq1": p + "lq1", "lk1": p + "lk1", "lq2": p + "lq2", "lk2": p + "lk2"}
            return DiffAttentionSpec("diff_attention", self.width, m.heads, m.kv_heads, m.dim, m.vdim, m.scale, m.diff, rotary, m.conv, True,
                                     self.norm_eps, m.kv_from, names)
        if isinstance(m, LatentLayer):
            rotary = RotarySpec("rotary", m.rot_dim, m.base, table_precision="float64", pairing="halves")
            names = {"q.weight": p + "q", "dkv.weight": p + "dkv", "dkv.norm": p + "dkv.norm", "uk.weight": p + "uk", "uv.weight": p + "uv",
                     "g.weight": p + "g", "o.weight": p + "o"}
            return LatentAttentionSpec("latent_attention", self.width, m.heads, m.dim, m.rot_dim, m.vdim, 0, m.kv_rank, m.scale, rotary,
                                       self.norm_eps, tensors=names, window=m.window, head_gate=True)
        names = {"in.weight": p + "in", "conv.weight": p + "conv", "conv.bias": p + "conv.b", "dt_bias": p + "dt_bias", "A_log": p + "A_log",
                 "D": p + "D", "norm": p + "norm", "o.weight": p + "o"}
        return StateSpaceDualSpec("mamba2", self.width, m.heads, m.vdim, m.state, m.groups, m.conv, m.norm_groups, self.norm_eps, names)

    def _mlp_spec(self, mlp: ExpertsMlp, q: str) -> RoutedMlpSpec:
        names = {"router.weight": q + "router", "correction": q + "correction"}
        for e in range(mlp.experts):
            for s in ("gate", "up", "down"):
                names[f"e{e}.{s}"] = q + f"e{e}.{s}"
        return RoutedMlpSpec("routed_mlp", self.width, mlp.experts, mlp.top, mlp.ff, "silu", 0, False, names, gated=True,
                             identity=mlp.identity, scoring="softmax_all", correction=True)

    def to_spec(self) -> ModelSpec:
        layers = []
        for i, (m, mlp) in enumerate(zip(self.mixers, self.mlps)):
            mixer = self._mixer_spec(m, f"l{i}.mix.")
            feed = self._mlp_spec(mlp, f"l{i}.mlp.") if mlp is not None else None
            norm2 = self._norm(f"l{i}.norm2") if mlp is not None else None
            # a layer without feed-forward uses neither its second norm nor its second streams' tensors, should the
            # checkpoint have them
            unused = () if mlp is not None else (f"l{i}.norm2",)
            if self.streams is None:
                layers.append(LayerSpec("prenorm", mixer, feed, self._norm(f"l{i}.norm1", unused), norm2))
            else:
                mix = lambda p, ignored=(): StreamMixSpec(self.streams, {"in": p + "in", "out": p + "out", "mix": p + "mix"}, ignored=ignored)
                unused2 = () if mlp is not None else tuple(f"l{i}.hc2.{s}" for s in ("in", "out", "mix"))
                layers.append(MultiStreamLayerSpec("multistream", mixer, feed, self._norm(f"l{i}.norm1", unused), norm2,
                                                   mix(f"l{i}.hc1.", unused2), mix(f"l{i}.hc2.") if mlp is not None else None))
        spec = ModelSpec(architecture=ARCHITECTURE, embedding=EmbeddingSpec(self.vocab, self.width, {"weight": "embed"}),
                         layers=tuple(layers), order=tuple(range(len(layers))), final_norm=self._norm("final.norm"),
                         head=HeadSpec(self.vocab, self.width, True), max_positions=MAX_POSITIONS, streams=self.streams)
        spec.validate()
        return spec

    def _norm(self, name: str, ignored=()) -> NormSpec:
        return NormSpec("rmsnorm", self.width, self.norm_eps, {"weight": name}, ignored=tuple(ignored))

    # ------------------------------------------------------------------ random weights
    def random_tensor_plan(self):
        """(name, shape, law) of every tensor of a random checkpoint; the laws are those of ``weights.random_init``."""
        w = self.width
        plan = [("embed", (self.vocab, w), "matrix")]
        for i, (m, mlp) in enumerate(zip(self.mixers, self.mlps)):
            plan.append((f"l{i}.norm1", (w,), "norm"))
            if mlp is not None:
                plan.append((f"l{i}.norm2", (w,), "norm"))
            p = f"l{i}.mix."
            if isinstance(m, DiffAttentionLayer):
                nq, nk, nv = m.heads * 2 * m.dim, m.kv_heads * 2 * m.dim, m.kv_heads * m.vdim
                own = (("q", nq),) if m.kv_from is not None else (("q", nq), ("k", nk), ("v", nv))
                for s, n in own:
                    plan += [(p + s, (n, w), "matrix"), (p + s + ".b", (n,), "bias")]
                if m.conv:
                    plan += [(p + f"{s}.conv", (n, m.conv), "filter") for s, n in own]
                plan += [(p + s, (m.dim,), "filter") for s in ("lq1", "lk1", "lq2", "lk2")]
                plan += [(p + "g", (m.heads * m.vdim, w), "matrix"), (p + "o", (w, m.heads * m.vdim), "matrix"), (p + "o.b", (w,), "bias")]
            elif isinstance(m, LatentLayer):
                plan += [(p + "q", (m.heads * (m.dim + m.rot_dim), w), "matrix"), (p + "dkv", (m.kv_rank + m.rot_dim, w), "matrix"),
                         (p + "dkv.norm", (m.kv_rank,), "norm"), (p + "uk", (m.heads * m.dim, m.kv_rank), "matrix"),
                         (p + "uv", (m.heads * m.vdim, m.kv_rank), "matrix"), (p + "g", (m.heads, w), "matrix"),
                         (p + "o", (w, m.heads * m.vdim), "matrix")]
            else:
                inner, bc = m.heads * m.vdim, 2 * m.groups * m.state
                plan += [(p + "in", (2 * inner + bc + m.heads, w), "matrix"), (p + "conv", (inner + bc, m.conv), "filter"),
                         (p + "conv.b", (inner + bc,), "bias"), (p + "dt_bias", (m.heads,), "step_bias"), (p + "A_log", (m.heads,), "a_log"),
                         (p + "D", (m.heads,), "norm"), (p + "norm", (inner,), "norm"), (p + "o", (w, inner), "matrix")]
            if mlp is not None:
                q = f"l{i}.mlp."
                for e in range(mlp.experts):
                    plan += [(q + f"e{e}.gate", (mlp.ff, w), "matrix"), (q + f"e{e}.up", (mlp.ff, w), "matrix"),
                             (q + f"e{e}.down", (w, mlp.ff), "matrix")]
                plan += [(q + "router", (mlp.experts + mlp.identity, w), "filter"), (q + "correction", (mlp.experts + mlp.identity,), "bias")]
            if self.streams is not None:
                for hc in ("hc1.", "hc2.") if mlp is not None else ("hc1.",):
                    s = self.streams
                    plan += [(f"l{i}.{hc}in", (s,), "blend"), (f"l{i}.{hc}out", (s,), "norm"), (f"l{i}.{hc}mix", (s, s), "mixing")]
        plan.append(("final.norm", (w,), "norm"))
        return plan
