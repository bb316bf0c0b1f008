"""Typed descriptions of a model: what each part is and how the parts are arranged.

A :class:`ModelSpec` is pure data.  An architecture (see ``registry.py``) turns its
typed configuration into one; ``parts.model.DecoderModel`` builds the parts it names
from the part registries.  A spec of a part carries every size and constant of that
part, and ``tensors`` maps the part's own tensor names to names in the checkpoint, so
no part needs to know which model it belongs to.

Role in the reference: ``crates/mach-model/src/config.rs:15-142`` keeps one flat
struct for all families and dispatches inside one forward function; here the
per-layer choice is data.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Mapping, Optional, Sequence


class ConfigError(ValueError):
    """A configuration that cannot be built; the message names the key and the value."""


@dataclass(frozen=True)
class NormSpec:
    kind: str
    width: int
    eps: float
    tensors: Mapping[str, str] = field(default_factory=dict)
    # a norm whose weight is stored around zero: the weight applied is ``offset`` plus the stored one
    offset: float = 0.0
    # whether a second vector ("scale" among the tensors) multiplies the normed row as well (a layer's scale)
    scaled: bool = False
    # checkpoint names that may be present without being used
    ignored: Sequence[str] = ()


@dataclass(frozen=True)
class YarnSpec:
    """YaRN scaling of a rotation's frequencies (``crates/mach-server/src/startup.rs:172-199``): between the
    pair indices that ``beta_fast`` and ``beta_slow`` rotations over ``original_max_positions`` mark, a frequency
    goes over from its own value to ``1 / factor`` of it; cosines and sines are multiplied by
    ``mscale(factor, mscale) / mscale(factor, mscale_all_dim)`` with ``mscale(f, m) = 0.1 m ln f + 1``."""
    factor: float
    original_max_positions: int
    beta_fast: float = 32.0
    beta_slow: float = 1.0
    mscale: float = 1.0
    mscale_all_dim: float = 0.0


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of pairs ``(j, j + rotary_dim/2)`` with ``freq_j = theta^(-2j/rotary_dim)``, or those frequencies
    scaled as ``yarn`` says."""
    kind: str
    head_dim: int
    theta: float
    tensors: Mapping[str, str] = field(default_factory=dict)
    yarn: Optional[YarnSpec] = None
    # how many numbers of a head are rotated, the first ones (None: all of them); the frequencies and YaRN's pair
    # indices are then those of a head of this size
    rotary_dim: Optional[int] = None
    # the precision in which the table of frequencies is worked out before it is rounded to 32-bit
    table_precision: str = "float32"
    # which numbers of the rotated part make a pair: "halves" (j, j + rotary_dim/2) or "neighbours" (2j, 2j + 1); the
    # table of frequencies is the same, the pairing is the business of the mixer's kernel
    pairing: str = "halves"


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query attention over a paged cache.

    ``window``: number of most recent keys a row may see (None = all).
    ``kv_source``: index of another layer whose cache this layer reads instead of
    writing its own (None = own cache).
    ``scale``: what the scores are multiplied by before the softmax (None = ``head_dim ** -0.5``,
    ``crates/mach-model/src/config.rs:231-234``).
    """
    kind: str
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    position: Optional[RotarySpec]
    window: Optional[int] = None
    kv_source: Optional[int] = None
    tensors: Mapping[str, str] = field(default_factory=dict)
    scale: Optional[float] = None


@dataclass(frozen=True)
class TalkingAttentionSpec:
    """Grouped-query attention whose heads exchange their scaled scores before the softmax
    (``score_h = sum_g talk[h, g] score_g``), with keys ``head_dim`` and values ``v_head_dim`` wide.

    ``qk_norm``: an RMS norm (``norm_eps``) over the whole query projection and one over the whole key projection,
    before the rotation.  ``talk``: whether there is an exchange matrix.  ``window`` / ``keep_first``: a row sees the
    last ``window`` positions up to its own (None: all) and the request's first ``keep_first``.  ``value_blend``:
    None, ``"source"`` (the layer's own values are kept for the layers below to blend with) or ``"blend"``
    (``v = (1 - w) v + w v_source`` with a learned number ``w``; the blended values are cached).
    """
    kind: str
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    v_head_dim: int
    position: Optional[RotarySpec]
    scale: float
    window: Optional[int] = None
    keep_first: int = 0
    qk_norm: bool = False
    norm_eps: float = 1e-6
    talk: bool = True
    value_blend: Optional[str] = None
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class ConvAttentionSpec:
    """Grouped-query attention whose values are its keys, behind a short convolution.

    ``q = W_q h``, ``k = W_k h``; with ``conv_taps`` > 1 a causal convolution over time on every channel of q and k
    (``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, no bias), whose last ``conv_taps - 1`` inputs are a request's state; the
    values are the keys as they leave the convolution; with ``unit_norm`` q and k of every head are divided by their
    root mean square (``norm_eps``, no weight); ``q_temp`` = (coef, every): the query at position p is multiplied by
    ``1 + coef ln(floor((p + 1) / every) + 1)`` (None: not); ``score = scale q . k``, causal softmax; with ``gate`` head
    h's output is multiplied by ``sigmoid(W_g h)_h``; output projection."""
    kind: str
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    scale: float
    conv_taps: int = 0
    unit_norm: bool = True
    norm_eps: float = 1e-6
    q_temp: Optional[tuple] = None
    gate: bool = True
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention through a latent: per token the cache keeps an RMS-normed vector ``c`` of ``kv_rank`` numbers and one
    rotated key part of ``rot_dim`` numbers that all heads share.  Queries come through a normed bottleneck of
    ``q_rank``; a head's query is ``[head_dim plain | rot_dim rotated]``, its key ``[W_uk c | rotated part]``, its value
    ``W_uv c`` (``v_head_dim``).  ``position`` describes the rotation of the ``rot_dim`` part (None: none); its cosines and
    sines carry YaRN's factor, the plain part and ``scale`` do not.  ``sink``: the softmax's denominator also holds
    ``exp(sink_h)``, a learned number per head without key or value.  ``kv_source``: index of another such layer whose
    cache this layer reads (with its own ``W_uk``, ``W_uv``) instead of writing one."""
    kind: str
    hidden: int
    heads: int
    head_dim: int
    rot_dim: int
    v_head_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    position: Optional[RotarySpec]
    norm_eps: float = 1e-6
    sink: bool = False
    kv_source: Optional[int] = None
    tensors: Mapping[str, str] = field(default_factory=dict)
    # ``q_rank`` 0: no bottleneck, the heads' queries are one projection of the input ("q.weight")
    # a row at position i sees the keys j with ``0 <= i - j < window`` (None: every j <= i)
    window: Optional[int] = None
    # a head's output is multiplied by the sigmoid of one number a head, a projection of the mixer's input ("g.weight")
    head_gate: bool = False


@dataclass(frozen=True)
class DiffAttentionSpec:
    """Differential grouped-query attention: every head has two softmax maps over the same values, each with queries and
    keys of its own (q is ``heads x 2 x head_dim``, k ``kv_heads x 2 x head_dim``, a head's two maps side by side), and its
    result is ``a1 - lambda a2`` with ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff`` one number a layer, divided by its
    root mean square over the head's ``v_head_dim`` values (``norm_eps``, no weight) and multiplied by ``1 - diff``; the
    heads side by side are multiplied by ``sigmoid(W_g h)`` and projected.  With ``conv_taps`` > 0 a causal convolution
    over time on every channel of q, k and v comes right behind the projections (no bias; the last ``conv_taps - 1``
    inputs are a request's state); ``position``: the rotation of every map of q and k.  ``kv_source``: index of another
    such layer whose keys and values this layer reads instead of having its own."""
    kind: str
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    v_head_dim: int
    scale: float
    diff: float
    position: Optional[RotarySpec] = None
    conv_taps: int = 0
    bias: bool = True
    norm_eps: float = 1e-6
    kv_source: Optional[int] = None
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class StateSpaceDualSpec:
    """The second Mamba layer: ``heads`` heads of ``head_dim`` value channels with a state of ``states x head_dim`` each,
    ``S <- exp(-exp(A_log) dt) S + dt B x^T``, ``y = S^T C + D x`` with one step size a head and token (``dt = softplus(. +
    dt_bias)``) and B and C shared by the heads of a group.  The input projection is ``[z | x | B | C | dt]``; x, B and C
    pass a causal convolution of ``conv_taps`` per channel with bias and SiLU; ``y silu(z)`` is RMS-normed in
    ``norm_groups`` equal parts (``norm_eps``, a weight per channel) and projected."""
    kind: str
    hidden: int
    heads: int
    head_dim: int
    states: int
    groups: int
    conv_taps: int
    norm_groups: int = 1
    norm_eps: float = 1e-6
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class SelectiveScanSpec:
    """A Mamba layer: input projection to ``[x | z]`` of ``inner`` channels each, a causal convolution of
    ``conv_taps`` taps per channel with SiLU, step sizes from a ``dt_rank`` bottleneck, a scan over ``states``
    states a channel, the gate ``silu(z)`` and an output projection."""
    kind: str
    hidden: int
    inner: int
    states: int
    dt_rank: int
    conv_taps: int
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class LightningSpec:
    """Linear attention with one decay per head: ``S <- decay_h S + k v^T``, ``o = S^T q`` with SiLU on q, k and v; the
    heads' outputs are normed together (``norm_eps``), gated by a sigmoid and projected."""
    kind: str
    hidden: int
    heads: int
    head_dim: int
    v_head_dim: int
    decay: Sequence[float]
    norm_eps: float = 1e-6
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class ChunkedAttentionSpec:
    """Grouped-query attention with keys ``head_dim`` and values ``v_head_dim`` wide, behind a short convolution on q, k and v.

    ``q, k, v = W h (+ bias)``; with ``conv_taps`` > 0 a causal convolution over time on every channel of q, k and v
    (``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, no bias), whose last ``conv_taps - 1`` inputs are a request's state; with
    ``qk_norm`` an RMS norm (``norm_eps``, a weight per coordinate) over the whole of q and one over the whole of k;
    ``position``: the rotation of q and k (its ``rotary_dim`` first numbers of a head, pairs as its ``pairing`` says; None:
    none); ``score = scale q . k``, then with ``softcap`` ``softcap tanh(score / softcap)``; a row at position i sees the
    keys j <= i with ``floor(i / chunk) = floor(j / chunk)`` (``chunk`` None: every j <= i) and, with ``window``, ``i - j <
    window``; softmax; output projection."""
    kind: str
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    v_head_dim: int
    scale: float
    position: Optional[RotarySpec] = None
    conv_taps: int = 0
    bias: bool = True
    qk_norm: bool = True
    norm_eps: float = 1e-6
    softcap: float = 0.0
    chunk: Optional[int] = None
    window: Optional[int] = None
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class GatedRecurrenceSpec:
    """A recurrent block around a real-gated linear recurrent unit: two branches of ``width`` channels,
    ``y = gelu_tanh(W_y h + b_y)`` and ``u = conv(W_x h + b_x) + b_conv`` (a causal convolution of ``conv_taps`` taps per
    channel); the channels are cut into ``blocks`` equal parts, in each ``r = sigmoid(A u + b_a)`` and ``i = sigmoid(B u +
    b_i)`` with square matrices; ``a = exp(-decay_factor r softplus(lam))``, ``S <- a S + sqrt(1 - a^2) (i u)`` from zero;
    the output is ``W_o (S y)``."""
    kind: str
    hidden: int
    width: int
    blocks: int
    conv_taps: int
    decay_factor: float = 8.0
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class TimeMixSpec:
    """Time mixing with a decay per key channel that depends on the token.  Each of r, k, v, g, w reads its own mix of a
    token's input with the one before it, ``h + (h' - h) mu``; ``r, k, v = W mix`` (``heads`` x ``head_dim``), the gate
    ``silu(W_g mix_g)``, the decay ``w = exp(-exp(W_2 tanh(W_1 mix_w) + w0))`` through a bottleneck of ``decay_rank`` (None:
    whatever the checkpoint's tensors have); per head ``o = (S + diag(u) k v^T)^T r``, ``S <- diag(w) S + k v^T``; a head's
    ``o`` is divided by its root mean square (``norm_eps``), times a weight, times the gate, and projected."""
    kind: str
    hidden: int
    heads: int
    head_dim: int
    decay_rank: Optional[int] = None
    norm_eps: float = 1e-6
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class SideBySideSpec:
    """Several mixers that read the same input; each one's output is RMS-normed over the model's width (``norm_eps``) with a
    weight of its own (``tensors``: ``norm.<i>``), and the result is their mean."""
    kind: str
    hidden: int
    branches: Sequence[object]
    norm_eps: float = 1e-6
    tensors: Mapping[str, str] = field(default_factory=dict)


@dataclass(frozen=True)
class RoutedMlpSpec:
    """A feed-forward of ``experts`` small layers ``W_down act(W_up h)`` without biases, of which a token uses the ``top``
    with the largest router logits ``W_r h (+ bias)``, weighted by the softmax over the chosen logits alone; with
    ``shared`` > 0 one more such layer of that size runs for every token and is added."""
    kind: str
    hidden: int
    experts: int
    top: int
    intermediate: int
    activation: str = "gelu"
    shared: int = 0
    router_bias: bool = True
    tensors: Mapping[str, str] = field(default_factory=dict)
    # an expert is ``W_down (act(W_gate h) * (W_up h))`` ("e<i>.gate" beside "e<i>.up")
    gated: bool = False
    # the router has this many outputs more, which stand for experts without tensors that return their input
    identity: int = 0
    # "softmax_chosen": the weights are the softmax over the chosen logits; "softmax_all": scores are the softmax over
    # every router output, and the weights the chosen scores over their sum (+ 1e-20)
    scoring: str = "softmax_chosen"
    # with "softmax_all": a vector ("correction") added to the scores for the choice only
    correction: bool = False


@dataclass(frozen=True)
class GatedMlpSpec:
    """``down(act(gate(x)) * up(x))``; with ``bias`` every projection has one."""
    kind: str
    hidden: int
    intermediate: int
    activation: str = "silu"
    tensors: Mapping[str, str] = field(default_factory=dict)
    bias: bool = False


@dataclass(frozen=True)
class LayerSpec:
    """One pre-norm block: the specs of the four parts it arranges.  ``block`` names the registered arrangement,
    which builds its parts from the fields it reads; another arrangement brings a spec class of its own (any object
    with ``block`` and the fields that arrangement reads)."""
    block: str
    mixer: object
    feed_forward: object
    mixer_norm: object
    feed_forward_norm: object


@dataclass(frozen=True)
class SandwichLayerSpec:
    """A block with a norm before and after each branch: ``x += post(mixer(pre(x)))``, then the same around the
    feed-forward; ``feed_forward`` None: the layer has none (then its two norms are None too)."""
    block: str
    mixer: object
    feed_forward: Optional[object]
    mixer_norm: object
    mixer_post_norm: object
    feed_forward_norm: Optional[object]
    feed_forward_post_norm: Optional[object]


@dataclass(frozen=True)
class PostNormLayerSpec:
    """A block whose branches read the stream itself and are normed on their way out: ``x += post(mixer(x))``, then
    ``x += post(feed_forward(x))``; ``feed_forward`` None: the layer has none."""
    block: str
    mixer: object
    feed_forward: Optional[object]
    mixer_post_norm: object
    feed_forward_post_norm: Optional[object]


@dataclass(frozen=True)
class StreamMixSpec:
    """How one branch reads and writes several residual streams: ``u = sum_s in[s] x_s`` is the branch's input, and all
    streams at once become ``x_t = sum_s mix[s, t] x_s + out[t] y``."""
    streams: int
    tensors: Mapping[str, str] = field(default_factory=dict)
    kind: str = "stream_mix"
    # checkpoint names that may be present without being used
    ignored: Sequence[str] = ()


@dataclass(frozen=True)
class MultiStreamLayerSpec:
    """A pre-norm block over several residual streams: each branch reads a weighted sum of the streams through its norm
    and is written back into all of them (``mixer_streams``, ``feed_forward_streams``); ``feed_forward`` None: the layer
    has none."""
    block: str
    mixer: object
    feed_forward: Optional[object]
    mixer_norm: object
    feed_forward_norm: Optional[object]
    mixer_streams: StreamMixSpec
    feed_forward_streams: Optional[StreamMixSpec]


@dataclass(frozen=True)
class ParallelLayerSpec:
    """A block whose branches read one norm: ``h = norm(x); x += mixer(h) + feed_forward(h)``; ``feed_forward`` None:
    the layer has none."""
    block: str
    mixer: object
    feed_forward: Optional[object]
    norm: object


@dataclass(frozen=True)
class EmbeddingSpec:
    """Token embedding: rows of a table, times ``scale``."""
    vocab: int
    width: int
    tensors: Mapping[str, str] = field(default_factory=dict)
    kind: str = "embedding"
    scale: float = 1.0


@dataclass(frozen=True)
class PairEmbeddingSpec:
    """Token embedding plus a row of a second table chosen by the token and the one before it: row ``(previous * mul_prev +
    token * mul_cur) mod buckets``, and row ``buckets`` (the last) for a request's first token."""
    vocab: int
    width: int
    buckets: int
    mul_prev: int
    mul_cur: int
    tensors: Mapping[str, str] = field(default_factory=dict)
    kind: str = "pair_embedding"


@dataclass(frozen=True)
class HeadSpec:
    """Output projection.  ``tied``: use the embedding table; ``tied=None``: use the head
    tensor if the checkpoint has it, else the embedding table."""
    vocab: int
    width: int
    tied: Optional[bool]
    tensors: Mapping[str, str] = field(default_factory=dict)
    kind: str = "linear"
    scale: float = 1.0  # the logits are multiplied by it
    softcap: float = 0.0  # then ``softcap * tanh(logits / softcap)``; 0: no cap


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    embedding: EmbeddingSpec
    layers: Sequence[LayerSpec]
    order: Sequence[int]
    final_norm: object
    head: HeadSpec
    max_positions: int
    # several residual streams, all equal to the embedding at the start and summed at the end (None: the one stream)
    streams: Optional[int] = None

    def validate(self) -> None:
        n = len(self.layers)
        if not self.order:
            raise ConfigError("order: a model runs at least one layer")
        for i in self.order:
            if not 0 <= i < n:
                raise ConfigError(f"order names layer {i}, but there are {n} layers")
        for i, layer in enumerate(self.layers):
            src = getattr(getattr(layer, "mixer", None), "kv_source", None)
            if src is not None:
                if not 0 <= src < n or src == i:
                    raise ConfigError(f"layer {i}: kv_source {src} is not another layer")
                if getattr(getattr(self.layers[src], "mixer", None), "kv_source", None) is not None:
                    raise ConfigError(f"layer {i}: kv_source {src} itself reads another layer's cache")
                if self.order.index(src) > self.order.index(i):
                    raise ConfigError(f"layer {i} reads the cache of layer {src}, which runs later")
