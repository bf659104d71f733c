"""A model as data: what each layer is made of, and the order in which layers run.

A plan holds no tensors and no code.  Each spec names a part by `kind` (looked up in
the part registries of `parts.base`) and carries every size and constant that part
needs, so no part ever asks which model it is in.  The run list is data too: it may
name a layer twice, or let a run read the cache that another run writes.
"""

from dataclasses import dataclass
from typing import Any, Optional


@dataclass(frozen=True)
class NormSpec:
    """kind "rmsnorm": x / sqrt(mean(x^2) + eps) * gain.  kind "grouped_rmsnorm": the row is cut into `groups` equal
    consecutive parts, each divided by its own root mean square, the whole times the gain."""

    kind: str
    size: int
    eps: float
    groups: int = 1
    offset: float = 0.0  # added to the stored gain (1.0: a gain stored around zero); the sum is kept in 32 bits


@dataclass(frozen=True)
class RotarySpec:
    """Rotary position encoding of a head's first `rotary_dim` coordinates.
    kind "rope_half": pairs are (i, i + rotary_dim/2)."""

    kind: str
    rotary_dim: int
    theta: float


@dataclass(frozen=True)
class ScaledRotarySpec:
    """A rotation ("rope_half" layout) whose frequencies are stretched for contexts beyond `original` positions:
    with dim(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(dim(fast)), 0), hi =
    min(ceil(dim(slow)), rotary_dim - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns by
    position * (f_i / factor * ramp_i + f_i (1 - ramp_i)), and cosines and sines are multiplied by 0.1 ln(factor) + 1.
    kind "rope_half_scaled"."""

    kind: str
    rotary_dim: int
    theta: float
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class NeighbourRotarySpec:
    """Rotary position encoding of a head's first `rotary_dim` coordinates whose pairs are neighbours, (2i, 2i + 1).
    kind "rope_neighbours".  With `factor` > 0 the frequencies are stretched as `ScaledRotarySpec` says."""

    kind: str
    rotary_dim: int
    theta: float
    factor: float = 0.0
    original: float = 0.0
    fast: float = 0.0
    slow: float = 0.0


@dataclass(frozen=True)
class DecayAttentionSpec:
    """Linear attention with a fixed decay per head and no softmax: S = decay_h S + k v^T, o = S^T q.  q, k
    [heads, key_dim] and v [heads, value_dim] pass `activation` (None or "silu"); k is also multiplied by `key_scale`.
    out_norm "heads": every head's o is divided by its root mean square, no gain; "all": the concatenated heads are
    RMS-normed together and multiplied by a gain.  The result times `gate` ("sigmoid" or "silu") of a projection of
    the input goes through the output projection."""

    kind: str  # "decay_attention"
    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    decay: tuple  # per head
    activation: Optional[str]
    key_scale: float
    out_norm: str
    out_norm_eps: float
    gate: str


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Causal softmax attention whose keys and values are matrices times a cached latent [kv_rank] per token, beside
    one rotated key part [rot_dim] shared by all heads; queries pass a normed latent of their own [q_rank] and are,
    per head, `head_dim` coordinates that are not rotated and then `rot_dim` that are.  score = scale (q . k of both
    parts).  The concatenated heads [heads, value_dim] times sigmoid of a projection of the input go through the
    output projection.  own_latent False: the layer has no projection to the latent; it reads the pages of the run
    that its run names as its cache."""

    kind: str  # "latent_attention"
    hidden_size: int
    num_heads: int
    head_dim: int
    rot_dim: int
    value_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    norm_eps: float
    position: Any  # of the rot_dim coordinates; a position spec of pairs "half", or None
    own_latent: bool = True


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged cache."""

    kind: str  # "attention"
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float  # multiplies q.k before the softmax
    qk_norm: Optional[NormSpec]  # per-head norm of q and k before the rotation, or None
    position: Optional[RotarySpec]  # applied to q and k, or None
    window: int = 0  # > 0: a query at p sees keys p-window+1..p only; 0: all keys


@dataclass(frozen=True)
class MixedHeadsAttentionSpec:
    """Grouped-query softmax attention whose heads' scores are mixed by a matrix [heads, heads] before the
    softmax (`mix_heads`), over a window that keeps the sequence's first `keep_first` tokens visible
    (window 0: all keys).  `values` "keys": there is no value projection, a key as projected (before its
    rotation) is also the value; "own": values have a projection of their own.  `out_gate`: the part also
    computes sigmoid-gate logits [hidden] of its input (with a bias) for whoever adds its output to the stream."""

    kind: str  # "mixed_heads_attention"
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    position: Optional[RotarySpec]
    window: int = 0
    keep_first: int = 0
    mix_heads: bool = True
    values: str = "keys"
    out_gate: bool = False


@dataclass(frozen=True)
class GatedMLPSpec:
    """Dense gated feed-forward: down(act(gate(x)) * up(x))."""

    kind: str  # "gated_mlp"
    hidden_size: int
    intermediate_size: int
    activation: str  # "silu": silu(gate) * up; "clamped_swish": g sigmoid(1.702 g) (u + 1), g = min(gate, limit), u = clamp(up, +-limit)
    limit: float = 0.0


@dataclass(frozen=True)
class ShortConvSpec:
    """Causal convolution per channel over the last `taps` tokens (the last tap is the current token's)."""

    taps: int


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Gated delta rule: per head a state [key_dim, value_dim] that decays, is corrected towards the
    token's value along its key and is read along its query; q, k, v pass a short convolution and silu,
    q and k become unit vectors (eps inside the root), the output is normed per head and gated.
    num_kv_heads heads of q and k serve num_heads heads of v."""

    kind: str  # "delta_rule"
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    conv: ShortConvSpec
    out_norm_eps: float  # of the RMS norm of every head's output
    unit_eps: float = 1e-6  # inside the root of the unit norms


@dataclass(frozen=True)
class GatedAttentionSpec:
    """Softmax attention whose concatenated heads are multiplied by sigmoid(gate(h)) before the output
    projection.  Keys and queries are `key_dim` wide, values `value_dim`; no position encoding."""

    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    qk_norm: Optional[NormSpec]
    window: int = 0


@dataclass(frozen=True)
class LinearRecurrenceSpec:
    """Real-gated linear recurrent unit: S = a S + sqrt(1 - a^2) i u with a = exp(-decay_scale r softplus(lam)),
    the gates r and i from block-diagonal matrices on u = conv(x(h)); the output is S * gelu(y(h))."""

    width: int
    blocks: int
    conv: ShortConvSpec
    decay_scale: float = 8.0


@dataclass(frozen=True)
class SideBySideSpec:
    """Two mixers that read the same input; their outputs are added with a weight each, inside one
    output projection: left_scale * attention + right_scale * recurrence."""

    kind: str  # "side_by_side"
    hidden_size: int
    left: GatedAttentionSpec
    right: LinearRecurrenceSpec
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class SoftmaxCoreSpec:
    """A grouped-query causal softmax attention as one of the cores of a "joined" mixer: keys and queries `key_dim`
    wide, values `value_dim`.  bias: q, k and v have biases.  whole_norm_eps > 0: q and k are RMS-normed over their
    whole projection (all heads at once) with gains of that size.  position: a rotation of q and k, or None.
    value_mix "first": the core's values (of the step's tokens) are kept for later layers under `value_mix_key`;
    "later": its values become (1 - lam) v + lam v_first before they are cached, lam a scalar of its own.
    out_gate: the concatenated heads are multiplied by sigmoid of a projection of the input."""

    kind: str  # "softmax_core"
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    bias: bool = False
    whole_norm_eps: float = 0.0
    position: Any = None
    value_mix: str = "none"
    value_mix_key: str = "values"
    out_gate: bool = False


@dataclass(frozen=True)
class MatrixMemorySpec:
    """A matrix memory with exponential gates, per head: a state S [key_dim, value_dim], a normaliser n [key_dim] and
    a running maximum m (0 at the start) of the gates' logarithms i = cap tanh(. / cap) and f = logsigmoid(cap tanh(. / cap)):
    m' = max(f + m, i); S' = e^(f + m - m') S + e^(i - m') k v^T, n' likewise with k; o = S'^T q / (max(|n' . q|, e^(-m')) +
    1e-6) with q times key_dim^(-1/2).  Every head's o over its root mean square, the heads times a gain [heads x
    value_dim] and sigmoid of a projection of the input.  One of the cores of a "joined" mixer."""

    kind: str  # "matrix_memory"
    num_heads: int
    key_dim: int
    value_dim: int
    gate_cap: float
    out_norm_eps: float


@dataclass(frozen=True)
class JoinedMixerSpec:
    """Several cores that read the same input; one input product makes what all of them need and one output product
    takes scales[c] * core c's result side by side, so the weighted sum of the cores is the product's own sum."""

    kind: str  # "joined"
    hidden_size: int
    cores: tuple
    scales: tuple


@dataclass(frozen=True)
class ChannelDeltaRuleSpec:
    """The gated delta rule of `DeltaRuleSpec` with a decay per head and key channel, g = exp(-exp(A_h) softplus(W_2
    (W_1 h) + b)) laid out heads x key_dim and acting on the rows of S; the output is normed per head (a gain
    [value_dim] shared by the heads) and times sigmoid(G_2 (G_1 h)).  decay_rank and gate_rank: rows of W_1 and G_1."""

    kind: str  # "channel_delta_rule"
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    conv: ShortConvSpec
    decay_rank: int
    gate_rank: int
    out_norm_eps: float
    unit_eps: float = 1e-6


@dataclass(frozen=True)
class TableExpertsSpec:
    """Gated feed-forward experts of which every token uses `top`, named by a table indexed with the
    token id; each chosen expert weighs 1 / top."""

    kind: str  # "table_experts"
    hidden_size: int
    intermediate_size: int
    num_experts: int
    top: int
    vocab_size: int
    activation: str  # "silu"


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """Experts chosen by a router: scores = `score`(router h) in fp32, the `top` largest are chosen and weigh
    their scores divided by the chosen scores' sum (+ 1e-20).  An expert is down(act(up h)) without a gate
    (`activation` "relu2": relu squared).  shared_size > 0: one more expert of that width runs for every token and
    is added.  `out_gate` as for `MixedHeadsAttentionSpec`."""

    kind: str  # "routed_experts"
    hidden_size: int
    intermediate_size: int
    num_experts: int
    top: int
    activation: str  # "relu2"
    score: str = "sigmoid"
    shared_size: int = 0
    out_gate: bool = False


@dataclass(frozen=True)
class GatedRoutedExpertsSpec:
    """Gated experts chosen by a router: z = router h + bias in fp32, the `top` largest z are chosen and weigh the
    softmax over the chosen z alone (`score` "softmax_of_chosen").  `score` "softmax": s = softmax(z) over all
    experts; the experts form `groups` equal groups of neighbours, a group scores its largest s, and the `top`
    largest s among the experts of the `keep_groups` best groups are chosen; they weigh s * weight_scale, not
    renormalised.  An expert is down(act(gate h, up h)) with the
    activation of `GatedMLPSpec` and `limit`.  shared_size > 0: one more such expert (with `shared_limit`) runs for
    every token and is added."""

    kind: str  # "gated_routed_experts"
    hidden_size: int
    intermediate_size: int
    num_experts: int
    top: int
    activation: str
    limit: float
    score: str = "softmax_of_chosen"
    router_bias: bool = True
    shared_size: int = 0
    shared_limit: float = 0.0
    groups: int = 1
    keep_groups: int = 1
    weight_scale: float = 1.0


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward with their norms, and how they are arranged.
    arrangement "prenorm": x += mixer(norm(x)); x += ffn(norm(x)).
    arrangement "two_norms": x += mixer(mixer_norm(x)) + ffn(ffn_norm(x)), both of the same x
    (ffn and ffn_norm None: the mixer alone).
    arrangement "gated_prenorm": x += m g(h) * mixer(h), h = norm(x); then the same with the feed-forward (or
    none): m = residual_scale, g the sigmoid gate whose logits the part computes from its input (`out_gate`).
    arrangement "depth_prenorm": "prenorm" (ffn None: the mixer alone) with two options.  token_shift: what the mixer
    reads is h_t + (h_(t-1) - h_t) * shift, h the mixer's norm of the stream (zeros before a sequence's first token;
    the last h is part of a request's state).  depth_slots > 0: the layer's result is kept as number depth_index + 1
    of depth_slots results (number 0 is what the embedding gave), and the stream goes on as their weighted sum with
    depth_index + 2 weights of the layer's own.
    arrangement "streams_prenorm": the stream is `streams` copies x_1 .. x_s (all what the embedding gave before the
    layer marked streams_first); a sublayer reads u = sum_s a[s] x_s through its norm and writes x_t <- sum_s M[s, t]
    x_s + residual_scale c[t] y with a, M, c of its own; the layer marked streams_last leaves their sum as the
    stream.  streams 0: one stream with a = M = c = 1, that is x += residual_scale y."""

    arrangement: str
    mixer: Any
    mixer_norm: NormSpec
    ffn: Any
    ffn_norm: Optional[NormSpec]
    residual_scale: float = 1.0
    token_shift: bool = False
    depth_index: int = 0
    depth_slots: int = 0
    streams: int = 0
    streams_first: bool = False
    streams_last: bool = False


@dataclass(frozen=True)
class Run:
    """One entry of the run list: execute layer `layer`.

    cache: id of the cache this run's mixer uses (None: a cache of its own, named after
           the run's index).  Two runs with the same id share one cache.
    writes: whether this run stores what it computes into that cache; a run that only
           reads another run's cache sets this to False.
    reenter: before this run the stream is replaced by reentry [x ; x0], x0 being what the embedding (and
           its norm) put into the stream; the plan then names `reentry`.
    """

    layer: int
    cache: Optional[int] = None
    writes: bool = True
    reenter: bool = False


@dataclass(frozen=True)
class ModelPlan:
    vocab_size: int
    hidden_size: int
    layers: tuple  # of BlockSpec
    run: tuple  # of Run
    final_norm: NormSpec
    tied_head: bool
    max_positions: int
    embedding_scale: float = 1.0  # multiplies the embedding rows as they enter the stream
    logit_scale: float = 1.0  # multiplies the head's output
    logit_softcap: float = 0.0  # > 0: logits = cap * tanh(logits / cap), after the scale
    embed_norm: Optional[NormSpec] = None  # a norm of the embedding rows before they become the stream
    reentry: bool = False  # a matrix [hidden, 2 hidden] through which runs marked `reenter` take [x ; x0]

    def cache_id(self, run_index: int) -> int:
        r = self.run[run_index]
        return run_index if r.cache is None else r.cache


def sequential_run(num_layers: int) -> tuple:
    """Every layer once, in order, each with a cache of its own."""
    return tuple(Run(i) for i in range(num_layers))
