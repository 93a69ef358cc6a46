"""Descriptions of the parts a model is put together from.

A spec is plain data: a ``kind`` that names an entry of the part registry and
the sizes and constants that part needs.  A model is a list of layer specs plus
the order in which the layers run; nothing in a spec says which architecture it
came from, and nothing in a part reads anything but its own spec.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional


@dataclass(frozen=True)
class NormSpec:
    """A normalisation over the last axis."""
    kind: str = "rms_norm"
    eps: float = 1e-6
    gain_offset: float = 0.0                # the stored gain plus this is the gain (1.0: gains stored around zero)


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.  ``rotary_half`` rotates the pairs
    (i, i + dim/2) of each head by position * theta^(-2i/dim)."""
    kind: str = "rotary_half"
    dim: int = 0
    theta: float = 10000.0
    max_positions: int = 0


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query attention over a paged cache."""
    kind: str = "paged_attention"
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    qk_norm: Optional[NormSpec] = None      # per-head norm on q and k before the position encoding
    position: Optional[PositionSpec] = None
    window: Optional[int] = None            # keys j with pos - window < j <= pos; None = all keys
    scale: Optional[float] = None           # None = 1/sqrt(head_dim)
    qkv_bias: bool = False                  # q, k and v projections carry a bias each
    out_bias: bool = False                  # the output projection carries one


@dataclass(frozen=True)
class GatedMlpSpec:
    """down(act(gate(x)) * up(x))."""
    kind: str = "gated_mlp"
    intermediate_size: int = 0
    activation: str = "silu"
    # the tensors' names inside the feed-forward, where a family stores them under others: (gate, up, down)
    names: Optional[tuple] = None


@dataclass(frozen=True)
class LayerSpec:
    """One layer: which block arrangement, and its mixer, feed-forward and norm."""
    block: str = "pre_norm"
    mixer: Any = None
    feed_forward: Any = None
    norm: Any = None
    weight_prefix: str = ""
    names: Optional[dict] = None            # other tensor-name parts for the block's members (norm1, mixer, norm2, feed_forward)
    stream_copies: Optional[int] = None     # for an arrangement over several copies of the stream: how many
    layer_scale: bool = False               # a sublayer's output times a gain a column before it joins the stream (``ls1``, ``ls2``)


@dataclass(frozen=True)
class ScheduleEntry:
    """One step of the order in which layers run.  A layer may appear twice;
    ``cache_from`` lets this run read the cache another layer wrote instead of
    writing its own."""
    layer: int
    cache_from: Optional[int] = None
    # A layer that runs several times with the same weights keeps pages and state of its own for every run:
    # runs with different ``cache_key`` (any numbers; None is the layer's own index) share nothing.  ``cache_from``
    # names the key that is read.
    cache_key: Optional[int] = None
    # The stream as it was right behind the embedding (and its transforms) is added to the stream before this run:
    # a stretch of layers that runs again starts every further pass from what it left plus what the model began with.
    add_embedding: bool = False


@dataclass(frozen=True)
class ModelSpec:
    """Everything the generic decoder needs, independent of the architecture."""
    hidden_size: int
    vocab_size: int
    layers: tuple
    schedule: tuple
    final_norm: Any
    tie_word_embeddings: bool
    max_positions: int
    embed_name: str = "model.embed_tokens.weight"
    final_norm_name: str = "model.norm.weight"
    head_name: str = "lm_head.weight"
    # Tensors a checkpoint of this family carries and the model does not use (buffers, tables that are
    # computed here): shell patterns over tensor names, e.g. "*.rotary_emb.inv_freq".  They are neither
    # loaded nor reported as unexpected.
    ignored_tensors: tuple = ()
    # What the decoder does beside the layers, by the names of registered transforms:
    # ``extra["embed_transform"]`` is applied to the 32-bit stream right after the embedding gather (a scale,
    # a learned position added to it), ``extra["logit_transform"]`` to the 32-bit logits (a soft cap, a
    # scale).  Each transform reads its own constants from ``extra`` too.  None of the two by default.
    extra: dict = field(default_factory=dict)


# ---- mixers that carry a state from token to token, and layers built around them --------------------

@dataclass(frozen=True)
class LinearAttentionSpec:
    """Linear attention with one fixed decay a head: S = decay S + k v^T, o = S^T q, with q, k and v through
    silu; the read-out normalised over all heads together, times sigmoid(gate)."""
    kind: str = "lightning_attention"
    num_heads: int = 0
    head_dim: int = 0            # size of q and k a head
    value_dim: int = 0           # size of v a head
    decay: tuple = ()            # one a head
    eps: float = 1e-6


@dataclass(frozen=True)
class MlstmSpec:
    """A matrix memory a head with exponential input and forget gates, held stable by a running maximum."""
    kind: str = "mlstm"
    num_heads: int = 0
    head_dim: int = 0
    value_dim: int = 0
    gate_cap: float = 15.0       # the gates' pre-activations pass cap * tanh(x / cap)
    eps: float = 1e-6


@dataclass(frozen=True)
class GatedDeltaSpec:
    """The gated delta rule: S = g S; S += k (beta (v - S^T k))^T; o = S^T q, behind short convolutions."""
    kind: str = "gated_delta"
    num_heads: int = 0           # heads of v
    num_qk_heads: int = 0        # heads of q and k (divides num_heads)
    head_dim: int = 0
    value_dim: int = 0
    conv_taps: int = 4
    eps: float = 1e-6


@dataclass(frozen=True)
class ConvAttentionSpec:
    """Grouped-query softmax attention over a paged cache whose q, k and v pass a short causal convolution
    right behind their projections; value heads may have another size than query and key heads."""
    kind: str = "conv_attention"
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    value_dim: int = 0
    conv_taps: int = 1
    qk_norm_eps: Optional[float] = None     # None: no norm a head on q and k
    rotary_dim: int = 0                     # how many values of a head turn (0: none)
    rotary_base: float = 10000.0
    scale: Optional[float] = None           # None = 1/sqrt(head_dim)
    window: Optional[int] = None


@dataclass(frozen=True)
class ParallelMixersSpec:
    """Several mixers that read the same rows; their outputs are added with a weight each.
    ``branches``: ((tensor-name part, mixer spec, weight), ...)."""
    kind: str = "parallel_mixers"
    branches: tuple = ()


@dataclass(frozen=True)
class DenseMlpSpec:
    """down(act(up(x)))."""
    kind: str = "dense_mlp"
    intermediate_size: int = 0
    activation: str = "gelu_tanh"


# ---- attention with sinks, distance penalties and keys rebuilt from a small vector --------------------

@dataclass(frozen=True)
class SinkAttentionSpec:
    """Grouped-query softmax attention over a paged cache whose softmax has one more term in its denominator
    (a sink: a score without a key or a value), with optional extras: q and k divided by their root mean
    square over a head (no gain), a query temperature that grows with the logarithm of the position, a
    penalty a head on the distance between query and key, and a window."""
    kind: str = "sink_attention"
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    value_dim: int = 0
    scale: Optional[float] = None           # None = 1/sqrt(head_dim)
    qk_unit_eps: Optional[float] = None     # None: q and k are used as projected
    # q at position p times 1 + coef * ln(floor((p + 1) / every) + 1); None: no temperature
    temperature_coef: Optional[float] = None
    temperature_every: int = 1
    # score_ij -= slope_h (i - j); "geometric": slope_h = 2^(-slope_span (h + 1) / heads); None: no penalty
    distance_slopes: Optional[str] = None
    slope_span: float = 8.0
    window: Optional[int] = None            # keys j with i - window < j <= i; None: all keys up to i
    sink: Optional[str] = "zero"            # "zero": a sink of score 0; "learned": one a head (tensor ``sink``); None
    # "window": as above.  "block": positions are cut into blocks of ``window`` counted from position 0 of the
    # request, and a query sees the keys of its own block up to itself.
    mask: str = "window"
    qk_gain: bool = False                   # the unit q and k times a gain over the head (tensors ``q.norm``, ``k.norm``)
    qkv_bias: bool = False                  # q, k and v projections carry a bias each (``q.b``, ``k.b``, ``v.b``)


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values of all heads are rebuilt from one small vector a token (``kv_rank``
    values, normalised) and whose heads share one rotated key part of ``rotary_dim`` values: the pages hold
    those two and nothing else.  A query head is [head_dim values that are not rotated | rotary_dim rotated]."""
    kind: str = "latent_attention"
    num_heads: int = 0
    head_dim: int = 0                       # the unrotated part of a query/key head
    rotary_dim: int = 0                     # the rotated part, shared by the heads on the key side
    value_dim: int = 0
    kv_rank: int = 0
    rotary_turned: int = 0                  # how many values of the rotated part turn (pairs 2i, 2i + 1)
    rotary_base: float = 10000.0
    max_positions: int = 0                  # rows of the rotation's tables; 0: no tables, angles worked out in the kernel
    scale: Optional[float] = None           # None = 1/sqrt(head_dim + rotary_dim)
    norm_eps: float = 1e-6                  # of the norm on the small vector
    sink: Optional[str] = "learned"         # as in SinkAttentionSpec
    gated: bool = True                      # a head's read-out times sigmoid(gate projection of the layer's input)
    gate_each: str = "head"                 # one gate a "head" (tensor ``g`` [heads, width]) or an "element" ([heads * value_dim, width])
    window: Optional[int] = None
    borrows: bool = False                   # no projection onto the small vector: the schedule names the layer whose pages are read
    # the rotation's frequencies rescaled by wavelength: (factor, low, high, original), see ``TiedAttentionSpec``
    rotary_scaling: Optional[tuple] = None


# ---- several copies of the stream, experts chosen by a table ----------------------------------------

@dataclass(frozen=True)
class TableExpertsSpec:
    """``experts`` small gated feed-forwards, down(act(gate x) * (up x)), of which a token uses the ``top`` that
    a table names for its id (tensor ``table`` [vocabulary, top]); each of them counts 1/top."""
    kind: str = "table_experts"
    experts: int = 0
    top: int = 0
    intermediate_size: int = 0
    vocab_size: int = 0
    activation: str = "silu"


# ---- values that are the keys, a norm over all heads at once, experts behind a router ------------------

@dataclass(frozen=True)
class TiedAttentionSpec:
    """Grouped-query softmax attention over a paged cache without a value projection: a token's values are its keys
    as projected (bias included), before the keys are normed and turned.  q and k may carry biases; ``qk_norm_eps``
    norms q over ALL its heads at once (one root mean square over the whole projection, a gain a column, tensors
    ``q.norm`` and ``k.norm``) and k likewise; the first ``rotary_dims`` values of every head turn in pairs
    (2i, 2i + 1) by position * f_i, f_i = base^(-2i/dims).  ``rotary_scaling`` = (factor, low, high, original)
    rescales the frequencies by their wavelength l = 2 pi / f: kept where l < original / high, divided by factor
    where l > original / low, and between the two blended by s = (original / l - low) / (high - low)."""
    kind: str = "tied_attention"
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: Optional[float] = None           # None = 1/sqrt(head_dim)
    qk_bias: bool = False                   # tensors ``q.b`` and ``k.b``
    qk_norm_eps: Optional[float] = None     # None: q and k are used as projected
    rotary_dims: int = 0                    # 0: no rotation
    rotary_base: float = 10000.0
    rotary_scaling: Optional[tuple] = None
    window: Optional[int] = None            # the size of the window or of the blocks; None: every key up to the query
    mask: str = "window"                    # "window" or "block", as in SinkAttentionSpec


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """``experts`` small gated feed-forwards, down(act(gate x) * (up x)), and behind them ``identity`` experts whose
    output is their input, of which a token uses the ``top`` that a router chooses.  The router's logits (tensor
    ``router`` [experts + identity, width], 32-bit sums) pass ``score`` (softmax over all of them); the choice is by
    score plus ``correction`` (a tensor of that name, where ``corrected``); experts form ``groups`` equal groups of
    neighbours, a group counts by its best choice score, and only experts of the best ``groups_kept`` groups can be
    chosen (``groups`` 1: no groups).  A chosen expert weighs its score (without the correction), divided, where
    ``normalised``, by the chosen scores' sum plus ``weight_eps``."""
    kind: str = "routed_experts"
    experts: int = 0
    identity: int = 0
    top: int = 0
    intermediate_size: int = 0
    activation: str = "silu"
    score: str = "softmax"
    corrected: bool = True
    groups: int = 1
    groups_kept: int = 1
    normalised: bool = True
    weight_eps: float = 1e-20
