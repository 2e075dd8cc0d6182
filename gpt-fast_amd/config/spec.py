"""Descriptions of a model as data: what each layer is made of and in which order
layers run.

An architecture's configuration (read from its ``config.json``) is turned into a
:class:`ModelPlan` by that architecture's ``plan`` function.  Everything below the
plan (parts, cache, step function, generation) reads only the plan, never the
architecture's name.  Every size and constant a part needs is a field of its spec.

A spec's ``kind`` selects the part class in the registries of ``parts``; a test or an
application can define a new spec class with a new ``kind`` and register a part for it.
"""
from dataclasses import dataclass
from typing import List, Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last dimension (reference model.py:230-241).
    ``weight_offset`` is added to the stored weight before it is used: 0 for weights stored
    around one, 1 for weights stored around zero (``x / rms * (1 + w)``).
    kind "rms": a weight per element.  kind "rms_scalar": one stored number for all elements.
    kind "none": no norm at all; the rows are only handed on in the compute type (a sublayer
    that reads the residual stream itself).
    kind "layer": the layer norm with a weight and no bias, ``(x - mean) / sqrt(var + eps) * w``
    with the variance as the mean of the squared deviations."""
    dim: int
    eps: float
    kind: str = "rms"
    weight_offset: float = 0.0


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.

    kind "rope": rotate pairs of the first ``rotary_dim`` elements of each query and
    key head by ``position * frequency[i]`` (reference model.py:266-293).  ``layout``
    is "interleaved" (pairs (2i, 2i+1), the reference's) or "half" (pairs
    (i, i + rotary_dim/2)).  ``scaling`` is None or a dict with ``rope_type`` and that
    rule's constants (reference model.py:244-263 for "llama3"; "linear" divides every
    frequency by ``factor``; "yarn" divides the slow end of the ladder by ``factor`` along a
    ramp between two wavelengths and multiplies cos and sin by ``0.1 ln(factor) + 1``, see
    ``parts.position.yarn_scaled``).
    kind "none": no position information is added.
    kind "learned": a table of ``max_positions`` learned rows of ``dim`` elements; row p is
    added to the embedded row of the token at position p (a plan's ``input_position``).
    """
    kind: str = "rope"
    rotary_dim: int = 0
    base: float = 10000.0
    layout: str = "interleaved"
    scaling: Optional[Tuple[Tuple[str, object], ...]] = None   # dict items, hashable
    dim: int = 0                  # "learned": the rows' width
    max_positions: int = 0        # "learned": the table's rows

    def scaling_dict(self) -> Optional[dict]:
        return None if self.scaling is None else dict(self.scaling)


@dataclass(frozen=True)
class AttentionSpec:
    """Causal attention with grouped key/value heads over the cache
    (reference model.py:167-216).  ``window`` None means every earlier key is read;
    an integer W means keys at distance < W only."""
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: PositionSpec
    scale: Optional[float] = None          # None: 1/sqrt(head_dim)
    window: Optional[int] = None
    kind: str = "attention"


@dataclass(frozen=True)
class DifferentialAttentionSpec:
    """Causal attention whose heads each hold ``n_maps`` = 2 softmax maps over the same
    values: query and key rows lie head by head as [map 1, map 2], each map ``head_dim``
    wide, values ``value_dim`` wide.  A head's result is ``a1 - lam * a2`` with
    ``lam = exp(lq1 . lk1) - exp(lq2 . lk2) + lam_init`` (four learned vectors of
    ``head_dim``), divided by its root mean square over ``value_dim`` (``eps`` inside the
    root), times ``1 - lam_init``, times a sigmoid gate per head if ``head_gate``.
    ``window`` W: keys at distance < W; ``keep_first`` F: the keys at positions < F stay
    visible beyond the window, at their true positions.  Position i sees j if
    ``j <= i and (i - j < W or j < F)``."""
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    value_dim: int
    position: PositionSpec
    lam_init: float
    eps: float
    scale: Optional[float] = None          # None: 1/sqrt(head_dim)
    window: Optional[int] = None
    keep_first: int = 0
    head_gate: bool = True
    kind: str = "differential_attention"


@dataclass(frozen=True)
class NormedAttentionSpec:
    """Causal attention with grouped key/value heads whose queries and keys are RMS-normed per
    head (``qk_norm_eps`` inside the root) and multiplied by a weight of ``head_dim`` elements
    that all heads share (one for q, one for k), before they are rotated.  ``position`` rotates
    the first ``position.rotary_dim`` elements of every head (any layout and scaling of
    ``PositionSpec``).  score = (q . k) * scale, then ``softcap tanh(score / softcap)`` if
    ``softcap``; ``window`` W: keys at distance < W only; ordinary softmax; values of
    ``value_dim``."""
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    value_dim: int
    position: PositionSpec
    scale: float
    qk_norm_eps: Optional[float] = None
    softcap: Optional[float] = None
    window: Optional[int] = None
    kind: str = "normed_attention"


@dataclass(frozen=True)
class GatedDeltaSpec:
    """Recurrent mixer with the gated delta rule.  q and k have ``n_kv_heads`` heads of
    ``key_dim``, v ``n_heads`` heads of ``value_dim``; head h of v uses head
    ``h // (n_heads / n_kv_heads)`` of q and k.  Each channel of q, k and v passes a causal
    convolution over ``conv_taps`` tokens (no bias, zeros before the start) and silu; q and k
    become unit vectors per head (``x / sqrt(sum(x^2) + unit_eps)``), q times
    ``key_dim^-1/2``; ``beta = sigmoid(w_b x)``, ``g = exp(-exp(A_log) softplus(w_a x +
    dt_bias))`` per head; per head a float32 state ``S [key_dim, value_dim]``, zero at a
    sequence's start: ``S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q``.  Each head's
    o is divided by its root mean square (``eps``), times a weight of ``value_dim`` elements that
    the heads share, times silu of a gate projection, then projected out.  The convolutions'
    last ``conv_taps - 1`` inputs are part of the sequence's state."""
    dim: int
    n_heads: int
    n_kv_heads: int
    key_dim: int
    value_dim: int
    conv_taps: int
    eps: float
    unit_eps: float = 1e-6
    kind: str = "gated_delta"


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Several mixers side by side that read the same input: ``branches`` = ((name, spec), ...),
    each any mixer spec.  The result is the mean of the branches' results, each first divided
    by its root mean square over the model width (``eps`` inside the root) and multiplied by a
    weight per element of its own (parameter ``<name>_out``).  Each branch keeps its own cache
    (``cache.store.JointNeed``); a branch's parameters are named ``<name>.<parameter>``."""
    dim: int
    branches: Tuple[Tuple[str, object], ...]
    eps: float
    kind: str = "parallel"


@dataclass(frozen=True)
class MatrixMemorySpec:
    """Recurrent mixer with a matrix memory per head (the mLSTM cell of xLSTM): state
    ``S [key_dim, value_dim]``, normaliser ``n [key_dim]`` and a running maximum ``m`` of the
    log gates, all float32 and zero at a sequence's start.  With log input gate
    ``i = cap tanh(. / cap)``, log forget gate ``f = logsigmoid(cap tanh(. / cap))``:
    ``m' = max(f + m, i)``, ``S' = exp(f + m - m') S + exp(i - m') k v^T``, n likewise with k,
    ``o = S'^T q / (max(|n' . q|, exp(-m')) + den_eps)``; each head's o is divided by its root
    mean square (``eps``), times a weight per element, times sigmoid of a gate projection,
    then projected out.  ``gate_cap`` None leaves the gates' pre-activations uncapped."""
    dim: int
    n_heads: int
    key_dim: int
    value_dim: int
    eps: float
    gate_cap: Optional[float] = None
    den_eps: float = 1e-6
    kind: str = "matrix_memory"


@dataclass(frozen=True)
class MixedHeadsAttentionSpec:
    """Causal attention with grouped key/value heads whose scores are mixed across heads before
    the softmax.  Projections of q, k, v and the output have biases if ``biases``; q and k are
    divided by their root mean square over ``head_dim`` per head (``qk_norm_eps``; None: not
    normed); then, for query i, key j <= i and head g,

        s_g = (q_g . k_j) * scale * temperature[g]          (a learned number per head)
        s_g = softcap * tanh(s_g / softcap)                 (if ``softcap``)
        s_g = s_g + table[bucket(i - j), g]                 (if ``bias_rows``)
        score_h = sum_g talk[h, g] s_g                      (if ``mix_heads``)

    and head h's softmax over j weighs the values of kv head ``h // (H / G)``.  The distance
    table has ``bias_rows`` rows: with ``half = bias_rows // 2``, distance n < half has its own
    row n; further distances share rows in logarithmic steps,
    ``half + floor(ln(n / half) / ln(bias_max / half) * (bias_rows - half))``, the last row
    taking everything beyond."""
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    value_dim: int
    scale: float
    softcap: Optional[float] = None
    bias_rows: int = 0
    bias_max: float = 0.0
    qk_norm_eps: Optional[float] = None
    head_temperature: bool = True
    mix_heads: bool = True
    biases: bool = True
    kind: str = "mixed_heads_attention"


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values are expanded from one latent vector per token.  The
    query goes through a latent of ``q_rank`` with an RMS norm, then up to ``n_heads`` heads of
    ``head_dim`` plain and ``rot_dim`` rotated elements; one projection gives the token's
    latent of ``kv_rank`` (RMS-normed) and one rotated key part of ``rot_dim`` that all heads
    share; a head's plain key is ``w_uk`` of the latent, its value ``w_uv`` of it
    (``value_dim``).  score = (q_plain . k_plain + q_rot . k_rot) * scale.  ``position``
    rotates the first ``position.rotary_dim`` elements of the rotated parts.  ``window`` W:
    keys at distance < W only.  The cache holds the latent and the rotated key part.
    ``q_rank`` None: the query has no latent, one projection takes x straight to the heads.
    ``rot_dim`` 0: no rotated part."""
    dim: int
    n_heads: int
    head_dim: int
    rot_dim: int
    value_dim: int
    q_rank: Optional[int]
    kv_rank: int
    scale: float
    eps: float
    position: PositionSpec
    window: Optional[int] = None
    kind: str = "latent_attention"


@dataclass(frozen=True)
class SinkAttentionSpec:
    """Causal attention with grouped key/value heads, no rotation, and these steps, each of
    which a field switches:

    * ``biases``: the projections of q and k have biases;
    * ``values_are_keys``: there is no value projection, a kv head's value is its key as
      projected (bias added, before any norm), so ``value_dim == head_dim``;
    * ``whole_norm_eps``: q and k are each divided by the root mean square of the WHOLE
      projection (all heads at once, before the split) and multiplied by a weight per element
      (None: not normed);
    * ``q_temp_coef``, ``q_temp_every``: the query at position p is multiplied by
      ``1 + coef * ln(floor((p + 1) / every) + 1)`` (coef None: not);
    * ``log_distance_bias``: ``r1[h] * ln(1 + r2[h] * (i - j))`` is taken off the score of
      query i and key j <= i, with two learned numbers per head;
    * ``sink``: the softmax's denominator has one more term exp(0): a key of score zero that
      carries no value.

    score = (q . k) * scale, before the bias."""
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    value_dim: int
    scale: float
    biases: bool = True
    values_are_keys: bool = True
    whole_norm_eps: Optional[float] = None
    q_temp_coef: Optional[float] = None
    q_temp_every: int = 1
    log_distance_bias: bool = True
    sink: bool = True
    kind: str = "sink_attention"


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """A mixture of ``n_experts`` small feed-forwards without biases, ``w_down act(w_up x)`` or,
    if ``gated``, ``w_down (act(w_gate x) * (w_up x))``, of which each token uses ``top``.
    Router: ``z = w_router x`` and the scores ``s = softmax(z)`` over all experts, or
    ``sigmoid(z)`` (``scoring``), in float32.  The choice is made on ``s`` plus, with
    ``choice_correction``, a stored number per expert (the weights never see it).  The experts
    form ``n_groups`` equal groups of neighbours; a group's score is the sum of its
    ``group_top`` largest choice scores (1: its largest); only experts of the ``keep_groups``
    best groups can be chosen (the others count as minus infinity), and of those the ``top``
    with the largest choice scores are.  Their weights are their ``s`` over the sum of the
    chosen ``s`` (plus ``weight_eps``).  ``shared_hidden`` > 0: one more expert of that inner
    size and the same form runs for every token, with weight one or, with ``shared_gate``,
    ``sigmoid(w_sg x)`` (one number per token)."""
    dim: int
    n_experts: int
    top: int
    hidden: int
    n_groups: int = 1
    keep_groups: int = 1
    shared_hidden: int = 0
    activation: str = "gelu"
    weight_eps: float = 1e-20
    scoring: str = "softmax"
    choice_correction: bool = False
    group_top: int = 1
    gated: bool = False
    shared_gate: bool = False
    kind: str = "routed_experts"


@dataclass(frozen=True)
class PairEmbeddingSpec:
    """An embedding of the pair (previous token, token), added to a token's embedded row: row
    ``(previous * mul_prev + token * mul_cur) mod buckets`` of a table of ``buckets + 1`` rows;
    a sequence's first token takes the last row.  The previous token of a step's first token
    is part of the sequence's state."""
    dim: int
    buckets: int
    mul_prev: int
    mul_cur: int
    name: str = "pair_embedding"
    kind: str = "pair_embedding"


@dataclass(frozen=True)
class DecayedMemorySpec:
    """Linear attention with a fixed decay per head (lightning attention, retention): q, k
    (``key_dim``) and v (``value_dim``) are ``activation`` ("silu", or None: nothing) of their
    projections; ``position`` (a rope ``PositionSpec``, or None) then rotates q and k, and k is
    multiplied by ``key_scale``; per head a float32 state ``S [key_dim, value_dim]``, zero at a
    sequence's start: ``S' = decay_h S + k v^T``, ``o = S'^T q``.  The heads' results are
    divided by their root mean square (``eps``) - ``norm`` "row": all heads side by side as one
    row; "head": every head by itself - times a weight per element if ``norm_weight``, times
    ``gate`` ("sigmoid" or "silu") of a gate projection, and projected out."""
    dim: int
    n_heads: int
    key_dim: int
    value_dim: int
    decay: Tuple[float, ...]
    eps: float
    activation: Optional[str] = "silu"
    position: Optional[PositionSpec] = None
    key_scale: float = 1.0
    norm: str = "row"
    norm_weight: bool = True
    gate: str = "sigmoid"
    kind: str = "decayed_memory"


@dataclass(frozen=True)
class DenseFeedForwardSpec:
    """``w_down( act(w_up x) )`` without biases.  ``activation`` "xielu": with two learned
    numbers p, q (the parameter ``act``): z > 0: ``softplus(p) z^2 + z/2``; z <= 0:
    ``(1/2 + softplus(q)) (exp(z) - 1 - z) + z/2``.  Others: "silu", "gelu_tanh" (no
    parameter)."""
    dim: int
    hidden: int
    activation: str = "xielu"
    kind: str = "dense"


@dataclass(frozen=True)
class InputMixSpec:
    """A step on the residual stream that stands before a run: ``x <- W [x; x0]`` with
    ``W [dim, 2 dim]`` (the columns for x first) and x0 the embedded rows of the step's tokens.
    ``name`` is the tensor's name; runs that name the same spec share the matrix."""
    dim: int
    name: str
    kind: str = "input_mix"


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """w2( act(w1 x) * (w3 x) ) without biases (reference model.py:219-227); ``activation``
    "silu" or "gelu_tanh"."""
    dim: int
    hidden: int
    activation: str = "silu"
    kind: str = "gated"


@dataclass(frozen=True)
class LayerSpec:
    """One block.  ``arrangement`` names how norms, mixer, feed-forward and the residual
    stream are wired ("pre_norm": reference model.py:161-164).  ``name`` is the prefix of
    the layer's tensors.  Parameter sub-names are those of the arrangement.  A block whose
    ``feed_forward`` is None has the mixer's sublayer only.  In the "post_norm" arrangement
    the norm stands after the sum, ``x <- out_norm(residual_scale * x + ls * sublayer(read(x)))``:
    ``mixer_norm`` / ``feed_forward_norm`` say how a sublayer reads the stream (kind "none": the
    stream itself), ``mixer_out_norm`` / ``feed_forward_out_norm`` are the norms of the sums, and
    ``layer_scale`` gives each sublayer's result a stored weight per element ``ls``."""
    name: str
    mixer: object
    mixer_norm: NormSpec
    feed_forward: object = None
    feed_forward_norm: Optional[NormSpec] = None
    arrangement: str = "pre_norm"
    mixer_name: str = "mixer"
    mixer_norm_name: str = "mixer_norm"
    feed_forward_name: str = "feed_forward"
    feed_forward_norm_name: str = "feed_forward_norm"
    # "sandwich_norm": a second norm on each sublayer's result, before it joins the stream
    mixer_out_norm: Optional[NormSpec] = None
    feed_forward_out_norm: Optional[NormSpec] = None
    mixer_out_norm_name: str = "mixer_out_norm"
    feed_forward_out_norm_name: str = "feed_forward_out_norm"
    # "sandwich_norm" with ``result_gate``: each sublayer's result is multiplied, element by
    # element and before its out norm, by sigmoid(W h + b), h being what the sublayer reads
    result_gate: bool = False
    mixer_gate_name: str = "mixer_gate"
    feed_forward_gate_name: str = "feed_forward_gate"
    # "post_norm": the stream's factor in the sum, and a weight per element on each result
    residual_scale: float = 1.0
    layer_scale: bool = False
    mixer_scale_name: str = "mixer_scale"
    feed_forward_scale_name: str = "feed_forward_scale"


@dataclass(frozen=True)
class Run:
    """One entry of the order in which layers run.  ``layer`` indexes
    ``ModelPlan.layers``; a layer may be named by several entries (its weights are then
    used more than once).  ``cache`` names the cache entry the mixer reads and writes;
    it defaults to an entry of this run's own.  A run with ``cache_from`` = index of an
    earlier run reads that run's cache and writes nothing.  ``enter`` is the spec of a step on
    the residual stream that stands before this run (``InputMixSpec``), or None."""
    layer: int
    cache_from: Optional[int] = None
    enter: object = None


@dataclass
class ModelPlan:
    """A whole decoder: embedding, layers in run order, final norm, output head.
    ``max_positions`` bounds prompt + new tokens of a generated request."""
    dim: int
    vocab_size: int
    layers: List[LayerSpec]
    order: List[Run]
    final_norm: NormSpec
    tie_embeddings: bool = False
    max_positions: int = 2048
    embedding_name: str = "tok_embeddings.weight"
    final_norm_name: str = "norm"               # prefix of the final norm's tensors ("norm.weight")
    head_name: str = "output.weight"
    stop_tokens: Tuple[int, ...] = ()
    # Optional steps around the layers; None leaves the step out (the reference has none
    # of them, model.py:136-146).
    embedding_scale: Optional[float] = None     # embedded rows are multiplied by this
    input_position: object = None               # a position spec whose part adds to the embedded
    input_position_name: str = "input_position"  # rows (``add_to_stream``); prefix of its tensors
    # further parts that add to the embedded rows (``PairEmbeddingSpec``); each may keep state
    # per sequence in a cache entry of its own
    input_adds: Tuple[object, ...] = ()
    logit_scale: Optional[float] = None         # logits are multiplied by this,
    logit_softcap: Optional[float] = None       # then capped: cap * tanh(logits / cap)

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model plan needs at least one layer")
        for n, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"order[{n}] names layer {run.layer}, "
                                 f"but there are {len(self.layers)} layers")
            if run.cache_from is not None:
                if not 0 <= run.cache_from < n:
                    raise ValueError(f"order[{n}].cache_from={run.cache_from} must name "
                                     f"an earlier entry of the order")
                if self.order[run.cache_from].cache_from is not None:
                    raise ValueError(f"order[{n}].cache_from={run.cache_from} names an "
                                     f"entry that itself borrows a cache")
