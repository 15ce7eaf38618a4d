"""A model as data: the specs that parts are built from.

A :class:`ModelSpec` is what an architecture's factory makes of its typed configuration.
It lists blocks (each a mixer, a feed-forward and their norms, every size a field), the
order in which blocks run (:class:`LayerCall`, a list that may name a block twice or let a
call read the cache of an earlier call) and the names of the tensors that fill them.
Nothing below this file knows which architecture it serves.

The reference keeps the same facts in ``ArchitectureSpec``
(``src/Inference/architecture_spec.jl:218-364``), per-layer mixer kinds in
``ShortConvSpec`` (``:169-178``) and position policy in ``RoPEPolicy`` (``:47-103``).

A spec of a new part is any frozen dataclass with a ``kind`` string; the part class
registered under that kind (``gesso_amd.parts.registry``) receives it unchanged.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


@dataclass(frozen=True)
class RMSNormSpec:
    """``x / sqrt(mean(x^2) + eps) * (offset + w)``: ``offset`` is what the stored weight lies around (0: the weight
    itself multiplies; 1: a weight stored around zero)."""

    size: int
    eps: float
    kind: str = "rmsnorm"
    offset: float = 0.0


@dataclass(frozen=True)
class LayerNormSpec:
    """``(x - mean(x)) / sqrt(var(x) + eps) * w + b``, the variance the mean of the squared deviations; ``bias``: whether
    there is a ``b``."""

    size: int
    eps: float
    bias: bool = True
    kind: str = "layernorm"


@dataclass(frozen=True)
class GroupRMSNormSpec:
    """RMS norm in parts: the row is cut into ``groups`` equal consecutive parts, each is divided by its own
    ``sqrt(mean(part^2) + eps)``, and the whole is multiplied by the weight."""

    size: int
    eps: float
    groups: int = 1
    kind: str = "group_rmsnorm"


@dataclass(frozen=True)
class RopeSpec:
    """Rotary encoding over the first ``rotary_dim`` features of a head; ``layout``: pairs ``(i, i + rotary_dim/2)``
    (``"half"``) or ``(2i, 2i + 1)`` (``"interleaved"``)."""

    head_dim: int
    rotary_dim: int
    theta: float
    max_position: int
    layout: str = "half"
    kind: str = "rope"
    frequency_divisor: float = 1.0     # every pair's frequency is divided by this (positions stretched evenly)


@dataclass(frozen=True)
class ScaledRopeSpec:
    """Rotary encoding whose slow pairs are slowed for contexts longer than the frequencies were chosen for.

    Pair ``i`` of ``rotary_dim / 2`` turns by ``f_i = theta^(-2i/rotary_dim)`` a position.  With
    ``pair_of(t) = rotary_dim ln(original / (2 pi t)) / (2 ln theta)`` (the pair that makes ``t`` turns over
    ``original`` positions), ``lo = max(floor(pair_of(fast)), 0)``, ``hi = min(ceil(pair_of(slow)), rotary_dim - 1)``
    and ``ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)`` the frequency becomes
    ``f_i / factor * ramp_i + f_i (1 - ramp_i)``, and cos and sin are both multiplied by
    ``amplitude_slope * ln(factor) + 1``.  ``factor = None``: plain rotation."""

    head_dim: int
    rotary_dim: int
    theta: float
    max_position: int
    factor: Optional[float] = None
    original: float = 0.0
    fast: float = 32.0
    slow: float = 1.0
    amplitude_slope: float = 0.1
    layout: str = "half"
    kind: str = "scaled_rope"


@dataclass(frozen=True)
class StretchedRopeSpec:
    """Rotary encoding whose frequencies are stretched by wavelength for contexts longer than ``original``.

    Pair ``i`` turns by ``f_i = theta^(-2i/rotary_dim)`` a position; with the wavelength ``l_i = 2 pi / f_i`` the pair
    keeps ``f_i`` where ``l_i < original / high``, gets ``f_i / factor`` where ``l_i > original / low``, and between the
    two, with ``s = (original / l_i - low) / (high - low)``, the blend ``(1 - s) f_i / factor + s f_i``.
    ``factor = None``: plain rotation."""

    head_dim: int
    rotary_dim: int
    theta: float
    max_position: int
    factor: Optional[float] = None
    original: float = 0.0
    low: float = 1.0
    high: float = 4.0
    layout: str = "half"
    kind: str = "stretched_rope"


@dataclass(frozen=True)
class NoPositionSpec:
    kind: str = "none"


@dataclass(frozen=True)
class AttentionSpec:
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: Any                      # a position-encoding spec
    qk_norm: Optional[RMSNormSpec]     # per-head norm of q and k before the rotation
    window: Optional[int] = None       # keys a query sees, itself included; None = all
    bias: bool = False
    scale: Optional[float] = None      # None = 1/sqrt(head_dim)
    kind: str = "attention"
    value_dim: Optional[int] = None    # width of a value head; None = head_dim
    chunk: Optional[int] = None        # positions are cut into runs of this many from 0 on, a query sees its own run
    sink: bool = False                 # the softmax's denominator has one more term, exp(0), which has no value
    value_position: Any = None         # a position-encoding spec: values are cached turned by their own position, a
                                       # head's weighted sum is turned back by the query's
    qk_norm_weight: bool = True        # False: the head norm of q and k has no weight (it may then stand after the
                                       # turn as well as before it: a turn keeps a head's sum of squares)
    out_bias: Optional[bool] = None    # whether the output projection has a bias (None: as ``bias``)
    softcap: Optional[float] = None    # scores become softcap * tanh(score / softcap)
    keep_first: int = 0                # with a window: the first positions of a sequence that stay visible beyond it
    head_sinks: bool = False           # the softmax's denominator has one more term exp(s_h), s_h a stored number a head
    out_gate: Optional[str] = None     # "sigmoid": the heads side by side are multiplied by sigmoid(W_g x) before the
                                       # output projection
    value_mix: bool = False            # the mixers that say so share values: the first of them to run in a step keeps
                                       # its values v_first, each later one caches (1 - m) v + m v_first, m a stored number


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention through low-rank bottlenecks: queries from a normed latent of ``q_rank`` features; keys and values
    of all heads from one normed latent row of ``kv_rank`` features per token, plus ``rot_dim`` rotated key features
    that all heads share.  A head has ``plain_dim`` unrotated and ``rot_dim`` rotated query/key features (in that
    order) and ``value_dim`` value features.  ``gated``: head ``h``'s output is multiplied by
    ``sigmoid(W_g x)[h]``; with ``gate_each`` every output feature has a gate of its own (``W_g`` has
    ``n_heads * value_dim`` rows).  ``position`` is the encoding of the ``rot_dim`` part (its ``head_dim`` = ``rot_dim``);
    its pairs may be laid out either way."""

    hidden: int
    n_heads: int
    plain_dim: int
    rot_dim: int
    value_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    eps: float                         # of the two latent norms
    position: Any
    window: Optional[int] = None       # keys a query sees, itself included; None = all
    gated: bool = True
    kind: str = "latent_attention"
    gate_each: bool = False


@dataclass(frozen=True)
class LinearAttentionSpec:
    """Attention without a softmax, through a matrix state per head that fades by a fixed factor a token:
    ``S_t = decay_h S_(t-1) + k_t v_t^T`` (``key_dim x value_dim``, float32, zero at a request's start),
    ``o_t = S_t^T q_t``.

    ``activation``: applied to the q, k and v products (``"silu"`` or None).  ``position``: turns q and k (a
    position-encoding spec).  ``key_scale``: multiplies k after the turn.  ``out_norm``: ``"joint"`` = the heads' outputs
    side by side are normed as one row with a weight, ``"head"`` = each head's output is divided by its own root mean
    square, no weight.  ``gate``: the normed row is multiplied by this function of a further product of the input
    (``"sigmoid"`` or ``"silu"``)."""

    hidden: int
    n_heads: int
    key_dim: int
    value_dim: int
    decay: Tuple[float, ...]
    eps: float
    position: Any = NoPositionSpec()
    activation: Optional[str] = None
    key_scale: float = 1.0
    out_norm: str = "joint"
    gate: str = "sigmoid"
    kind: str = "linear_attention"


@dataclass(frozen=True)
class GatedDeltaSpec:
    """The gated delta rule.  ``q, k`` (``qk_heads`` heads of ``key_dim``) and ``v`` (``n_heads`` of ``value_dim``) are
    products of the input that pass a causal convolution over time per channel (``conv_taps`` taps, no bias) and silu;
    q and k become unit vectors per head (``x / sqrt(sum(x^2) + unit_eps)``), q also times ``key_dim^-0.5``; head ``h``
    uses q/k head ``h // (n_heads / qk_heads)``.  ``beta = sigmoid(W_b x)`` and
    ``g = exp(-exp(A_log) softplus(W_a x + dt_bias))`` per head; ``S <- g S; u = beta (v - S^T k); S <- S + k u^T;
    o = S^T q``; each head's ``o`` is RMS-normed with a weight of ``value_dim``, times ``silu(W_g x)``, then projected."""

    hidden: int
    n_heads: int
    qk_heads: int
    key_dim: int
    value_dim: int
    conv_taps: int
    eps: float
    unit_eps: float = 1e-6
    kind: str = "gated_delta"


@dataclass(frozen=True)
class GatedLinearSpec:
    """Linear attention with a decay per key channel: ``alpha = sigmoid(W_up (W_down x) + b)^(1/tau)`` (the decay's
    product goes through ``decay_rank`` features), ``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``,
    ``o_t = S_t^T (q_t key_dim^-0.5)``; each head's ``o`` is RMS-normed with a weight of ``value_dim``, times
    ``silu(W_g x)``, then projected."""

    hidden: int
    n_heads: int
    key_dim: int
    value_dim: int
    decay_rank: int
    tau: float
    eps: float
    kind: str = "gated_linear"


@dataclass(frozen=True)
class MixerPairSpec:
    """Two mixers side by side that read the same input: ``left_scale * left(x) + right_scale * right(x)``.  Each keeps
    its own cache.  ``branch_norm_eps``: each side's output is first RMS-normed over the model width with a weight of
    its own (``left_norm.weight``, ``right_norm.weight``); None: the outputs as they are."""

    left: Any
    right: Any
    left_scale: float = 1.0
    right_scale: float = 1.0
    kind: str = "mixer_pair"
    branch_norm_eps: Optional[float] = None
    hidden: Optional[int] = None       # the model width (the branch norms' size)


@dataclass(frozen=True)
class ShortConvSpec:
    hidden: int
    width: int                         # taps, the current input included (conv_L_cache)
    bias: bool = False
    kind: str = "short_conv"


@dataclass(frozen=True)
class SwiGLUSpec:
    hidden: int
    intermediate: int
    kind: str = "swiglu"


@dataclass(frozen=True)
class GatedMLPSpec:
    """``W_down (act(W_gate x + b_gate) * (W_up x + b_up)) + b_down``; ``activation``: ``"gelu_tanh"``
    (``0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))``) or ``"silu"``; ``bias``: whether the three products have one."""

    hidden: int
    intermediate: int
    activation: str = "gelu_tanh"
    bias: bool = True
    kind: str = "gated_mlp"


@dataclass(frozen=True)
class ClampedGLUSpec:
    """``W_down (g sigmoid(alpha g) (u + 1))`` with ``g = min(W_gate x, limit)``, ``u = clamp(W_up x, -limit, limit)``;
    no biases."""

    hidden: int
    intermediate: int
    limit: float
    alpha: float = 1.702
    kind: str = "clamped_glu"


@dataclass(frozen=True)
class TableMoESpec:
    """A mixture of small feed-forwards whose routing is a table: token id ``v`` uses the ``top`` experts
    ``table[v, :]``, each with weight ``1 / top``.  An expert is ``W_down act(W_up x)``, ``act`` the square of relu.
    ``shared_ff``: a further expert of that width runs for every token, scaled by ``sigmoid(w_gate . x)`` when
    ``shared_gate`` (None: no shared expert)."""

    hidden: int
    vocab: int
    n_experts: int
    top: int
    expert_ff: int
    shared_ff: Optional[int] = None
    shared_gate: bool = True
    kind: str = "table_moe"


@dataclass(frozen=True)
class StateSpaceSpec:
    """A state-space mixer whose decay and step size depend on the token.  ``inner = n_heads * head_dim``; the input
    product gives ``[z: inner | x: inner | B: groups * state | C: groups * state | dt: n_heads]``; x, B and C pass a causal
    convolution of ``conv_taps`` taps per channel (with a bias) and silu; ``dt = softplus(dt + dt_bias)``; per head ``h``
    (group ``h // (n_heads / groups)``) ``S_t = exp(-exp(A_log[h]) dt_t) S_(t-1) + dt_t B_t x_t^T`` (``state x head_dim``,
    float32, zero at a request's start), ``y_t = S_t^T C_t + D[h] x_t``; ``y * silu(z)`` is RMS-normed in ``norm_groups``
    equal parts, times a weight, and projected back."""

    hidden: int
    n_heads: int
    head_dim: int
    state: int
    groups: int
    norm_groups: int
    conv_taps: int
    eps: float
    kind: str = "state_space"


@dataclass(frozen=True)
class RoutedMoESpec:
    """A mixture of gated feed-forwards chosen by a router over the token's features.  The router has
    ``n_experts + n_identity`` outputs; its scores are their softmax; the ``top`` outputs with the largest
    score + ``correction`` (a stored vector, when ``correction``) are chosen and weighted by their scores divided by the
    chosen scores' sum (+ 1e-20).  The last ``n_identity`` outputs name no weights: such an expert gives back its input.
    An expert is ``W_down (g sigmoid(alpha g) (u + 1))`` with ``g = min(W_gate x, limit)``,
    ``u = clamp(W_up x, -limit, limit)``.  ``shared_ff``: a further expert of that width and ``shared_limit`` runs for every
    token and is added (None: none).  ``score = "sigmoid"``: the scores are each output's sigmoid instead of their
    softmax; ``renormalize = False``: the weights are the chosen scores as they are; ``route_scale`` multiplies them."""

    hidden: int
    n_experts: int
    top: int
    expert_ff: int
    limit: float
    n_identity: int = 0
    alpha: float = 1.702
    correction: bool = True
    shared_ff: Optional[int] = None
    shared_limit: Optional[float] = None
    kind: str = "routed_moe"
    score: str = "softmax"
    renormalize: bool = True
    route_scale: float = 1.0


@dataclass(frozen=True)
class BlockSpec:
    """One block: ``h += mixer(norm(h)); h += ffn(norm(h))`` for ``arrangement="prenorm"``.

    ``names`` maps a part-local tensor name, prefixed by the part's role
    (``mixer.``, ``mixer_norm.``, ``ffn.``, ``ffn_norm.``), to the tensor's name in the
    weight file.
    """

    mixer: Any
    mixer_norm: Any
    ffn: Any                           # None = no feed-forward in this block
    ffn_norm: Any
    names: Mapping[str, str] = field(compare=False, hash=False, default_factory=dict)
    kind: str = "prenorm"


@dataclass(frozen=True)
class OutNormBlockSpec:
    """One block whose norms stand on the sub-layers' outputs: ``h += mult * norm_a(mixer(h));
    h += mult * norm_b(ffn(h))``; the sub-layers read ``h`` itself.  ``names`` as in :class:`BlockSpec`."""

    mixer: Any
    mixer_norm: Any
    ffn: Any                           # None = no feed-forward in this block
    ffn_norm: Any
    mult: float = 1.0
    names: Mapping[str, str] = field(compare=False, hash=False, default_factory=dict)
    kind: str = "outnorm"


@dataclass(frozen=True)
class ParallelBlockSpec:
    """One block whose sub-layers read the same stream: ``h += mixer(norm_a(h)) + ffn(norm_b(h))``.  ``names`` as in
    :class:`BlockSpec`."""

    mixer: Any
    mixer_norm: Any
    ffn: Any                           # None = no feed-forward in this block
    ffn_norm: Any
    names: Mapping[str, str] = field(compare=False, hash=False, default_factory=dict)
    kind: str = "parallel"


@dataclass(frozen=True)
class SharedNormBlockSpec:
    """One block with a single norm that both sub-layers read: with ``a = norm(h)``,
    ``h += mixer(a + conv(a)) + ffn(a)``.  ``input_taps``: the mixer's input gets a causal convolution over time added
    to it, ``conv(a)_t = sum_j w[:, j] a_(t - taps + 1 + j)`` per channel, no bias (None: the mixer reads ``a`` itself); its
    last ``taps - 1`` inputs are part of a request's state.  ``names`` as in :class:`BlockSpec` (roles ``norm.``,
    ``input_conv.``, ``mixer.``, ``ffn.``)."""

    mixer: Any
    norm: Any
    ffn: Any                           # None = no feed-forward in this block
    input_taps: Optional[int] = None
    names: Mapping[str, str] = field(compare=False, hash=False, default_factory=dict)
    kind: str = "shared_norm"


@dataclass(frozen=True)
class ReentrySpec:
    """Before the schedule entries ``at`` (in their order, ``t = 0, 1, ...``) the stream is mixed with the embedding
    output ``x0`` again: ``x <- W [x; x0] + step[t]`` with ``W (hidden, 2 hidden)`` (the stream's columns first) and
    ``step (len(at), hidden)``.  The model's names ``reentry.weight`` and ``reentry.step`` say where they are stored."""

    at: Tuple[int, ...]


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order: block ``layer`` runs here.

    ``cache`` is the position in the schedule of an earlier call whose cache this call
    reads instead of keeping its own (None = its own).
    """

    layer: int
    cache: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden: int
    vocab: int
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[LayerCall, ...]
    final_norm: Any
    tie_embeddings: bool
    max_position: int
    names: Mapping[str, str] = field(compare=False, hash=False, default_factory=dict)
    # names: "embed" -> table, "final_norm.weight" -> ..., "head" -> untied head
    eos_token_ids: Tuple[int, ...] = ()
    ignored_tensors: Tuple[str, ...] = ()   # suffixes that a file may hold and nobody reads
    embed_scale: Optional[float] = None     # the embedding rows are multiplied by this (None: as they are)
    embed_norm: Any = None                  # a norm spec: the embedding rows are normed before the first block
                                            # (its tensors under names "embed_norm.<local>")
    logit_softcap: Optional[float] = None   # logits = cap * tanh(logits / cap) (None: as they are)
    reentry: Optional[ReentrySpec] = None   # see :class:`ReentrySpec`

    def __post_init__(self):
        n = len(self.blocks)
        for i, call in enumerate(self.schedule):
            if not 0 <= call.layer < n:
                raise ValueError(f"schedule entry {i} names block {call.layer}, there are {n}")
            if call.cache is not None and not 0 <= call.cache < i:
                raise ValueError(f"schedule entry {i} reads the cache of entry {call.cache}, which does not run before it")
        if self.reentry is not None:
            at = tuple(self.reentry.at)
            if not at or list(at) != sorted(set(at)) or not 0 <= at[0] <= at[-1] < len(self.schedule):
                raise ValueError(f"re-entry points {at} must be distinct schedule entries in ascending order")
