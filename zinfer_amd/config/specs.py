"""Specifications of the parts a model is put together from.

A specification is plain data: every size and constant a part needs, nothing about the model
it ends up in.  The reference describes a layer the same way, as a ``Spec`` of sizes plus a
``LayerLayout`` of optional slots (`src/model/layers/rmsnorm_gqa_swiglu_block.zig:10-51`) and
an ``AttentionSpec`` (`src/model/layers/gqa_attention/spec.zig:3-26`); here each slot is a
specification of its own so that layers of one model may differ.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Tuple


@dataclass(frozen=True)
class RmsNormSpec:
    """n = x * w / sqrt(mean(x^2) + eps) over ``width`` elements."""
    width: int
    eps: float


@dataclass(frozen=True)
class LayerNormSpec:
    """n = (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b over ``width`` elements;
    ``centred`` False leaves the mean in (an RMS norm with a bias).  The gain is the tensor
    ``prefix + weight_name``, the bias ``prefix + bias_name`` (None: no bias)."""
    width: int
    eps: float
    centred: bool = True
    weight_name: str = "weight"
    bias_name: Optional[str] = "bias"
    gain_offset: float = 0.0               # the gain is this plus the stored weight


@dataclass(frozen=True)
class RotaryHalfSplitSpec:
    """Rotation of the pairs (i, i + head_dim/2) by position * theta^(-2i/head_dim)."""
    head_dim: int
    theta: float
    max_positions: int


@dataclass(frozen=True)
class NoPositionSpec:
    """No position encoding inside the mixer."""


@dataclass(frozen=True)
class GqaAttentionSpec:
    """Causal grouped-query attention.  ``window`` None = every earlier key; an integer =
    only the last ``window`` positions (the query's own included)."""
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    qk_norm_eps: Optional[float]          # None: no per-head norm of q and k
    position: object                       # a position-encoding specification
    window: Optional[int] = None
    scale: Optional[float] = None          # None: 1/sqrt(head_dim)


@dataclass(frozen=True)
class TiedKeyValueAttentionSpec:
    """Causal grouped-query attention whose values are its keys as projected (there is no
    value projection, and the cache holds keys only), without a position encoding.
    ``window`` as in ``GqaAttentionSpec``.  ``sink``: the soft-max's denominator holds one more
    term of score 0 that brings no value.  ``output_gate``: the concatenated heads are
    multiplied by sigmoid(W_g h), h being the input the projections read, before the output
    projection.  The ``*_name`` fields are the tensor names below the mixer's prefix."""
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    scale: Optional[float] = None          # None: 1/sqrt(head_dim)
    window: Optional[int] = None
    sink: bool = False
    output_gate: bool = False
    q_name: str = "q_proj.weight"
    k_name: str = "k_proj.weight"
    gate_name: str = "g_proj.weight"
    o_name: str = "o_proj.weight"


@dataclass(frozen=True)
class LeadingRotarySpec:
    """Rotation of the first ``dims`` elements of a head (the rest pass unchanged) in the pairs
    (i, i + dims/2) by the angle position * frequencies[i]; cosine and sine are multiplied by
    ``magnitude``.  The frequencies are plain data, so that any rule for them (a base alone,
    wavelengths slowed beyond a length, a ramp between two turn counts) gives the same part;
    ``config.rotary`` holds the rules.  There is no table of positions: the angle is formed
    from the position where it is used, in 32-bit.  ``interleaved``: the pairs are the
    neighbours (2i, 2i + 1) instead, pair i turning by frequencies[i]."""
    dims: int
    frequencies: Tuple[float, ...]
    magnitude: float = 1.0
    interleaved: bool = False


@dataclass(frozen=True)
class MaskedGqaAttentionSpec:
    """Causal grouped-query attention with separate key and value sizes and these options:
    ``qk_norm_eps``: an RMS norm over the whole q projection and one over the whole k projection
    (all heads at once) with gains of those sizes, before the rotation; ``rotary``: a
    ``LeadingRotarySpec`` or None; ``softcap``: scores become cap * tanh(score / cap);
    ``window`` (the last ``window`` positions) and ``chunk`` (only keys of the query's own
    chunk of that many positions, counted from position 0); ``sink``: one learned number a head
    whose exponential joins the soft-max's denominator; ``head_gate``: head h's output is
    multiplied by sigmoid(W_g h)_h, one number a head.  ``qk_norm_per_head``: the norm of q and
    of k runs over every head on its own instead, with one gain of ``head_dim`` for all heads.
    ``bias``: q, k and v have biases (``bias_suffix`` behind the matrix's name), added before
    the norm.  The ``*_name`` fields are the tensor names below the mixer's prefix."""
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    value_dim: int
    scale: float
    qk_norm_eps: Optional[float] = None
    qk_norm_per_head: bool = False
    bias: bool = False
    bias_suffix: str = ".b"
    rotary: Optional[LeadingRotarySpec] = None
    softcap: Optional[float] = None
    window: Optional[int] = None
    chunk: Optional[int] = None
    sink: bool = False
    head_gate: bool = False
    q_name: str = "q_proj.weight"
    k_name: str = "k_proj.weight"
    v_name: str = "v_proj.weight"
    o_name: str = "o_proj.weight"
    q_norm_name: str = "q_norm.weight"
    k_norm_name: str = "k_norm.weight"
    sink_name: str = "sinks"
    gate_name: str = "g_proj.weight"


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values come from one latent row a token: q = W_uq N(W_dq h)
    laid out head by head as [head_dim plain | rot_dim rotated]; W_dkv h = [latent of kv_rank,
    normed | rot_dim, not normed, rotated: one key part shared by all heads]; per head the
    plain key is W_uk latent and the value W_uv latent; the score is scale * (q_plain . k_plain
    + q_rot . k_rot).  The cache holds the latent and the rotated part only.  ``window`` /
    ``chunk`` as in ``MaskedGqaAttentionSpec``; ``element_gate``: the concatenated heads are
    multiplied by sigmoid(W_g h) before the output projection; ``head_gate``: head h's output
    is multiplied by sigmoid(W_g h)_h, one number a head (W_g is then [heads, hidden]).
    ``q_rank`` None: no query latent, q = W_q h with the matrix ``uq_name`` [heads * (head_dim +
    rot_dim), hidden].  ``rot_dim`` 0: no rotated part, the key is the latent alone."""
    hidden_size: int
    n_heads: int
    head_dim: int
    rot_dim: int
    value_dim: int
    q_rank: Optional[int]
    kv_rank: int
    scale: float
    norm_eps: float
    rotary: Optional[LeadingRotarySpec] = None
    window: Optional[int] = None
    chunk: Optional[int] = None
    element_gate: bool = False
    head_gate: bool = False
    dq_name: str = "q_a_proj.weight"
    dq_norm_name: str = "q_a_layernorm.weight"
    uq_name: str = "q_b_proj.weight"
    dkv_name: str = "kv_a_proj_with_mqa.weight"
    dkv_norm_name: str = "kv_a_layernorm.weight"
    uk_name: str = "k_b_proj.weight"
    uv_name: str = "v_b_proj.weight"
    gate_name: str = "g_proj.weight"
    o_name: str = "o_proj.weight"


@dataclass(frozen=True)
class DenseMlpSpec:
    """down(act(up(x))), no gate: ``activation`` is "gelu" (the exact form with erf),
    "gelu_tanh", "silu" or "relu2" (the square of max(x, 0))."""
    hidden_size: int
    intermediate_size: int
    activation: str = "gelu"
    up_name: str = "up_proj.weight"
    down_name: str = "down_proj.weight"


@dataclass(frozen=True)
class GatedLinearAttentionSpec:
    """A mixer whose memory is one matrix a head, S [head_dim, value_dim], carried from token to
    token in 32-bit: S_t = diag(a_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with
    q = W_q h * ``q_scale`` (None: head_dim^(-1/2)), k = W_k h, v = W_v h and a decay a key
    channel a_t = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau) through a narrow middle of ``decay_rank``.
    Each head's o goes through an RMS norm over value_dim with one gain for all heads, the heads
    side by side are multiplied by silu(W_g h), then W_o.  The ``*_name`` fields are the tensor
    names below the mixer's prefix."""
    hidden_size: int
    n_heads: int
    head_dim: int
    value_dim: int
    decay_rank: Optional[int]          # None: whatever the tensors hold
    tau: float
    norm_eps: float
    q_scale: Optional[float] = None
    q_name: str = "q"
    k_name: str = "k"
    v_name: str = "v"
    gate_name: str = "g"
    o_name: str = "o"
    norm_name: str = "norm"
    decay_down_name: str = "a1"
    decay_up_name: str = "a2"
    decay_bias_name: str = "a2.b"


@dataclass(frozen=True)
class TokenShiftRecurrenceSpec:
    """A mixer of the same kind whose inputs are blends of a token's row with the row before it:
    m_s = h + (h_prev - h) * mu_s for s in r, k, v, g, w (h_prev zero for a sequence's first
    token; the last row is part of the state).  r, k, v = W_s m_s (heads of ``head_dim``),
    gate = silu(W_g m_g), decay w = exp(-exp(W_w2 tanh(W_w1 m_w) + w0)) a head and key channel.
    o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t with a learned u [heads, head_dim] for the token's
    own outer product; then S_t = diag(w_t) S_(t-1) + k_t v_t^T.  Each head's o is divided by its
    root mean square; the heads side by side are multiplied by a gain [heads * head_dim] and the
    gate, then W_o.  The ``*_name`` fields are the tensor names below the mixer's prefix
    (``mix_name.format(s)`` for the blends' coefficients)."""
    hidden_size: int
    n_heads: int
    head_dim: int
    decay_rank: Optional[int]          # None: whatever the tensors hold
    norm_eps: float
    r_name: str = "r"
    k_name: str = "k"
    v_name: str = "v"
    gate_name: str = "g"
    o_name: str = "o"
    norm_name: str = "norm"
    bonus_name: str = "u"
    decay_down_name: str = "w1"
    decay_up_name: str = "w2"
    decay_bias_name: str = "w0"
    mix_name: str = "mu.{}"


@dataclass(frozen=True)
class GatedDeltaRuleSpec:
    """A mixer whose memory is one matrix a head, S [head_dim, value_dim], carried from token to
    token in 32-bit and corrected towards every token's value: S <- g_t S; w = beta_t (v_t -
    S^T k_t); S <- S + k_t w^T; o_t = S^T q_t.  q and k (``n_kv_heads`` heads of ``head_dim``)
    and v (``n_heads`` heads of ``value_dim``; value head n reads q/k head floor(n / (n_heads /
    n_kv_heads))) each pass a causal convolution over time a channel (``conv_taps`` taps, the
    last one the token's own, zeros before a sequence's start; the taps - 1 rows before a step
    are part of the state) and silu; q and k then become unit vectors a head, x / sqrt(sum x^2 +
    ``unit_eps``), and q is multiplied by ``q_scale`` (None: head_dim^(-1/2)).  One decay and one
    step size a head and token: g = exp(-exp(A) softplus(W_a h + dt)), beta = sigmoid(W_b h).
    Each head's o goes through an RMS norm over value_dim with one gain for all heads, the heads
    side by side are multiplied by silu(W_g h), then W_o.  The ``*_name`` fields are the tensor
    names below the mixer's prefix (``conv_suffix`` behind a matrix's name: its taps)."""
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    value_dim: int
    conv_taps: int
    norm_eps: float
    unit_eps: float = 1e-6
    q_scale: Optional[float] = None
    q_name: str = "q"
    k_name: str = "k"
    v_name: str = "v"
    conv_suffix: str = ".conv"
    beta_name: str = "b"
    decay_name: str = "a"
    decay_log_name: str = "A_log"
    decay_bias_name: str = "dt_bias"
    gate_name: str = "g"
    norm_name: str = "norm"
    o_name: str = "o"


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers side by side that read the same input: ``left_scale`` * left(h) +
    ``right_scale`` * right(h).  Each has its own tensors (below ``left_prefix`` and
    ``right_prefix``) and its own cache or state."""
    left: object
    right: object
    left_scale: float = 1.0
    right_scale: float = 1.0
    left_prefix: str = "left."
    right_prefix: str = "right."


@dataclass(frozen=True)
class PlainExpertSpec:
    """down(act(up(x))), no gate and no bias; ``activation`` as in ``DenseMlpSpec``."""
    intermediate_size: int
    activation: str = "relu2"


@dataclass(frozen=True)
class GatedExpertSpec:
    """down(act(gate(x), up(x))) with g = min(gate, limit), u = clamp(up, -limit, limit)
    (``limit`` None: neither is clamped) and act = g * sigmoid(alpha * g) * (u + shift)."""
    intermediate_size: int
    limit: Optional[float] = None
    alpha: float = 1.0
    shift: float = 0.0


@dataclass(frozen=True)
class MoeSpec:
    """Of ``n_experts`` experts every token uses the ``top_k`` whose router logits
    z = W_r x (+ b_r) are largest, weighted by the soft-max over those logits alone; an
    optional ``shared`` expert runs for every token with weight 1.  ``scoring`` "sigmoid"
    instead: the scores are s = sigmoid(z), the choice goes by s plus a learned correction
    [n_experts] (``correction_name``; None: none) that does not enter the weights, and the
    weights are the chosen experts' s over their sum (+ 1e-20); with ``groups`` = (count, keep)
    the experts form ``count`` equal groups of neighbours, a group is marked by the sum of its
    two largest choice scores, and only experts of the ``keep`` best groups can be chosen.
    ``scoring`` "softmax_all": as "sigmoid" with s = softmax(z) over all the router's outputs.
    ``group_mark``: how many of a group's largest choice scores make its mark (2 or 1).
    ``normalize`` False: the weights are the chosen s themselves; either way they are
    multiplied by ``weight_scale``.  ``n_identity``: the router has that many outputs more
    than there are experts; one of them, chosen, stands for an expert without tensors whose
    output is its input (times the weight); they count as experts in groups and choice.
    ``shared_gate_name``: the shared expert's output is multiplied by sigmoid(w . x), one
    number a token, w being that tensor [1, hidden] below ``shared_prefix``.
    ``expert`` is a ``GatedExpertSpec`` or a ``PlainExpertSpec`` (no gate matrix).  Tensor names
    below the part's prefix: the router's matrix and bias, ``expert_prefix.format(e)`` and
    ``shared_prefix`` followed by the matrices' names."""
    hidden_size: int
    n_experts: int
    top_k: int
    expert: object
    shared: Optional[GatedExpertSpec] = None
    router_bias: bool = False
    scoring: str = "softmax"
    correction_name: Optional[str] = None
    groups: Optional[Tuple[int, int]] = None
    group_mark: int = 2
    normalize: bool = True
    weight_scale: float = 1.0
    n_identity: int = 0
    shared_gate_name: Optional[str] = None
    router_name: str = "gate.weight"
    router_bias_name: str = "gate.bias"
    expert_prefix: str = "experts.{}."
    shared_prefix: str = "shared_expert."
    gate_name: str = "gate_proj.weight"
    up_name: str = "up_proj.weight"
    down_name: str = "down_proj.weight"


@dataclass(frozen=True)
class SwiGluSpec:
    """down(silu(gate(x)) * up(x)); the ``*_name`` fields are the tensor names below the
    part's prefix."""
    hidden_size: int
    intermediate_size: int
    gate_name: str = "gate_proj.weight"
    up_name: str = "up_proj.weight"
    down_name: str = "down_proj.weight"


@dataclass(frozen=True)
class PreNormBlockSpec:
    """x += mixer(norm1(x)); x += ff(norm2(x)).  ``mixer_prefix`` and the other prefixes are
    the tensor-name prefixes below the layer's own prefix."""
    mixer: object
    feed_forward: object
    mixer_norm: object
    ff_norm: object
    mixer_prefix: str = "self_attn."
    ff_prefix: str = "mlp."
    mixer_norm_prefix: str = "input_layernorm."
    ff_norm_prefix: str = "post_attention_layernorm."


@dataclass(frozen=True)
class SandwichNormBlockSpec:
    """x += post1(mixer(norm1(x))); x += post2(ff(norm2(x))): every sublayer has a norm before
    it and one after it, ahead of the residual sum.  ``feed_forward`` None: the layer is its
    mixer alone (and declares neither ``ff_norm`` nor ``ff_post_norm``)."""
    mixer: object
    feed_forward: Optional[object]
    mixer_norm: object
    mixer_post_norm: object
    ff_norm: Optional[object] = None
    ff_post_norm: Optional[object] = None
    mixer_prefix: str = "self_attn."
    ff_prefix: str = "mlp."
    mixer_norm_prefix: str = "input_layernorm."
    mixer_post_norm_prefix: str = "post_attention_layernorm."
    ff_norm_prefix: str = "pre_feedforward_layernorm."
    ff_post_norm_prefix: str = "post_feedforward_layernorm."


@dataclass(frozen=True)
class PostNormBlockSpec:
    """x += norm1(mixer(x)); x += norm2(ff(x)): the sublayers read the stream as it is, and the
    only norms stand behind them, ahead of the residual sums.  ``feed_forward`` None: the layer
    is its first line (and declares no ``ff_post_norm``)."""
    mixer: object
    feed_forward: Optional[object]
    mixer_post_norm: object
    ff_post_norm: Optional[object] = None
    mixer_prefix: str = "self_attn."
    ff_prefix: str = "mlp."
    mixer_post_norm_prefix: str = "post_attention_layernorm."
    ff_post_norm_prefix: str = "post_feedforward_layernorm."


@dataclass(frozen=True)
class ParallelBlockSpec:
    """x += mixer(norm1(x)) + ff(norm2(x)): both sublayers read the same x, each through a norm
    of its own.  ``feed_forward`` None: the layer is its mixer alone (and declares no
    ``ff_norm``)."""
    mixer: object
    feed_forward: Optional[object]
    mixer_norm: object
    ff_norm: Optional[object] = None
    mixer_prefix: str = "self_attn."
    ff_prefix: str = "mlp."
    mixer_norm_prefix: str = "input_layernorm."
    ff_norm_prefix: str = "post_attention_layernorm."


@dataclass(frozen=True)
class StreamBlockSpec:
    """A layer over ``streams`` copies X_1 .. X_S of the residual stream instead of one.  For
    each sublayer c (the mixer, then the feed-forward if there is one): u = sum_s a_c[s] X_s;
    y = sublayer_c(norm_c(u)); X_t <- sum_s M_c[s, t] X_s + b_c[t] y for all t at once from the
    old X.  a_c [S], M_c [S, S] (indexed [from, to]) and b_c [S] are the tensors
    ``coef_prefix.format(c) + in_name | mix_name | out_name`` below the layer's prefix;
    ``learned`` False: there are no such tensors, a = b = 1 and M the identity (with one
    stream that is the plain pre-norm layer x += sublayer(norm(x)))."""
    streams: int
    mixer: object
    feed_forward: Optional[object]
    mixer_norm: object
    ff_norm: Optional[object] = None
    learned: bool = True
    mixer_prefix: str = "mix."
    ff_prefix: str = "mlp."
    mixer_norm_prefix: str = "norm1"
    ff_norm_prefix: str = "norm2"
    coef_prefix: str = "hc{}."
    in_name: str = "in"
    mix_name: str = "mix"
    out_name: str = "out"


@dataclass(frozen=True)
class SinusoidalPositionSpec:
    """A position vector added to the embedding row, formed from the position where it is used:
    entry 2i is sin(p * f_i), entry 2i + 1 cos(p * f_i), f_i = base^(-2i / width)."""
    base: float = 10000.0


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named
    twice); ``cache_of`` None gives this run a cache of its own, an integer makes it read
    the cache that the run at that earlier schedule position writes.  ``reentry``: before this
    run the stream is replaced by W [x ; x0], x0 being the stream as the embedding left it and W
    the model's ``reentry_name`` tensor [hidden, 2 hidden] (a pass over looped layers begins)."""
    layer: int
    cache_of: Optional[int] = None
    reentry: bool = False


@dataclass(frozen=True)
class ModelSpec:
    """Everything the generic decoder needs: sizes, one block specification per layer, the
    order the layers run in, and tensor names."""
    vocab_size: int
    hidden_size: int
    max_positions: int
    layers: Tuple[object, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    tie_word_embeddings: bool
    embed_name: str = "model.embed_tokens.weight"
    final_norm_prefix: str = "model.norm."
    head_name: str = "lm_head.weight"
    layer_prefix: str = "model.layers.{}."
    eos_token_ids: Tuple[int, ...] = ()
    default_stop_sequences: Tuple[str, ...] = ()
    embedding_multiplier: float = 1.0       # the embedding row times this enters the stream
    logit_scale: float = 1.0                # logits = head(x) * logit_scale ...
    logit_softcap: Optional[float] = None   # ... then cap * tanh(logits / cap) if given
    # a learned position table [max_positions, hidden]: its row at a token's position is added
    # to the embedding row (not scaled); None: positions enter through the mixers only
    position_table_name: Optional[str] = None
    # a position vector computed from the position and added to the embedding row
    sinusoidal_positions: Optional[SinusoidalPositionSpec] = None
    # the matrix [hidden, 2 hidden] of the schedule entries that say ``reentry``
    reentry_name: Optional[str] = None
    # the residual stream in that many copies [streams, T, hidden], all equal to the embedding's
    # output at the start and added up before the final norm (the blocks are ``StreamBlockSpec``
    # layers); None: the one stream [T, hidden]
    streams: Optional[int] = None
    # the number each of ``layers`` goes by in ``layer_prefix`` (None: its index): a model whose
    # file numbers all runs while some of them bring no tensors of their own
    layer_numbers: Optional[Tuple[int, ...]] = None
