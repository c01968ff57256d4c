"""Typed descriptions of the parts a model is assembled from.

A model configuration (see ``gpt2.py``) turns the keys of its ``config.json`` into these
records: one :class:`LayerSpec` per layer and a run order (:class:`LayerCall` list).  The
parts in ``deliverance_amd.parts`` are built from the records alone, so a part never
learns which model it sits in, and two layers of one model may carry different mixers
and feed-forwards.

The reference keeps the same facts as fields of one flat ``Config`` object
(safetensors/src/main/java/io/teknek/deliverance/safetensors/Config.java:315-377) and as
constructor arguments of its block classes
(core/src/main/java/io/teknek/deliverance/generator/TransformerBlock.java:26-41).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot describe a model (missing key, bad value)."""


@dataclass(frozen=True)
class NormSpec:
    """``kind == "layernorm"``: mean and variance, gain and optional bias.  ``kind == "rmsnorm"``: the row
    divided by its root mean square (eps inside the root) times ``gain_offset + weight``; a gain that is
    stored around zero has ``gain_offset`` 1.  Others are added through ``parts.register_norm``."""
    kind: str
    width: int
    eps: float
    bias: bool = True
    gain_offset: float = 0.0


@dataclass(frozen=True)
class PositionSpec:
    """Where a token's position enters the model.

    ``kind == "learned"``: a table of ``max_positions`` rows is added to the token
    embedding.  ``kind == "none"``: nothing.  Other kinds may act on queries and keys
    inside an attention mixer (see ``parts.positions``).
    """
    kind: str
    max_positions: int = 0
    params: Tuple[Tuple[str, float], ...] = ()


@dataclass(frozen=True)
class DistanceBiasSpec:
    """A learned value per head that is added to a score by the distance n = i - j >= 0 between query and
    key (after the scale; the scale does not multiply it).  The table has ``n_buckets`` rows: distances
    below ``n_buckets // 2`` have a row each, larger ones share rows in steps that grow like a logarithm
    up to ``max_distance``, from where the last row is used:

        half = n_buckets // 2
        bucket(n) = n                                                            for n < half
                  = min(n_buckets - 1,
                        half + floor(ln(n / half) / ln(max_distance / half) * (n_buckets - half)))   else
    """
    n_buckets: int
    max_distance: int


@dataclass(frozen=True)
class QueryTemperatureSpec:
    """Queries at position p are multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``: scores sharpen
    as a sequence grows, in steps of ``every`` positions."""
    coef: float
    every: int


@dataclass(frozen=True)
class QKNormSpec:
    """Queries and keys pass a root-mean-square norm with a plain gain (eps inside the root) before positions
    act on them.  ``whole``: one norm over all of a token's query entries and one over all of its key entries,
    before they are split into heads, with gains of those lengths; else one norm a head with a gain of
    ``head_dim`` entries that the heads share."""
    eps: float
    whole: bool = True


@dataclass(frozen=True)
class AttentionSpec:
    kind: str            # "attention"
    width: int           # model width E
    n_heads: int
    n_kv_heads: int
    head_dim: int        # per-head size of queries and keys
    scale: float         # multiplies q.k before the softmax
    qkv_bias: bool = True
    out_bias: bool = True
    window: Optional[int] = None     # None: every earlier key; w: the last w keys
    position: Optional[PositionSpec] = None  # acts on q and k (none for learned tables)
    v_head_dim: Optional[int] = None         # per-head size of values; None: head_dim
    distance_bias: Optional[DistanceBiasSpec] = None
    query_temperature: Optional[QueryTemperatureSpec] = None
    qk_norm: Optional["QKNormSpec"] = None   # queries and keys normalised before any rotation
    score_softcap: float = 0.0               # positive: score <- cap * tanh(score / cap), after the scale
    keep_first: int = 0                      # with a window: the first keys of a sequence stay visible for good
    # the values are the keys as projected, before any rotation: there is no value matrix (v_head_dim = head_dim)
    values_are_keys: bool = False
    # one more term in the softmax's denominator that has no value: None, "zero" (exp(0) = 1) or "learned"
    # (exp(sink_h), a parameter ``sink`` per query head; not multiplied by the scale)
    sink: Optional[str] = None
    # the heads' results are multiplied, element by element, with this function of one more projection of the
    # mixer's input before the output projection: None or "sigmoid" (parameter ``gate_weight`` [heads * value size, width])
    out_gate: Optional[str] = None

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim


@dataclass(frozen=True)
class RampedSpeedsSpec:
    """Slower turns for long contexts.  With place(t) = dims * ln(original / (2 pi t)) / (2 ln base),
    lo = max(floor(place(fast)), 0) and hi = min(ceil(place(slow)), dims - 1), pair i keeps its speed where
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) is 0 and turns ``factor`` times slower where it is 1:
    speed_i <- speed_i / factor * ramp_i + speed_i * (1 - ramp_i).  Sine and cosine are multiplied by
    0.1 ln(factor) + 1."""
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class RotarySpec:
    """Pairs of the first ``dims`` entries of a query or key vector are turned by the angle position * speed_i,
    speed_i = base^(-2i / dims), i = 0 .. dims / 2 - 1; entries behind ``dims`` pass.  ``interleaved``: pair i is
    (2i, 2i + 1), else (i, i + dims / 2).  (u, v) becomes (u cos a - v sin a, v cos a + u sin a).  ``scaling``
    changes the speeds and the length of the turned pairs (``RampedSpeedsSpec``)."""
    kind: str            # "rotary"
    dims: int
    base: float
    interleaved: bool = True
    scaling: Optional[RampedSpeedsSpec] = None


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values are linear maps of one narrow normalised vector a token.

    The mixer's input h goes down to [ query latent (q_rank) | latent (kv_rank) | key piece (rot_dim) ].  Both
    latents pass a root-mean-square norm with a gain (``norm_eps``).  Queries are ``up_q`` of the query latent:
    per head ``head_dim`` entries that meet the head's keys ``up_k`` of the latent, and ``rot_dim`` entries that are
    turned by the position and meet the turned key piece, which all heads share.  Values are ``up_v`` of the latent,
    ``v_head_dim`` a head.  The cache keeps the latent and the turned key piece, nothing per head."""
    kind: str            # "latent_attention"
    width: int
    n_heads: int
    head_dim: int        # unrotated entries of a head's queries and keys
    rot_dim: int         # rotated entries (a head's queries; one shared key piece)
    v_head_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    norm_eps: float
    rotary: RotarySpec
    window: Optional[int] = None
    # a learned number per head (parameter ``sink``) whose exponential joins the softmax's denominator: it has no
    # key and no value and is not multiplied by the scale
    sink: bool = False


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with a fixed decay per head and neither softmax nor denominator.  Per head a matrix S
    (``head_dim`` x ``v_head_dim``, 32-bit) is carried from token to token: S <- decay_h S + k v^T, o = S^T q.
    q and k are turned by the position (``rotary``) and k is then multiplied by head_dim^-1/2.  Each head's o is
    divided by its root mean square (``norm_eps``, no gain), the heads are multiplied by ``gate`` ("silu") of one
    more projection and projected back to the width."""
    kind: str            # "retention"
    width: int
    n_heads: int
    head_dim: int
    v_head_dim: int
    decay: Tuple[float, ...]
    norm_eps: float
    rotary: Optional[RotarySpec] = None
    gate: str = "silu"


@dataclass(frozen=True)
class SelectiveScanSpec:
    """A selective state-space mixer: the input goes up to [ x | z ] of ``inner`` channels each; x passes a causal
    filter of ``conv_taps`` taps per channel and SiLU; from x come a step size per channel (through ``dt_rank``
    numbers, a matrix, a bias and softplus) and two vectors B, C of ``state`` entries; per channel c and state
    index j, S[c, j] <- exp(dt_c A[c, j]) S[c, j] + dt_c x_c B_j with A = -exp(A_log), y_c = sum_j S[c, j] C_j + D_c x_c;
    the output is the down-projection of y * silu(z).  The state (S and the filter's last inputs) is 32-bit."""
    kind: str            # "selective_scan"
    width: int
    inner: int
    state: int
    dt_rank: int
    conv_taps: int


@dataclass(frozen=True)
class DeltaRuleSpec:
    """A gated delta-rule mixer.  Per value head a matrix S (``head_dim`` x ``v_head_dim``, 32-bit) is carried from
    token to token: S <- g * S (a decay in (0, 1) for every row of S), u = beta * (v - S^T k), S <- S + k u^T,
    o = S^T q.  q and k (``n_kv_heads`` of them, shared by groups of value heads) and v come from projections
    followed by a short causal filter of ``conv_taps`` taps a channel and SiLU; q and k are scaled to unit length per
    head (``unit_eps`` under the root) and q by head_dim^-1/2.  beta = logistic of a projection, one a head.
    The decay is exp(-exp(A_log) * softplus(a + dt_bias)) with one ``A_log`` a head and a projection a that has one
    entry a head (``decay == "head"``) or one a head and key channel (``"channel"``); ``decay_rank`` > 0: that
    projection is two matrices with so many numbers in between.  o is divided by its root mean square per head
    (``norm_eps``), multiplied by a gain shared by the heads and by ``gate`` ("silu" | "sigmoid") of one more
    projection (two matrices when ``gate_rank`` > 0), and projected back to the width."""
    kind: str            # "delta_rule"
    width: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    v_head_dim: int
    conv_taps: int
    norm_eps: float
    decay: str = "head"
    decay_rank: int = 0
    gate: str = "silu"
    gate_rank: int = 0
    unit_eps: float = 1e-6


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Several mixers that read the same input; the result is sum_k scales[k] * branches[k](h).  Every branch keeps
    a cache slot of its own: branch k of a layer call with slot c uses slot c + k."""
    kind: str            # "parallel"
    branches: Tuple[object, ...]
    scales: Tuple[float, ...]


@dataclass(frozen=True)
class DenseFeedForwardSpec:
    kind: str            # "dense"
    width: int
    inner: int
    activation: str      # "gelu_new" | "gelu" | "gelu_pytorch_tanh" | "relu" | "silu" | "relu2"
    bias: bool = True


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """``down(act(gate h) * (up h))``, no biases.  The activation "glu_capped" takes ``limit``: with
    g = min(gate h, limit) and u = clamp(up h, -limit, limit) the middle is g * logistic(1.702 g) * (u + 1)."""
    kind: str            # "gated"
    width: int
    inner: int
    activation: str
    limit: float = 0.0


@dataclass(frozen=True)
class ExpertsFeedForwardSpec:
    """``n_experts`` feed-forwards of ``inner`` columns, of which every token uses ``top``; the output is the
    weighted sum of theirs.  ``router == "token_table"``: a table [vocab, top] of integers names each token id's
    experts (a row's entries differ), each with weight 1 / top.  ``router == "logistic_top"``: a matrix
    [n_experts, width] gives 32-bit logits z; the ``top`` experts with the largest logistic(z) are used, with those
    scores as weights (``renormalize``: divided by their sum).  ``gated``: an expert is down(act(gate h) * (up h)),
    else down(act(up h)).  ``weight_on``: "output" (weight * expert(h)) or "input" (expert(weight * h)).
    ``router == "softmax_top"``: logits z = matrix h + bias (32-bit); the ``top`` largest logits are used (the lower
    index wins a tie), with the softmax over just those as weights.
    ``shared_inner`` > 0: one more feed-forward of that many columns runs for every token with weight 1 and is
    added; it is ungated, or (``shared_gated``) of the gated form with ``shared_limit``.  ``limit``: the constant of
    the activation "glu_capped" (``GatedFeedForwardSpec``)."""
    kind: str            # "experts"
    width: int
    inner: int
    n_experts: int
    top: int
    activation: str
    router: str = "token_table"
    vocab_size: int = 0
    gated: bool = True
    weight_on: str = "output"
    renormalize: bool = False
    shared_inner: int = 0
    shared_activation: Optional[str] = None
    limit: float = 0.0
    shared_gated: bool = False
    shared_limit: float = 0.0
    router_bias: bool = False


@dataclass(frozen=True)
class LayerSpec:
    """One block: ``x += mixer(norm1(x)); x += ff(norm2(x))`` with optional norm slots.

    The reference's block has five optional norm places
    (core/.../generator/TransformerBlock.java:26-32); the pre-norm pair is what its
    GPT-2 uses (TransformerBlock.java:35-41).  ``post_block_norm`` is the fifth (applied to
    the stream when both parts have joined it, TransformerBlock.java:199);
    ``residual_multiplier`` scales a part's output (after the norm behind it, if any) before
    it joins the stream (TransformerBlock.java:260-272; 1: plain addition).
    """
    mixer: object
    feed_forward: object
    pre_mixer_norm: Optional[NormSpec] = None
    post_mixer_norm: Optional[NormSpec] = None
    pre_ff_norm: Optional[NormSpec] = None
    post_ff_norm: Optional[NormSpec] = None
    weight_prefix: str = ""
    post_block_norm: Optional[NormSpec] = None
    residual_multiplier: float = 1.0
    # a learned vector of the model's width that multiplies the mixer's / the feed-forward's result, element by
    # element, after the norm behind it and before it joins the stream (parameters "mixer_scale", "ff_scale")
    mixer_scale: bool = False
    ff_scale: bool = False


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.

    ``layer`` indexes ``ModelConfig.layers`` (a layer may be named twice), ``cache`` is
    the cache slot its mixer uses, and ``write`` is False when the mixer only reads a
    slot that another call has filled in the same step.  ``mix_input``: right before this
    call the stream becomes W [stream; embedding output] (``ModelConfig.input_mix``).
    """
    layer: int
    cache: int
    write: bool = True
    mix_input: bool = False


@dataclass(frozen=True)
class ModelConfig:
    """What every architecture's typed configuration provides to the engine."""
    architecture: str
    vocab_size: int
    width: int
    max_positions: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[LayerCall, ...]
    embed_position: PositionSpec
    final_norm: Optional[NormSpec]
    tie_word_embeddings: bool
    bos_token_id: Optional[int]
    eos_token_ids: Tuple[int, ...]
    raw: dict = field(default_factory=dict, compare=False, hash=False)
    embed_scale: float = 1.0        # multiplies the token embedding before positions are added
    # logits are divided by it (the reference's logitMultiplier, AbstractGeneratorSampler.java:117-120)
    logit_multiplier: float = 1.0
    # logits <- cap * tanh(logits / cap) when positive
    logit_softcap: float = 0.0
    # a norm on the embedded tokens before the first layer (parameters "embed_norm")
    embed_norm: Optional[NormSpec] = None
    # a matrix [width, 2 width] (parameter "input_mix") that run-order entries with ``mix_input`` apply to the
    # stream beside the embedding output (the stream's half first)
    input_mix: bool = False

    @property
    def n_cache_slots(self) -> int:
        def slots(mixer):
            return len(mixer.branches) if isinstance(mixer, ParallelMixerSpec) else 1
        return max((c.cache + slots(self.layers[c.layer].mixer) for c in self.schedule), default=0)
