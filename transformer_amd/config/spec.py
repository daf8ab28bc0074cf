"""Architecture-neutral descriptions of a decoder, as plain data.

A model is a list of blocks plus a schedule. Every block names its parts
(norms, mixer, feed-forward) with all their sizes and constants, so two
blocks of one model may differ in any of them. The schedule is the order in
which blocks run; it may name a block twice or let a run read the cache that
an earlier run wrote.

Each spec class carries a ``kind`` string. ``transformer_amd.parts.registry``
maps that string to the class that executes it, so a new part is a new spec
class plus a registered executor; nothing in this file changes.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A configuration that cannot be built; the message names the key."""


@dataclass(frozen=True)
class NormSpec:
    size: int
    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class PositionSpec:
    """Rotation of (q, k) pairs by position * theta^(-2j/head_dim).

    style "half" pairs element j with j + head_dim/2, "interleaved" pairs 2j
    with 2j + 1. kind "none" leaves q and k as they are.
    """
    head_dim: int
    theta: float = 10000.0
    style: str = "half"
    kind: str = "rope"
    # (factor, low, high, original) or None: frequencies whose wavelength exceeds original/low
    # are divided by factor, those below original/high stay, and between the two the share of
    # the unscaled frequency grows linearly in original/wavelength from 0 to 1
    scaling: Optional[Tuple[float, float, float, float]] = None
    # (factor, original, fast, slow) or None: another way to slow the long wavelengths, a ramp over
    # the pair index i. n(t) = head_dim * ln(original / (2 pi t)) / (2 ln theta) is the index at
    # which t turns fit into ``original`` positions; lo = max(floor(n(fast)), 0), hi = min(ceil(n(slow)),
    # head_dim - 1), r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1), and f_i <- f_i / factor * r_i +
    # f_i * (1 - r_i). ``scaling`` and ``ramp`` exclude each other.
    ramp: Optional[Tuple[float, float, float, float]] = None
    magnitude: float = 1.0      # cos and sin are both multiplied by it


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over the per-sequence key/value cache.

    window: a query at position p reads keys in (p - window, p]; None = all.
    """
    hidden: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    position: PositionSpec
    window: Optional[int] = None
    qkv_bias: bool = False
    out_bias: bool = False
    kind: str = "attention"


@dataclass(frozen=True)
class SwiGLUSpec:
    hidden: int
    intermediate: int
    bias: bool = False
    kind: str = "swiglu"


@dataclass(frozen=True)
class BlockSpec:
    """x += mixer(norm1(x)); x += ffn(norm2(x))  (kind "prenorm"). ffn None (and norm2 None): the
    block has the mixer only."""
    norm1: object
    mixer: object
    norm2: object = None
    ffn: object = None
    kind: str = "prenorm"


@dataclass(frozen=True)
class RunSpec:
    """One entry of the schedule.

    block: index into ModelSpec.blocks.
    cache_of: None = this run owns a cache layer of its own (if its mixer
    needs one); an int names an EARLIER schedule entry whose cache layer this
    run reads instead of writing one.
    """
    block: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    vocab: int
    hidden: int
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[RunSpec, ...]
    final_norm: object
    tie_embeddings: Optional[bool] = None  # None: decided by the weight file
    max_position: Optional[int] = None
    stop_ids: Tuple[int, ...] = field(default_factory=tuple)
    # Optional parts around the blocks, for architectures that scale or shift the embedded
    # rows or transform the logits: specs of registered kinds whose executors offer
    # ``run(t, ctx)`` and change the float32 tensor in place ([nt, hidden] after the
    # embedding, [wanted, vocab] for the logits). The Llama decoder has neither.
    after_embed: object = None
    on_logits: object = None

    def validate(self) -> None:
        if self.vocab <= 0 or self.hidden <= 0:
            raise ConfigError("vocab and hidden must be positive")
        if not self.blocks or not self.schedule:
            raise ConfigError("a model needs at least one block and one schedule entry")
        for i, run in enumerate(self.schedule):
            if not 0 <= run.block < len(self.blocks):
                raise ConfigError(f"schedule[{i}] names block {run.block}, "
                                  f"model has {len(self.blocks)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < i:
                    raise ConfigError(f"schedule[{i}].cache_of={run.cache_of} must name an "
                                      f"earlier schedule entry")
                if self.schedule[run.cache_of].cache_of is not None:
                    raise ConfigError(f"schedule[{i}].cache_of={run.cache_of} names an entry "
                                      f"that itself borrows a cache")


# ---------------------------------------------------------------------------------------------
# Parts beyond the Llama decoder's. Each is usable by any architecture: its sizes and constants
# are fields, and the executor of its ``kind`` is registered in ``transformer_amd.parts``.

@dataclass(frozen=True)
class ScalarNormSpec:
    """RMS norm whose gain is ONE number for all coordinates (the file holds a 0-d tensor)."""
    size: int
    eps: float
    kind: str = "rmsnorm_scalar"


@dataclass(frozen=True)
class GLUSpec:
    """down(act(gate(h)) * up(h)); activation "silu" or "gelu_tanh"."""
    hidden: int
    intermediate: int
    activation: str = "silu"
    bias: bool = False
    kind: str = "glu"


@dataclass(frozen=True)
class PairHashEmbedSpec:
    """Added to the embedded rows: row (previous token * mul_prev + token * mul_cur) mod
    buckets of a second table, and row ``buckets`` (the last) for a sequence's first token."""
    hidden: int
    buckets: int
    mul_prev: int
    mul_cur: int
    kind: str = "pair_hash_embed"


@dataclass(frozen=True)
class LogitScaleSpec:
    """logits *= scale."""
    scale: float
    kind: str = "logit_scale"


@dataclass(frozen=True)
class NormedAttentionSpec:
    """Causal grouped-query softmax attention whose keys and values have widths of their own.

    qk_norm: q and k are RMS-normed over their whole projection (all heads at once) with a
    weight per coordinate, before the rotation. rot_dims: the first coordinates of every head
    that are rotated, in pairs (i, i + rot_dims/2), by position * rot_base^(-2i/rot_dims); 0 =
    no rotation. value_mix: None; "source" = this mixer's values are kept for the step;
    "mix" = v <- (1 - lambda) v + lambda * (the source's values of the same token), lambda a
    learned number, and the mixed v is what the cache holds. qk_norm_per_head: every head of q
    and of k is normed on its own, with ONE weight of the head's width for all heads of q and one
    for those of k. rot_scaling: see ``PositionSpec.scaling``."""
    hidden: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    eps: float
    qk_norm: bool = True
    rot_dims: int = 0
    rot_base: float = 10000.0
    value_mix: Optional[str] = None
    window: Optional[int] = None
    kind: str = "attention_normed"
    qk_norm_per_head: bool = False
    rot_scaling: Optional[Tuple[float, float, float, float]] = None


@dataclass(frozen=True)
class DiagonalRecurrenceSpec:
    """Two branches of ``channels``: y = gelu_tanh(Wy h + b) and u = causal conv of ``taps``
    over (Wx h + b); gates r, i = sigmoid of block-diagonal maps of u (``blocks`` blocks);
    a = exp(-decay_scale * r * softplus(lam)); S <- a S + sqrt(1 - a^2) * i * u; out = Wo (S * y).
    State per sequence: S and the last taps - 1 inputs of the convolution."""
    hidden: int
    channels: int
    blocks: int
    taps: int
    decay_scale: float = 8.0
    kind: str = "diagonal_recurrence"


@dataclass(frozen=True)
class GatedLinearAttentionSpec:
    """Per head a matrix state S [key_dim, value_dim]: S <- diag(alpha) S + k v^T, o = S^T q,
    q scaled by key_dim^-1/2, alpha = sigmoid(W2 (W1 h) + b)^(1/tau) per key channel (W1 maps
    to ``rank`` numbers); o is RMS-normed per head, gated by silu(Wg h) and projected."""
    hidden: int
    num_heads: int
    key_dim: int
    value_dim: int
    rank: int
    tau: float
    eps: float
    kind: str = "gated_linear_attention"


@dataclass(frozen=True)
class GatedBlockSpec:
    """x += mult * gate1 * mixer(shift(norm1(x))); x += mult * gate2 * ffn(norm2(x)).

    gated: each sublayer's result is multiplied by sigmoid(W h + b), h the normed input of the
    sublayer (before the shift). token_shift: the mixer reads h_t + (h_{t-1} - h_t) * mu with
    a learned mu per coordinate; h_{t-1} is the unshifted row of the previous token (zeros
    before the first) and is carried between steps. ffn None: the block has one sublayer."""
    norm1: object
    mixer: object
    norm2: object = None
    ffn: object = None
    hidden: int = 0
    mult: float = 1.0
    gated: bool = True
    token_shift: bool = True
    kind: str = "gated_prenorm"


# ---------------------------------------------------------------------------------------------
# Parts that the Kunitar decoder added; as above, every size and constant is a field.

@dataclass(frozen=True)
class EmbedScaleSpec:
    """An ``after_embed`` part: the embedded rows are multiplied by ``scale``."""
    scale: float
    kind: str = "embed_scale"


@dataclass(frozen=True)
class TokenSideTableSpec:
    """An ``after_embed`` part: a second table [vocab, width] indexed by the step's tokens,
    whose gathered rows (float32) the blocks' ``TokenSideSpec`` parts read for the rest of
    the step, each its own range of columns."""
    vocab: int
    width: int
    kind: str = "token_side_table"


@dataclass(frozen=True)
class ChainSpec:
    """Several ``after_embed`` / ``on_logits`` parts run one after another; part i's
    parameters are named ``<i>.<name>``."""
    parts: Tuple[object, ...]
    kind: str = "chain"


@dataclass(frozen=True)
class TokenSideSpec:
    """x += rms_norm(P (gelu_tanh(G x) * e)) * w: e = columns [offset, offset + dim) of the
    step's side-table rows, G [dim, hidden] reads the residual stream itself, P [hidden, dim]."""
    hidden: int
    dim: int
    offset: int
    eps: float
    kind: str = "token_side"


@dataclass(frozen=True)
class MLPSpec:
    """down(act(up(h))); activation "gelu" (erf), "gelu_tanh", "relu2" (relu squared), "silu"."""
    hidden: int
    intermediate: int
    activation: str = "gelu"
    kind: str = "mlp"


@dataclass(frozen=True)
class RoutedMLPSpec:
    """``experts`` feed-forward layers down(act(up(.))) of width ``intermediate``, of which a
    token uses the ``top`` with the largest router scores. score "sigmoid" (each expert's own)
    or "softmax" (over the experts); renormalize: the chosen scores are divided by their sum;
    weight_on "input": an expert is applied to weight * h, "output": its result is weighted.
    shared_intermediate: a further expert of that width that every token uses (None: none);
    shared_gate: its result is multiplied by sigmoid(g . h), one number per token."""
    hidden: int
    experts: int
    top: int
    intermediate: int
    activation: str = "relu2"
    score: str = "sigmoid"
    renormalize: bool = False
    weight_on: str = "input"
    shared_intermediate: Optional[int] = None
    shared_gate: bool = True
    kind: str = "routed_mlp"
    # router_bias: a learned number per expert is added to the router's logits.
    # form "mlp": down(act(up(h))). form "limited_glu": an expert has a gate and an up matrix,
    # g = min(gate(h), limit), u = clamp(up(h), -limit, limit), down(g * sigmoid(gate_slope * g)
    # * (u + up_shift)); ``activation`` is not used then. shared_limit: the shared expert's limit.
    # form "glu": an expert is down(act(gate(h)) * up(h)) with ``activation`` "silu" or "gelu_tanh", its
    # first matrix [gate rows | up rows] as in "limited_glu".
    # groups > 1: the experts form that many equal groups of neighbours; a group counts as the
    # largest score in it, and only experts of the ``keep_groups`` best groups can be chosen.
    router_bias: bool = False
    form: str = "mlp"
    limit: float = 0.0
    shared_limit: float = 0.0
    gate_slope: float = 1.702
    up_shift: float = 1.0
    groups: int = 1
    keep_groups: int = 1


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Softmax attention whose keys and values are linear maps of ONE cached latent per token.

    Queries: cq = rms_norm(Dq h) (q_rank wide), q = Uq cq, per head [nope_dim unrotated |
    rope_dim rotated]. Keys/values: Dkv h = [kv_rank | rope_dim]; the first part, RMS-normed,
    is the latent c, the second, rotated, is a key part that all heads share; per head k =
    [Uk c | shared part], v = Uv c (value_dim). Rotation: the first rot_dims coordinates of a
    rotated part in pairs (2i, 2i + 1) by position * rot_base^(-2i/rot_dims). window: a query
    at p reads keys in (p - window, p]; None: all. gated: head h's result is multiplied by
    sigmoid(g_h . h). own_kv False: no Dkv; the layer reads the rows that the layer whose cache
    it borrows stored (its schedule entry names it). cache_window: the window the cache layer
    is kept for (the widest of the layers that read it; None: everything)."""
    hidden: int
    num_heads: int
    nope_dim: int
    rope_dim: int
    value_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    eps: float
    rot_dims: int
    rot_base: float = 10000.0
    window: Optional[int] = None
    cache_window: Optional[int] = None
    gated: bool = True
    own_kv: bool = True
    kind: str = "latent_attention"


@dataclass(frozen=True)
class BonusRecurrenceSpec:
    """Per head a matrix state S [head_dim, head_dim]: o_t = (S + diag(u) k_t v_t^T)^T r_t, then
    S <- diag(w_t) S + k_t v_t^T, w_t = exp(-exp(W2 tanh(W1 m_w) + w0)) (W1 maps to decay_rank
    numbers). r, k, v, the output gate and the decay each read a token-shifted row of their
    own, h_t + (h_{t-1} - h_t) * mu_s. o is divided by its root mean square per head, times a
    weight per channel, times silu(gate), then projected."""
    hidden: int
    num_heads: int
    head_dim: int
    decay_rank: int
    eps: float
    kind: str = "bonus_recurrence"


@dataclass(frozen=True)
class SandwichBlockSpec:
    """x += scale1 * norm1b(mixer(norm1(x))); x += scale2 * norm2b(ffn(norm2(x))); then the
    optional ``side`` part adds what it derives from the stream and the step's tokens.
    layer_scale: scale1 / scale2 are learned vectors (else 1). ffn None: one sublayer."""
    norm1: object
    mixer: object
    norm1b: object
    norm2: object = None
    ffn: object = None
    norm2b: object = None
    side: object = None
    hidden: int = 0
    layer_scale: bool = True
    kind: str = "sandwich"


# ---------------------------------------------------------------------------------------------
# Parts that the Luduvik decoder added; as above, every size and constant is a field.

@dataclass(frozen=True)
class DecayLinearAttentionSpec:
    """Linear attention with ONE fixed decay per head and no softmax or denominator: per head a
    matrix state S [key_dim, value_dim], S_t = decay_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t.

    input_activation: None, or "silu" applied to the q, k and v projections. rot_dims: the first
    coordinates of every head of q and k that are rotated in pairs (i, i + rot_dims/2) by position
    * rot_base^(-2i/rot_dims) (0: none; rot_scaling as ``PositionSpec.scaling``). key_scale: k is
    multiplied by it after the rotation. head_norm "per_head": every head's readout is divided by
    its root mean square; "all_heads": the concatenated heads are normed together. norm_weight:
    the norm has a learned weight per channel. gate_activation: the normed readout is multiplied
    by silu or sigmoid of a gate projection, then projected."""
    hidden: int
    num_heads: int
    key_dim: int
    value_dim: int
    decays: Tuple[float, ...]
    eps: float
    input_activation: Optional[str] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_scaling: Optional[Tuple[float, float, float, float]] = None
    key_scale: float = 1.0
    head_norm: str = "per_head"
    norm_weight: bool = False
    gate_activation: str = "silu"
    kind: str = "decay_linear_attention"


@dataclass(frozen=True)
class BranchMeanSpec:
    """Several mixers side by side that read the same rows: the result is the mean of their
    results, each first RMS-normed over the model width with a weight vector of its own.
    names[i] prefixes the parameters of branches[i]."""
    hidden: int
    eps: float
    branches: Tuple[object, ...]
    names: Tuple[str, ...]
    kind: str = "branch_mean"


@dataclass(frozen=True)
class ParallelBlockSpec:
    """h = norm1(x); x += mixer(h) + ffn(h): one norm, both sublayers read its rows.
    ffn None: the block has the mixer only."""
    norm1: object
    mixer: object
    ffn: object = None
    kind: str = "parallel_prenorm"


# ---------------------------------------------------------------------------------------------
# Parts that the Saredra decoder added; as above, every size and constant is a field.

@dataclass(frozen=True)
class SinkAttentionSpec:
    """Causal grouped-query softmax attention with key and value widths of their own, whose scores
    may be capped and whose softmax denominator may hold one more term.

    score = q . k * scale; softcap: score <- softcap * tanh(score / softcap). window: a query at p
    reads keys in (p - window, p]; None: all. sink None: plain softmax; "unit": the denominator also
    holds exp(0) = 1; "learned": exp(s_h) with a learned s_h per head; the extra term has no value.
    rot_dims: the first coordinates of every head of q and k that turn by position * f_i, f_i =
    rot_base^(-2i/rot_dims), in pairs of ``rot_style`` ("interleaved": (2i, 2i + 1); "half": (i, i +
    rot_dims/2)); rot_ramp / rot_magnitude: see ``PositionSpec.ramp`` / ``.magnitude``.
    qkv_bias: q, k, v have biases, added in the projection. conv_taps > 0: a causal convolution of that
    many taps per channel (no bias, no activation) on q, k and v between projection and rotation; the
    last taps - 1 projected rows of a sequence are carried between steps. out_gate: the concatenated
    heads are multiplied by sigmoid(Wg h) before the output projection. own_kv False: no key and value
    projections; the layer reads what the layer whose cache it borrows stored (its schedule entry
    names it). cache_window: the window the cache layer is kept for (the widest of the layers that
    read it; 0: everything; None: the layer's own window)."""
    hidden: int
    num_heads: int
    num_kv_heads: int
    key_dim: int
    value_dim: int
    scale: float
    softcap: Optional[float] = None
    window: Optional[int] = None
    cache_window: Optional[int] = None
    sink: Optional[str] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    rot_style: str = "interleaved"
    rot_ramp: Optional[Tuple[float, float, float, float]] = None
    rot_magnitude: float = 1.0
    qkv_bias: bool = False
    conv_taps: int = 0
    out_gate: bool = False
    own_kv: bool = True
    kind: str = "attention_sink"


@dataclass(frozen=True)
class StateSpaceSpec:
    """A selective state-space mixer with a scalar decay per head (state-space duality).

    inner = num_heads * head_dim. One projection gives [z: inner | x: inner | B: groups * state | C:
    groups * state | dt: num_heads]; x, B and C pass a causal convolution of ``taps`` per channel (with
    bias) and silu; dt <- softplus(dt + dt_bias). Per head h of group h // (num_heads / groups): S_t =
    exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T (S is [state, head_dim], float32, zero at a
    sequence's start), y_t = S_t^T C_t + D_h x_t. y * silu(z) is RMS-normed in ``norm_groups`` equal
    parts of the row (each by its own root mean square), times a weight, then projected."""
    hidden: int
    num_heads: int
    head_dim: int
    state: int
    groups: int
    taps: int
    norm_groups: int
    eps: float
    kind: str = "state_space"


@dataclass(frozen=True)
class BranchSumSpec:
    """Several mixers side by side that read the same rows: the result is sum_i scales[i] *
    branches[i](h). names[i] prefixes the parameters of branches[i]."""
    hidden: int
    branches: Tuple[object, ...]
    names: Tuple[str, ...]
    scales: Tuple[float, ...]
    kind: str = "branch_sum"
