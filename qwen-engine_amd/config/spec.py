"""Architecture-neutral description of a decoder model.

A model is a list of layers, each put together from parts (norm, mixer,
feed-forward, position encoding), and a *schedule*: the order in which the
layers run.  Every size and constant is a field of a spec, so one model may use
different mixers and feed-forwards in different layers, and a new part only has
to define a spec dataclass with a ``kind`` string and register a builder for it
(see ``parts.registry``).

The specs are plain data: they can be built on a machine without a GPU and are
what the cache manager, the weight loader and the random-weights writer read.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * w over the last dimension."""
    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class RopeSpec:
    """Half-split rotary position encoding over ``rotary_dim`` features.

    Angles are ``position * theta ** (-2 i / rotary_dim)``; the pair of feature
    ``i`` is feature ``i + rotary_dim / 2``.
    """
    theta: float
    rotary_dim: int
    max_positions: int
    kind: str = "rope_half"


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query attention over a paged key/value cache.

    ``window`` is None for attention over all earlier keys, or the number of
    most recent keys (the query's own position included) that a query sees.
    ``qk_norm_eps`` is None when queries and keys are not normalised per head.
    """
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    qkv_bias: bool = False
    qk_norm_eps: Optional[float] = None
    window: Optional[int] = None
    position: Optional[object] = None  # a position-encoding spec, e.g. RopeSpec
    kind: str = "paged_attention"


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(silu(gate(x)) * up(x)), no biases.  ``names``: the tensors of gate, up and down inside the part."""
    intermediate_size: int
    kind: str = "swiglu"
    names: Tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")


@dataclass(frozen=True)
class ScalarRMSNormSpec:
    """y = g * x * rsqrt(mean(x^2) + eps) over the last dimension, g one number (a tensor of no dimensions)."""
    eps: float
    kind: str = "rmsnorm_scalar"


@dataclass(frozen=True)
class RopePairsSpec:
    """Rotary position encoding over neighbouring pairs: the pair (2i, 2i + 1), i < rotary_dim / 2, is
    turned by ``position * theta ** (-2 i / rotary_dim)``; features from rotary_dim on pass unchanged."""
    theta: float
    rotary_dim: int
    kind: str = "rope_pairs"


@dataclass(frozen=True)
class ShortConvSpec:
    """out_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j): a causal convolution over time on each channel,
    added to its input; the last ``taps - 1`` inputs of a request are state."""
    taps: int
    kind: str = "short_conv"


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values are linear maps of one cached latent per token (``kv_rank``
    numbers, RMS-normed), with one rotated key part of ``rot_dim`` numbers shared by all heads.  A head's
    query has ``head_dim`` unrotated and ``rot_dim`` rotated numbers, its value ``v_head_dim``.

    ``q_rank`` None: queries straight from the input; else through a normed latent of that size.
    ``output_gate``: the heads' outputs are multiplied by sigmoid of a projection of the mixer's input, a number
    per output, or, with ``gate_per_head``, one number per head.
    ``window`` None: all earlier keys; else the last ``window`` keys, the query's own included.  ``keep_window``:
    how many keys the layer's cache keeps where that is more than its own window (a later layer that reads this
    cache looks further back); None with a window: the window.
    ``own_latent`` False: the layer has no latent projection; it reads the cache of the layer that the schedule names.
    ``sink``: a learned number per head whose exponential joins the softmax's denominator and carries no value.
    ``position``: a rotation of neighbouring pairs (``RopePairsSpec``) or of half-split pairs
    (``RopeHalfAnglesSpec``) over the first numbers of the rotated part.
    """
    num_heads: int
    head_dim: int
    rot_dim: int
    v_head_dim: int
    kv_rank: int
    scale: float
    norm_eps: float
    q_rank: Optional[int] = None
    output_gate: bool = False
    position: Optional[object] = None
    kind: str = "latent_attention"
    gate_per_head: bool = False
    window: Optional[int] = None
    keep_window: Optional[int] = None
    sink: bool = False
    own_latent: bool = True


@dataclass(frozen=True)
class PolyNormMLPSpec:
    """down(act(up x)), act(z) = a N(z) + b N(z^2) + c N(z^3) + e with N(v) = v / sqrt(mean(v^2) + eps)
    over a token's ``intermediate_size`` values and (a, b, c, e) a tensor of the layer."""
    intermediate_size: int
    eps: float
    kind: str = "polynorm_mlp"


@dataclass(frozen=True)
class GroupedMoESpec:
    """A routed mixture of small gated feed-forwards.  Scores: softmax of the router's 32-bit logits over
    all experts; the experts form ``num_groups`` equal groups of neighbours, of which the ``keep_groups``
    with the largest best score stay; the ``top`` largest scores among those choose the experts and weigh
    them as they are.  An expert: g = min(gate x, limit), u = clamp(up x, -limit, limit),
    down(g * sigmoid(slope * g) * (u + 1))."""
    num_experts: int
    top: int
    num_groups: int
    keep_groups: int
    intermediate_size: int
    limit: float
    slope: float = 1.702
    kind: str = "grouped_moe"


@dataclass(frozen=True)
class PostNormLayerSpec:
    """One post-norm block: x <- mixer_norm(alpha x + mixer(conv(x))); x <- ffn_norm(alpha x + ffn(x)).
    ``conv`` (before the mixer) and ``ffn`` (with its norm) may be None.  ``names``: the checkpoint names
    inside ``prefix`` of mixer norm, mixer, feed-forward norm, feed-forward and convolution."""
    prefix: str
    mixer: object
    mixer_norm: object
    ffn: Optional[object]
    ffn_norm: Optional[object]
    alpha: float
    conv: Optional[object] = None
    names: Tuple[str, str, str, str, str] = ("norm1", "mix", "norm2", "mlp", "canon1")
    kind: str = "postnorm_block"


@dataclass(frozen=True)
class RopeHalfAnglesSpec:
    """Half-split rotation of the first ``rotary_dim`` numbers of a head (number i < rotary_dim / 2 pairs with
    i + rotary_dim / 2) by ``position * theta ** (-2 i / rotary_dim)``; the rest of the head passes unchanged.
    The kernels form angle, sine and cosine in 32-bit from the frequencies: no table, no limit of positions.
    ``scaling_factor``: every frequency is divided by it (positions stretched linearly)."""
    theta: float
    rotary_dim: int
    kind: str = "rope_half_angles"
    scaling_factor: float = 1.0


@dataclass(frozen=True)
class ConvAttentionSpec:
    """Grouped-query attention whose projected queries, keys and values (with biases if ``qkv_bias``) each pass
    a causal convolution of ``conv_taps`` taps over time on every channel before q and k are rotated (0: none).  Keys have
    ``head_dim`` numbers, values ``v_head_dim``.  ``window`` None: all earlier keys; else the last ``window`` keys
    (the query's own included) and, wherever the window stands, the request's first ``keep_first`` keys.
    ``sink``: the softmax's denominator has a 1 added (one more entry of score 0 that carries no value).
    ``names``: the tensors' names inside the part for q, k, v and the output projection; a bias is the
    projection's name + ``bias_suffix``, a convolution's weights [channels, taps] its name + ``conv_suffix``."""
    num_heads: int
    num_kv_heads: int
    head_dim: int
    v_head_dim: int
    scale: float
    conv_taps: int = 0
    qkv_bias: bool = False
    window: Optional[int] = None
    keep_first: int = 0
    sink: bool = False
    position: Optional[object] = None
    names: Tuple[str, str, str, str] = ("q", "k", "v", "o")
    bias_suffix: str = ".b"
    conv_suffix: str = ".conv"
    kind: str = "conv_attention"


@dataclass(frozen=True)
class BiasedMoESpec:
    """A routed mixture of small feed-forwards down(relu(up x)^2) without biases.  Scores: softmax of the
    router's 32-bit logits over ``num_experts + num_identity`` outputs; the ``top`` largest of score + correction
    (a tensor of the layer) are chosen; their weights are their scores without the correction, divided by their
    sum (+ 1e-20), times ``route_scale``.  The last ``num_identity`` outputs are identity experts: their output is
    the input itself, and they have no tensors."""
    num_experts: int
    num_identity: int
    top: int
    intermediate_size: int
    route_scale: float
    kind: str = "biased_moe"


@dataclass(frozen=True)
class ParallelLayerSpec:
    """One block with a single norm whose output both branches read: n = norm(x); x <- x + (mixer(n) + ffn(n)).
    ``ffn`` may be None.  ``names``: the checkpoint names inside ``prefix`` of norm, mixer and feed-forward; a
    norm that is one tensor carries the norm's name itself."""
    prefix: str
    norm: object
    mixer: object
    ffn: Optional[object]
    names: Tuple[str, str, str] = ("norm1", "mix", "mlp")
    kind: str = "parallel_block"


@dataclass(frozen=True)
class BareRMSNormSpec:
    """RMSNorm whose weight tensor carries the part's own name (no ``.weight`` behind it)."""
    eps: float
    kind: str = "rmsnorm_bare"


@dataclass(frozen=True)
class StreamScaleSpec:
    """The stream right after the embedding is multiplied by ``scale`` (in 32-bit); no tensors."""
    scale: float
    prefix: str = ""
    kind: str = "stream_scale"


@dataclass(frozen=True)
class ChunkAttentionSpec:
    """Grouped-query attention inside chunks of positions: with ``chunk`` = c, a query at position i sees the keys
    j <= i with i // c == j // c, chunks counted from the request's start (None: all earlier keys).  Keys have
    ``head_dim`` numbers, values ``v_head_dim``; all four projections have biases if ``bias``.
    ``qk_norm``: None, "head" (RMS norm of every q and k head with one weight of the head's size for all heads) or
    "whole" (RMS norm over all heads of q, and of k, at once, a weight per coordinate), before the rotation.
    ``values_from_keys``: there is no value projection; the values are the keys as projected, before their norm.
    ``value_norm_eps``: every value head is divided by its root mean square (no weight).
    ``value_blend``: None; "source": the values (after their norm) are also left for later layers of the step;
    "blend": v <- (1 - l) v + l v_source with l a tensor of the layer; what is blended is what is cached.
    ``distance_bias_rows`` = B > 0: a table [B, heads] is added to the scaled scores by distance n = i - j: row n
    for n < B // 2, else min(B - 1, B // 2 + floor(log(n / (B // 2)) / log(far / (B // 2)) * (B - B // 2))) with
    far = ``distance_bias_far``.  ``talking_heads``: the heads' scores are then mixed by a matrix [heads, heads]
    before the softmax.  ``names``: tensors of q, k, v, output projection; the others by the suffixes below."""
    num_heads: int
    num_kv_heads: int
    head_dim: int
    v_head_dim: int
    scale: float
    chunk: Optional[int] = None
    bias: bool = False
    qk_norm: Optional[str] = None
    qk_norm_eps: float = 0.0
    values_from_keys: bool = False
    value_norm_eps: Optional[float] = None
    value_blend: Optional[str] = None
    distance_bias_rows: int = 0
    distance_bias_far: float = 0.0
    talking_heads: bool = False
    position: Optional[object] = None
    names: Tuple[str, str, str, str] = ("q", "k", "v", "o")
    bias_suffix: str = ".b"
    norm_suffix: str = ".norm"
    blend_name: str = "vmix"
    distance_bias_name: str = "rel"
    talk_name: str = "talk"
    kind: str = "chunk_attention"


@dataclass(frozen=True)
class ShiftedDecaySpec:
    """A recurrence per head over a state S [head_dim][head_dim] whose inputs are blends of a token x and the token
    before it x' (zeros before the first): m_s = x + (x' - x) mu_s for s in r, k, v, g, w.  r, k, v = W m; gate =
    silu(W_g m_g); decay w = exp(-exp(W_2 tanh(W_1 m_w) + w0)) per key channel (W_1 has ``decay_rank`` rows);
    o_t = (S + diag(u) k_t v_t^T)^T r_t, then S <- diag(w_t) S + k_t v_t^T; each head's o divided by its root mean
    square, times a weight, times the gate, then the output projection."""
    num_heads: int
    head_dim: int
    decay_rank: int
    norm_eps: float
    kind: str = "shifted_decay"


@dataclass(frozen=True)
class DecayedLinearSpec:
    """Linear attention with one decay per head: q, k = silu(W x) with ``head_dim`` numbers a head, v = silu(W x)
    with ``v_head_dim``; S <- decay_h S + k_t v_t^T, o_t = S^T q_t; all heads' o normed together (RMS norm with a
    weight), times sigmoid(W_g x), then the output projection."""
    num_heads: int
    head_dim: int
    v_head_dim: int
    decay: Tuple[float, ...]
    norm_eps: float
    kind: str = "decayed_linear"


@dataclass(frozen=True)
class SideBySideMixerSpec:
    """Two mixers that read the same input; the result is left_scale * left + right_scale * right.  Their tensors
    lie under ``names`` inside the mixer.  At most one of them keeps keys and values and at most one a state."""
    left: object
    right: object
    left_scale: float
    right_scale: float
    names: Tuple[str, str] = ("left", "right")
    kind: str = "side_by_side"


@dataclass(frozen=True)
class GeluMLPSpec:
    """down(gelu(up x)) with the exact gelu 0.5 z (1 + erf(z / sqrt 2)), no biases."""
    intermediate_size: int
    names: Tuple[str, str] = ("up", "down")
    kind: str = "gelu_mlp"


@dataclass(frozen=True)
class LogitSoftcapSpec:
    """logits <- cap * tanh(logits / cap); no tensors."""
    cap: float
    prefix: str = ""
    kind: str = "logit_softcap"


@dataclass(frozen=True)
class BareLayerNormSpec:
    """y = (x - mean(x)) * rsqrt(mean((x - mean(x))^2) + eps) * w over the last dimension, no bias; the weight tensor
    carries the part's own name."""
    eps: float
    kind: str = "layernorm_bare"


@dataclass(frozen=True)
class DiffAttentionSpec:
    """Differential attention over grouped heads: every query head and every key head has two maps of ``head_dim``
    numbers, laid out [map 1 | map 2] in the projections; both maps of a head attend (causally, plain softmax) over
    the same values of ``v_head_dim`` numbers, and the head's output is a1 - lambda a2, divided by its root mean square
    (``norm_eps`` inside the root, no weight) and multiplied by 1 - ``diff``.  lambda = exp(lq1 . lk1) - exp(lq2 . lk2)
    + ``diff`` from four tensors of ``head_dim`` numbers.  ``qk_norm_eps`` not None: every map of every q and k head is
    RMS-normed with one weight of ``head_dim`` numbers for q and one for k, before the rotation, which turns the
    first numbers of every map (``position``).  ``output_gate``: a head's output times sigmoid of one number per head,
    a projection of the mixer's input.  ``names``: the tensors of q, k, v, the output projection and the gate; the
    norm weights are the projections' names + ``norm_suffix``; the four lambda tensors ``lambda_names``."""
    num_heads: int
    num_kv_heads: int
    head_dim: int
    v_head_dim: int
    scale: float
    diff: float
    norm_eps: float
    qk_norm_eps: Optional[float] = None
    output_gate: bool = False
    position: Optional[object] = None
    names: Tuple[str, str, str, str, str] = ("q", "k", "v", "o", "g")
    norm_suffix: str = ".norm"
    lambda_names: Tuple[str, str, str, str] = ("lq1", "lk1", "lq2", "lk2")
    kind: str = "diff_attention"


@dataclass(frozen=True)
class TopSoftmaxMoESpec:
    """A routed mixture of small gated feed-forwards down(silu(gate x) * up x) without biases.  The router's 32-bit
    logits (plus a bias tensor if ``router_bias``) choose the ``top`` largest; their weights are the softmax over the
    chosen logits alone.  ``shared_intermediate_size``: one more expert of that width that every token uses, added
    with the weight sigmoid(w_sg . x) if ``shared_gate``, else 1."""
    num_experts: int
    top: int
    intermediate_size: int
    router_bias: bool = False
    shared_intermediate_size: Optional[int] = None
    shared_gate: bool = False
    kind: str = "top_softmax_moe"


@dataclass(frozen=True)
class LayerSpec:
    """One pre-norm residual block: x += mixer(norm(x)); x += ffn(norm(x)).  ``ffn`` None: the layer is its mixer alone
    (its second norm is then used only if ``ffn_norm`` is given and the folder holds its tensors).

    ``prefix`` is the checkpoint name prefix of the layer's tensors
    (for instance ``model.layers.3``).
    """
    prefix: str
    mixer_norm: object
    mixer: object
    ffn_norm: object
    ffn: object
    kind: str = "prenorm_block"
    # checkpoint names of the four parts inside ``prefix``, in the order of the fields above
    part_names: Tuple[str, str, str, str] = ("input_layernorm", "self_attn", "post_attention_layernorm", "mlp")


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.

    ``layer`` indexes ``ModelSpec.layers`` (a layer may appear in several
    entries: its weights are shared, each entry has a cache of its own).
    ``cache_from`` is None, or the index of an earlier schedule entry whose
    cache this run reads instead of writing one of its own.
    """
    layer: int
    cache_from: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    embed_name: str
    final_norm_name: str
    head_name: str
    tie_head: bool
    max_positions: int
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    # optional parts around the layers: a spec with a ``kind`` (and a ``prefix`` for its tensors' names)
    stream_prologue: Optional[object] = None   # changes the stream right after the embedding
    logit_epilogue: Optional[object] = None    # changes the logits after the head

    def validate(self) -> None:
        if not self.layers:
            raise ValueError("a model needs at least one layer")
        for i, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule entry {i} names layer {entry.layer}, "
                                 f"the model has {len(self.layers)}")
            if entry.cache_from is not None:
                if not 0 <= entry.cache_from < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry "
                                     f"{entry.cache_from}, which does not run before it")
                if self.schedule[entry.cache_from].cache_from is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry "
                                     f"{entry.cache_from}, which has no cache of its own")
