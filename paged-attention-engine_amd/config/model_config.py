"""Typed descriptions of a model: specs of parts, layers, and the order they run in.

Nothing here knows an architecture.  An architecture's own config class (for
Qwen2: `models/qwen2.py`) reads its config.json keys and turns them into a
`ModelPlan`; the engine builds parts from the plan's specs by their `kind`.

The reference keeps the same constants in one frozen dataclass, `ModelDims`
(engine/model.py:43-80), and passes eps, theta, scale and group size to free
functions as arguments (engine/model.py:117,132,138; engine/attention.py:135-144).
Here every part's spec carries its own sizes and constants so that two layers of
one model may differ.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be turned into a model, with the key named."""


@dataclass(frozen=True)
class PartSpec:
    """Base of every spec: `kind` selects the implementation in the part registry."""

    kind: str


@dataclass(frozen=True)
class NormSpec(PartSpec):
    size: int = 0
    eps: float = 0.0
    kind: str = "rmsnorm"
    weight_name: str = "weight"  # the tensor's name below the norm's prefix
    weight_offset: float = 0.0   # the stored tensor plus this is the weight (1: a weight stored around zero)


@dataclass(frozen=True)
class FrequencyRamp:
    """Frequencies of a rotation stretched for contexts longer than the `original` one (YaRN): a pair
    that turns more than `fast` times over the original context keeps its frequency, one that turns
    fewer than `slow` times has it divided by `factor`, and the pairs between are blended linearly
    over their index; cosines and sines are multiplied by 0.1 ln(factor) + 1."""

    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class WavelengthRamp:
    """Frequencies of a rotation stretched by wavelength (the scaling of Llama 3.1): with l = 2 pi / f a pair's
    wavelength, a pair with l < original / high keeps its frequency, one with l > original / low has it divided
    by `factor`, and between the two the frequencies f / factor and f are blended linearly in original / l:
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low).  Cosines and sines keep their size."""

    factor: float
    original: float
    low: float
    high: float


@dataclass(frozen=True)
class PositionSpec(PartSpec):
    """Rotation of query and key by absolute position; `rotary_dim` leading
    features of each head are rotated in pairs: (i, i + rotary_dim/2) for kind
    "neox_rope", (2i, 2i + 1) for kind "interleaved_rope" (which also takes a `ramp`:
    a `FrequencyRamp` or a `WavelengthRamp`)."""

    rotary_dim: int = 0
    theta: float = 10000.0
    kind: str = "neox_rope"
    ramp: Optional[object] = None


@dataclass(frozen=True)
class MixerSpec(PartSpec):
    """Causal attention over the paged cache with grouped key/value heads.

    `window` None means every earlier key; otherwise a query at position p sees
    keys p-window+1 .. p.  `scale` multiplies the scores."""

    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    qkv_bias: bool = True
    out_bias: bool = False
    window: Optional[int] = None
    position: Optional[PositionSpec] = None
    kind: str = "attention"
    # names of the four projections below the mixer's prefix (each with `weight_suffix` and, where the
    # spec says so, ".bias"): an architecture that calls them otherwise sets these, not a new mixer
    q_name: str = "q_proj"
    k_name: str = "k_proj"
    v_name: str = "v_proj"
    o_name: str = "o_proj"
    weight_suffix: str = ".weight"
    # what some architectures' attention has besides (None / False: not there)
    value_dim: Optional[int] = None      # width of a value head when it differs from head_dim
    softcap: Optional[float] = None      # scores become softcap * tanh(score / softcap)
    sinks: bool = False                  # one learned number per query head joins the softmax's denominator
    sink_name: str = "sinks"
    fixed_sink: Optional[float] = None   # instead of learned sinks: every head's sink is this number (0: the
                                         # denominator is one larger than the sum of exponentials); no tensor
    qk_norm: Optional[str] = None        # "projection": RMS norm over the whole q and the whole k projection;
                                         # "per_head": over each head, with one weight [head_dim] shared by the heads
    qk_norm_eps: float = 1e-6
    q_norm_name: str = "q_norm.weight"
    k_norm_name: str = "k_norm.weight"
    # and some others' (a spec with any of these runs the mixer's convolution path):
    # "head" as `qk_norm`: every query and key head divided by its own root mean square, no weight
    mask: str = "window"                 # "chunk": `window` is a chunk length, position p sees keys from p - p % window on
    conv_taps: Optional[int] = None      # a causal convolution over time on every channel of q, k and v, after the projection
    conv_suffix: str = ".conv"           # its filters: <projection's name><suffix>, [channels, taps]
    distance_slope_base: Optional[float] = None  # b: score -= 2^(-b (h + 1) / heads) * (query position - key position)
    gate_name: Optional[str] = None      # a projection W_g of the mixer's input: heads *= sigmoid(W_g x) before W_o
    bias_suffix: str = ".bias"
    own_kv: bool = True                  # False: the layer has no key/value tensors at all; it reads another stop's cache

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def plain(self) -> bool:
        """The reference's attention and nothing more, with heads in multiples of 16 up to 256: what the kernels of
        the first path compute (any other head size takes the path for value widths, caps and sinks)."""
        return (self.value_dim in (None, self.head_dim) and self.softcap is None and not self.sinks
                and self.fixed_sink is None and self.qk_norm is None and not self.convolved and self.head_dim % 16 == 0 and 16 <= self.head_dim <= 256)

    @property
    def convolved(self) -> bool:
        """Whether the spec takes the path with convolutions, per-head norms, distance bias, chunks or a gate."""
        return (self.conv_taps is not None or self.qk_norm == "head" or self.mask != "window"
                or self.distance_slope_base is not None or self.gate_name is not None or not self.own_kv)


@dataclass(frozen=True)
class LatentMixerSpec(PartSpec):
    """Attention whose keys and values are products of one cached latent vector per token.

    Per token the mixer's input is projected down to `kv_rank` + `rope_dim` features: the first
    kv_rank, RMS-normed with a weight, are the latent c; the rest are one rotated key part shared by all
    heads.  Head h's key is [W_uk_h c | rotated part], its value W_uv_h c; a query head has `nope_dim`
    features that meet W_uk_h c and `rope_dim` rotated ones.  The cache holds c and the rotated part, nothing per head."""

    hidden_size: int = 0
    num_heads: int = 0
    nope_dim: int = 0
    rope_dim: int = 0
    value_dim: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    window: Optional[int] = None
    mask: str = "window"
    position: Optional[PositionSpec] = None   # rotation of the rope_dim part (its rotary_dim <= rope_dim)
    norm_eps: float = 1e-6
    kind: str = "latent_attention"
    q_name: str = "q"
    down_name: str = "dkv"
    down_norm_name: str = "dkv.norm"
    up_k_name: str = "uk"
    up_v_name: str = "uv"
    o_name: str = "o"
    weight_suffix: str = ""
    sinks: bool = False        # one learned number per head joins the softmax's denominator as exp(sink), unscaled
    sink_name: str = "sink"
    own_kv: bool = True        # False: no down projection and no norm of its own; the layer reads another stop's rows


@dataclass(frozen=True)
class DeltaMixerSpec(PartSpec):
    """The gated delta rule: a recurrent mixer with one state matrix [key_dim, value_dim] per head
    and short causal convolutions on q, k and v.  `num_kv_heads` query/key heads of `key_dim` serve
    `num_heads` value heads of `value_dim`."""

    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    conv_taps: int = 4
    norm_eps: float = 1e-6
    unit_eps: float = 1e-6   # inside the root when q and k are made unit vectors
    kind: str = "gated_delta"
    q_name: str = "q"
    k_name: str = "k"
    v_name: str = "v"
    gate_name: str = "g"
    beta_name: str = "b"
    decay_name: str = "a"
    o_name: str = "o"
    conv_suffix: str = ".conv"
    a_log_name: str = "A_log"
    dt_bias_name: str = "dt_bias"
    norm_name: str = "norm"
    weight_suffix: str = ""
    # what some designs' rule has besides:
    decay: str = "head"              # "channel": one decay per head and key channel (A_log stays per head, dt_bias [heads, key_dim])
    decay_rank: Optional[int] = None  # the decay's input is W_a2 (W_a1 h) with that many features between (names a1, a2)
    gate_rank: Optional[int] = None   # likewise the gate's, W_g2 (W_g1 h)
    gate_activation: str = "silu"    # or "sigmoid"
    low_rank_suffixes: Tuple[str, str] = ("1", "2")  # appended to decay_name / gate_name for the two narrow products


@dataclass(frozen=True)
class MatrixMemorySpec(PartSpec):
    """A matrix memory with exponential input and forget gates (the mLSTM cell): a recurrent mixer with, per head,
    a matrix [key_dim, value_dim], the sum of its gated keys and a running maximum of the gates' logarithms.
    `gate_cap` c bounds both gates' inputs by c tanh(z / c); `readout_floor` is added to the read-out's
    denominator max(|n . q|, exp(-m))."""

    hidden_size: int = 0
    num_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    gate_cap: float = 15.0
    norm_eps: float = 1e-6
    readout_floor: float = 1e-6
    kind: str = "matrix_memory"
    q_name: str = "q"
    k_name: str = "k"
    v_name: str = "v"
    gate_name: str = "g"          # the output gate sigmoid(W_g h)
    input_gate_name: str = "i"    # with a bias
    forget_gate_name: str = "f"   # with a bias
    o_name: str = "o"
    norm_name: str = "norm"       # one weight per head and value feature
    bias_suffix: str = ".b"
    weight_suffix: str = ""


@dataclass(frozen=True)
class LinearAttentionSpec(PartSpec):
    """Gated linear attention: a recurrent mixer with one state matrix [key_dim, value_dim] per head that decays,
    per token, by a factor of its own for every key channel: S <- diag(a_t) S + k_t v_t^T, o_t = S^T q_t, with
    a = sigmoid(z)^(1 / decay_temperature) and z through two narrow products with `decay_rank` features between
    and a bias.  q is multiplied by key_dim^-1/2; o is RMS-normed per head with a weight [value_dim] shared by the
    heads, gated by `gate_activation`(W_g h) and projected out."""

    hidden_size: int = 0
    num_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    decay_rank: int = 0
    decay_temperature: float = 1.0
    norm_eps: float = 1e-6
    gate_activation: str = "silu"    # or "sigmoid"
    kind: str = "gated_linear_attention"
    q_name: str = "q"
    k_name: str = "k"
    v_name: str = "v"
    gate_name: str = "g"
    decay_name: str = "a"            # the two narrow products are <decay_name>1 and <decay_name>2, the bias <decay_name>2<bias_suffix>
    o_name: str = "o"
    norm_name: str = "norm"
    bias_suffix: str = ".b"
    weight_suffix: str = ""


@dataclass(frozen=True)
class SideBySideSpec(PartSpec):
    """Two mixers that read the same input; the result is left_scale * left + right_scale * right.  Their
    tensors lie below `left_prefix` and `right_prefix` of the mixer's own prefix."""

    left: Optional[PartSpec] = None
    right: Optional[PartSpec] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    left_prefix: str = "left."
    right_prefix: str = "right."
    kind: str = "side_by_side"


@dataclass(frozen=True)
class ExpertsSpec(PartSpec):
    """A feed-forward of `num_experts` small gated experts W_down (act(W_gate h) * (W_up h)) of which a token
    uses `top`: router scores are the softmax of W_router h over all experts (float32); the experts form
    `groups` equal groups of neighbours, a group's score is its largest, and only experts of the `groups_kept`
    best groups can be chosen; the chosen experts' outputs are added with their scores times `route_scale`."""

    hidden_size: int = 0
    intermediate_size: int = 0
    num_experts: int = 0
    top: int = 1
    groups: int = 1
    groups_kept: int = 1
    route_scale: float = 1.0
    activation: str = "silu"
    kind: str = "experts"
    router_name: str = "router"
    choice_bias_name: Optional[str] = None  # a tensor [experts] added to the scores where experts are chosen (the
                                            # weights stay the scores themselves); None: no such tensor
    expert_prefix: str = "e"   # expert j's tensors lie below <expert_prefix><j>.
    gate_name: str = "gate"
    up_name: str = "up"
    down_name: str = "down"
    weight_suffix: str = ""


@dataclass(frozen=True)
class PairEmbeddingSpec:
    """A second embedding table added to the first, indexed by a hash of the token before and the token:
    row (previous * mul_prev + token * mul_cur) mod buckets; a sequence's first token takes row `buckets`,
    the table's last.  The token before a step's first is per-request state."""

    name: str
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class TokenSideSpec:
    """A layer's own input from the token: the layer reads `dim` columns, from `first_column` on, of a second
    token table `table_name` [vocab, table_width] shared by the layers, e = table[token][first_column : + dim], and
    adds  N(W_proj (act(W_gate x) * e))  to the stream x it has just written, N an RMS norm with a plain weight."""

    table_name: str
    table_width: int
    first_column: int
    dim: int
    vocab_size: int
    eps: float
    activation: str = "gelu_tanh"
    gate_name: str = "gate"
    proj_name: str = "proj"
    norm_name: str = "norm"
    weight_suffix: str = ""


@dataclass(frozen=True)
class FeedForwardSpec(PartSpec):
    hidden_size: int = 0
    intermediate_size: int = 0
    activation: str = "silu"
    kind: str = "swiglu"
    # names of the three projections below the feed-forward's prefix
    gate_name: str = "gate_proj"
    up_name: str = "up_proj"
    down_name: str = "down_proj"
    weight_suffix: str = ".weight"


@dataclass(frozen=True)
class LayerSpec:
    """One block: which parts, in which arrangement, under which tensor-name prefix."""

    prefix: str
    mixer: PartSpec
    feed_forward: Optional[PartSpec]   # None: the layer has no feed-forward (arrangements that allow it)
    mixer_norm: PartSpec
    feed_forward_norm: Optional[PartSpec]
    # tensor-name prefixes of the four parts below `prefix`
    mixer_prefix: str = "self_attn."
    feed_forward_prefix: str = "mlp."
    mixer_norm_prefix: str = "input_layernorm."
    feed_forward_norm_prefix: str = "post_attention_layernorm."
    arrangement: str = "prenorm"
    residual_scale: float = 1.0  # what a branch is multiplied by before it joins the stream ("branchnorm")
    # arrangement "hyper": the stream is `streams` copies joined by hyper-connections whose tensors
    # (in [S], out [S], mix [S, S] indexed [from, to]) lie under `connection_prefixes` (mixer, feed-forward;
    # None: the plain sum x <- x + y), and a branch's output is first multiplied, feature by feature, by
    # the tensors `layer_scale_names` (None: no such scale)
    streams: int = 1
    connection_prefixes: Optional[Tuple[str, str]] = None
    layer_scale_names: Optional[Tuple[str, str]] = None
    # arrangement "sandwich": a norm before and a norm after each sublayer, x <- x + norm_out(sublayer(norm(x)));
    # the norms after, with their prefixes, and what the token itself feeds the layer after its feed-forward
    mixer_out_norm: Optional[PartSpec] = None
    feed_forward_out_norm: Optional[PartSpec] = None
    mixer_out_norm_prefix: str = ""
    feed_forward_out_norm_prefix: str = ""
    token_side: Optional[TokenSideSpec] = None
    token_side_prefix: str = "side."


@dataclass(frozen=True)
class ScheduleEntry:
    """One stop of the forward pass.

    `layer` indexes `ModelPlan.layers` (a layer may be named by several
    entries: its weights are then shared while each entry keeps a cache of its
    own).  `cache_from` names an earlier *entry* whose cache this entry reads
    instead of writing one.  `add_embedding`: before this stop runs, the embedding's output (the
    stream as it was before the first stop) is added to the stream once more."""

    layer: int
    cache_from: Optional[int] = None
    add_embedding: bool = False


@dataclass(frozen=True)
class ModelPlan:
    architecture: str
    hidden_size: int
    vocab_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: PartSpec
    embedding_name: str
    head_name: Optional[str]  # None: the head shares the embedding matrix
    final_norm_prefix: str
    max_positions: Optional[int] = None
    # tensors a checkpoint of this architecture may hold without the model using them (a head stored
    # although it is tied to the embedding, say): the loader passes over them
    optional_names: Tuple[str, ...] = ()
    # what some architectures do around the blocks (the reference's model does none of it:
    # engine/model.py:401,453-455 gathers rows and multiplies by the head as they are)
    embedding_scale: float = 1.0            # the gathered rows are multiplied by this
    logit_scale: float = 1.0                # the logits are multiplied by this ...
    logit_softcap: Optional[float] = None   # ... and then, with a cap c, become c * tanh(logits / c)
    streams: int = 1                        # copies the residual stream is kept in (blocks of arrangement "hyper")
    pair_embedding: Optional[PairEmbeddingSpec] = None  # a hashed table of token pairs added to the embedding
    position_table_name: Optional[str] = None  # a learned row per position [max_positions, hidden], added unscaled
    extra: Mapping[str, Any] = field(default_factory=dict)

    def __post_init__(self) -> None:
        for i, entry in enumerate(self.schedule):
            if not 0 <= entry.layer < len(self.layers):
                raise ConfigError(f"schedule entry {i} names layer {entry.layer} of {len(self.layers)}")
            if entry.cache_from is not None and not 0 <= entry.cache_from < i:
                raise ConfigError(
                    f"schedule entry {i} reads the cache of entry {entry.cache_from}, "
                    "which is not an earlier entry")
        for i, layer in enumerate(self.layers):
            if layer.streams != self.streams:
                raise ConfigError(f"layer {i} keeps {layer.streams} copies of the stream, the model {self.streams}")
            if layer.streams != 1 and layer.arrangement != "hyper":
                raise ConfigError(f"layer {i}: only the arrangement 'hyper' keeps several copies of the stream")
        if self.position_table_name is not None and not self.max_positions:
            raise ConfigError("a table of learned positions needs max_positions, its number of rows")
        if self.schedule and self.schedule[0].add_embedding:
            raise ConfigError("the first stop of the schedule cannot add the embedding's output again")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError(f"logit_softcap must be positive, got {self.logit_softcap}")


def require(cfg: Mapping[str, Any], key: str, kind=int):
    """Fetch a required config.json key with a typed, named error."""
    if key not in cfg or cfg[key] is None:
        raise ConfigError(f"config.json lacks the key '{key}'")
    try:
        return kind(cfg[key])
    except (TypeError, ValueError) as err:
        raise ConfigError(f"config.json key '{key}' = {cfg[key]!r} is not {kind.__name__}") from err


def positive(name: str, value) -> None:
    if value <= 0:
        raise ConfigError(f"config.json key '{name}' must be positive, got {value}")
