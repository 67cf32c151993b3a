"""Architecture-neutral description of a decoder: parts, layers and run order.

A model is data before it is code: a `ModelSpec` lists one `LayerSpec` per
layer, each naming its mixer, feed-forward and norms by `kind` together with
every size and constant they need, and a `schedule` that says in which order
layers run and whose cache each of them uses.  Nothing in here knows a model
family; an architecture is a function from its config.json to a `ModelSpec`
(see `inferrs_amd.config.registry`).

The reference wires the same information into Rust structs per model
(`inferrs-models/src/models/qwen3.rs:28-45`, `:264-290`); here it is explicit
so that layers of one model may differ and parts can be reused.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Optional, Tuple


class SpecError(ValueError):
    """A specification that the parts or kernels cannot honour."""


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last dimension."""
    size: int
    eps: float
    add_one: bool = False          # weight is stored as (w - 1) when True
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class LayerNormSpec:
    """Layer norm over the last dimension: (x - mean) / sqrt(var + eps) * w + b, the variance the mean of the squared
    deviations.  The bias is stored under the weight's name + `bias_suffix`."""
    size: int
    eps: float
    bias_suffix: str = ".b"
    kind: str = "layernorm"


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter queries and keys.

    kind "rope": rotate the first `rot_dim` features of each head by
    angle = position * theta**(-2i/rot_dim); pairing "half" pairs feature i
    with i + rot_dim/2, "interleaved" pairs 2i with 2i+1.
    kind "none": nothing is applied.
    `scaling`: None, or a law that changes the angles' frequencies, as (name, factor, ...): ("linear", f)
    divides every frequency by f (positions are read as position / f); ("yarn", factor, original, fast,
    slow) divides the frequencies of the pairs that make fewer than `slow` turns over `original` positions
    by `factor`, keeps those that make more than `fast`, ramps linearly between them, and multiplies cos
    and sin by 0.1 ln(factor) + 1; ("llama3", factor, low, high, original) keeps the frequencies whose wavelength is
    shorter than original / high, divides those whose wavelength is longer than original / low by `factor`, and blends
    the two between them.  A law that has no entry in the position part is refused by name when
    the part is built.
    """
    kind: str = "rope"
    head_dim: int = 0
    rot_dim: int = 0
    theta: float = 10000.0
    pairing: str = "half"
    scaling: Optional[Tuple] = None


@dataclass(frozen=True)
class AttentionSpec:
    """Grouped-query softmax attention over a paged key/value cache."""
    hidden: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: PositionSpec
    qk_norm: Optional[NormSpec] = None     # per-head norm of q and k before rotation
    window: Optional[int] = None           # keys kept: the last `window` positions; None = all
    scale: Optional[float] = None          # None = 1/sqrt(head_dim)
    qkv_bias: bool = False                 # q_proj.bias, k_proj.bias, v_proj.bias are added to the projections
    o_bias: bool = False                   # o_proj.bias is added to the output projection
    sink: bool = False                     # the softmax's denominator holds one more term, exp(0): a key of score 0 without a value
    values_from_keys: bool = False         # no value projection: a value is the key projection's own row, taken ahead of the per-head norm and the turn by position
    names: Optional[Tuple[Tuple[str, str], ...]] = None    # (the part's tensor name, the name in the file) where they differ
    v_head_dim: Optional[int] = None       # the width of a head's values (and of its output); None: head_dim
    gate: bool = False                     # the joined heads are multiplied by sigmoid(W_g h) ("g_proj.weight") before the output projection
    own_kv: bool = True                    # False: no key or value projection (nor the keys' norm): the layer's stop of the schedule reads
                                           # another stop's cache (`ScheduleEntry.cache_of`) with its own queries, window and scale
    reader_windows: Tuple[Optional[int], ...] = ()   # the windows of the stops that read this layer's cache: it keeps what the widest needs
    mask_chunk: Optional[int] = None       # a query sees the keys of its own chunk of this many positions only (chunks counted from
                                           # position 0 of the sequence), up to itself; the cache keeps every position
    gate_per_head: bool = False            # with `gate`: one gate value a head ("g_proj.weight" is [n_heads, hidden])
    qk_unit_norm: bool = False             # q and k are brought to unit root mean square a head, without a weight (`qk_norm` gives
                                           # size and eps, no tensor is loaded).  A turn by position keeps a head's sum of
                                           # squares, so the norm ahead of the turn and behind it are the same number
    kind: str = "attention"

    @property
    def softmax_scale(self) -> float:
        return self.scale if self.scale is not None else self.head_dim ** -0.5

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim

    @property
    def kept_window(self) -> Optional[int]:
        """How many of the last positions the cache keeps: enough for this layer's window and for every reader's."""
        windows = (self.window,) + tuple(self.reader_windows)
        return None if self.mask_chunk or any(w is None for w in windows) else max(windows)


@dataclass(frozen=True)
class GatedMlpSpec:
    """down( act(gate(x)) * up(x) ).  `activation`: "silu", or "gelu_tanh" (GELU in its tanh form); `bias`: every
    projection has a bias vector beside its weight."""
    hidden: int
    intermediate: int
    activation: str = "silu"
    bias: bool = False
    kind: str = "gated_mlp"
    names: Optional[Tuple[Tuple[str, str], ...]] = None    # (the part's tensor name, the name in the file) where they differ


@dataclass(frozen=True)
class DenseMlpSpec:
    """down( act(up(x)) ), no gate and no biases.  `activation`: "gelu" (the exact one), "gelu_tanh" or "silu"."""
    hidden: int
    intermediate: int
    activation: str = "gelu"
    kind: str = "dense_mlp"


@dataclass(frozen=True)
class RetentionSpec:
    """A sum of outer products k v^T a head that fades by a constant factor a token and is read out with the query,
    un-normalised: S <- decay_h S + (k dim^-1/2) v^T, o = S^T q.  A head's o then gets unit root mean square (`norm_eps`,
    weightless); the heads side by side are gated by silu(W_g h) and go through W_o.  No biases anywhere."""
    hidden: int
    n_heads: int
    head_dim: int
    v_dim: int
    decay: Tuple[float, ...]
    norm_eps: float
    kind: str = "retention"


@dataclass(frozen=True)
class SideBySideSpec:
    """Two mixers that read the same input; the result is left_scale * left + right_scale * right.  Their tensors
    lie under `left_prefix` and `right_prefix` of the layer's mixer."""
    left: Any
    right: Any
    left_scale: float = 1.0
    right_scale: float = 1.0
    left_prefix: str = "left."
    right_prefix: str = "right."
    kind: str = "side_by_side"


@dataclass(frozen=True)
class MatrixMemorySpec:
    """The matrix memory with exponential gates (the mLSTM of the xLSTM): q is scaled by dim^-1/2; a log input gate
    i = cap tanh((W_i h + b_i) / cap) and a log forget gate f = logsigmoid(cap tanh((W_f h + b_f) / cap)) a head; under a
    running maximum m_t = max(f + m_(t-1), i) that starts at 0, S <- exp(f + m_(t-1) - m_t) S + exp(i - m_t) k v^T and
    n likewise with k alone; o = S^T q / (max(|n . q|, exp(-m_t)) + 1e-6).  A head's o then gets unit root mean square
    (`norm_eps`); the heads side by side are scaled by a weight vector, gated by sigmoid(W_g h) and go through W_o."""
    hidden: int
    n_heads: int
    head_dim: int
    v_dim: int
    gate_cap: float
    norm_eps: float
    kind: str = "mlstm"


@dataclass(frozen=True)
class StateSpaceSpec:
    """A selective state space with a scalar decay a head (Mamba-2): one product gives [z | x | B | C | dt] with
    inner = n_heads * v_dim and `groups` groups of `state` entries for B and C; the channels of x, B and C are each
    filtered over their last `conv` inputs (a bias, then SiLU); dt = softplus(dt + dt_bias); S <- exp(-exp(A_log) dt) S + dt B x^T,
    y = S^T C + D x; y * silu(z) is RMS-normed in `norm_groups` equal parts (`norm_eps`), times a weight, projected."""
    hidden: int
    n_heads: int
    v_dim: int
    state: int
    groups: int
    conv: int
    norm_groups: int
    norm_eps: float
    kind: str = "mamba2"


@dataclass(frozen=True)
class PassInputSpec:
    """What enters the stream before each pass over a looped range of layers: row t of the tensor `name` [times,
    hidden] before pass t, and, before every pass but the first, the embedding's output once more (`readd_embedding`)."""
    name: str
    times: int
    hidden: int
    readd_embedding: bool = True
    kind: str = "pass_input"


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Softmax attention whose keys and values are products of one low-rank row a token.

    q = W_q h, head by head [head_dim plain | rot_dim rotated]; W_dkv h = [kv_rank latent | rot_dim key part shared
    by the heads]; the latent is RMS-normed (`norm_eps`); a head's plain key is W_uk c, its value W_uv c
    (`v_dim` wide); score = (q_plain . k_plain + q_rot . k_rot) * scale.  Only the normed latent and the rotated
    key part are cached.  `position.rot_dim` of the `rot_dim` rotated features turn.  `gate`: the joined heads are
    multiplied by sigmoid(W_g h) before the output projection (`gate_per_head`: one gate value a head, "g" is
    [n_heads, hidden]).  `q_rank`: the queries come through a low-rank row of their own, q = W_uq rmsnorm(W_dq h) * w
    (tensors "dq", "dq.norm", "uq" instead of "q").  `sink`: the softmax's denominator holds one more term exp(s_h), a
    learned number a head (tensor "sink" [n_heads]) that has no key and no value and is not scaled."""
    hidden: int
    n_heads: int
    head_dim: int
    rot_dim: int
    v_dim: int
    kv_rank: int
    position: PositionSpec
    scale: float
    norm_eps: float
    gate: bool = True
    window: Optional[int] = None
    kind: str = "latent_attention"
    q_rank: Optional[int] = None
    sink: bool = False
    gate_per_head: bool = False


@dataclass(frozen=True)
class GatedRecurrenceSpec:
    """The real-gated linear recurrent unit behind a causal convolution a channel, beside a GELU branch:
    y = gelu_tanh(W_y h + b), u = conv(W_x h + b); r, i = sigmoid of block-diagonal products of u (`blocks` equal
    parts); a = exp(-decay * r * softplus(lam)); S <- a S + sqrt(1 - a^2) i u; output W_o (S * y)."""
    hidden: int
    width: int
    blocks: int
    conv: int                      # taps of the convolution; the last meets the current token
    decay: float = 8.0
    kind: str = "rglru"


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """`experts` gated feed-forwards of which a token runs `top`, chosen by the router's scores (`score`:
    "sigmoid" of each logit, or "softmax" over all); weights = score * `scale`, over the chosen ones
    renormalised to 1 first with `renormalize`.  An expert: g = min(W_gate h, limit), u = clamp(W_up h, -limit,
    limit), W_down (g * sigmoid(alpha g) * (u + 1)).  No biases.
    `identity`: the router has that many more outputs behind the experts'; one of them, chosen, stands for an expert
    that hands its input on.  `correction`: a tensor "correction" [experts + identity] is added to the scores for the
    choice only; the weights are the scores themselves.  `shared`: a `ClampedMlpSpec` that runs for every token beside
    the chosen experts (tensors under "shared."), its output added; `shared_gate`: times sigmoid(W_sg h), one number a
    token (tensor "shared.sg" [1, hidden], formed like a router's logit, in 32-bit).  `weight_on_input`: a chosen expert
    runs on weight * h and its output is added as it is (instead of weight * expert(h))."""
    hidden: int
    intermediate: int
    experts: int
    top: int
    scale: float = 1.0
    limit: float = 7.0
    alpha: float = 1.702
    score: str = "sigmoid"
    renormalize: bool = False
    identity: int = 0
    correction: bool = False
    shared: Any = None
    kind: str = "routed_experts"
    weight_on_input: bool = False
    shared_gate: bool = False


@dataclass(frozen=True)
class ClampedMlpSpec:
    """A gated feed-forward in the form of a routed expert, for every token: g = min(W_gate h, limit), u = clamp(W_up h,
    -limit, limit), W_down (g * sigmoid(alpha g) * (u + 1)).  Tensors "gate", "up", "down"; no biases."""
    hidden: int
    intermediate: int
    limit: float
    alpha: float = 1.702
    kind: str = "clamped_mlp"


@dataclass(frozen=True)
class PostNormSpec:
    """How a layer's sub-layers stand around a stream that is normed after every sum (kept in 32-bit):
    x <- norm(alpha x + part(x)), the parts reading x as it stands.  `bare_norm_name`: a layer without a feed-forward
    whose file still holds a second norm under this name runs it on the scaled stream alone, x <- norm(alpha x); a file
    without the tensor leaves the step out."""
    alpha: float = 1.0
    bare_norm_name: Optional[str] = None


@dataclass(frozen=True)
class TokenSideSpec:
    """What a token itself adds to the stream behind a layer: e = the layer's `dim` columns (from `offset`) of a second
    embedding table's row for the token (`EmbeddingSpec.side_name`); y = W_proj (act(W_gate x) * e); x <- x +
    rmsnorm(y) * w.  Tensors `prefix` + "gate" [dim, hidden], "proj" [hidden, dim], "norm" [hidden]."""
    dim: int
    offset: int
    prefix: str
    eps: float
    activation: str = "gelu_tanh"


@dataclass(frozen=True)
class ParallelSpec:
    """How a layer's sub-layers stand around a stream kept in 32-bit when both read ONE normed copy of it:
    h = norm(x); x <- x + mixer(h) + ffn(h).  `side`: a `TokenSideSpec` whose row enters behind the sum."""
    side: Any = None


@dataclass(frozen=True)
class StreamsSpec:
    """How a layer's sub-layers stand around `streams` residual streams (kept in 32-bit): sub-layer q reads
    sum_s in_q[s] x_s through its norm, its output is scaled feature by feature (`layer_scale`), and the streams
    become x_t = sum_s mix_q[s, t] x_s + out_q[t] * y.  `connections` False: no such tensors, every coefficient
    is 1 (with one stream: the ordinary residual sum).  Tensor names: `prefix` + "hc<q>.in" / ".out" / ".mix" and
    `prefix` + "ls<q>" for q = 1 (mixer) and 2 (feed-forward)."""
    streams: int
    hidden: int
    prefix: str
    connections: bool = True
    layer_scale: bool = True


@dataclass(frozen=True)
class LayerSpec:
    """One residual block: which parts, how they are arranged, and the tensor names they load from.

    `arrangement` names a registered block class (`parts.register_block`), which says how many
    norms it has and where they stand: "pre_norm" has two, before the mixer and before the
    feed-forward; "sandwich_norm" has a norm before and a norm behind each sub-layer around a 32-bit stream (norms in the
    order before the mixer, behind it, before the feed-forward, behind it; two norms for a layer without a feed-forward);
    "streams" is pre-norm around several residual streams (`residual`: a `StreamsSpec`) and takes a
    layer without a feed-forward (`ffn` None, one norm); "post_norm" norms the stream after every sum (`residual`: a
    `PostNormSpec`; norms in the order behind the mixer, behind the feed-forward; one norm for a layer without one);
    "parallel" has ONE norm, whose output both sub-layers read, and adds their outputs together (`residual`: a
    `ParallelSpec`).  `norms[i]` loads its weight from `norm_names[i]` (a norm with more tensors finds the others under
    that name plus a suffix of its spec's)."""
    mixer: Any
    ffn: Any
    norms: Tuple[NormSpec, ...]
    norm_names: Tuple[str, ...]
    mixer_prefix: str
    ffn_prefix: str
    arrangement: str = "pre_norm"
    residual: Any = None


@dataclass(frozen=True)
class EmbeddingSpec:
    """Token ids -> rows of the stream.  kind "embedding": a gather from a [vocab, hidden] table, times `scale`;
    `wide`: the rows leave in 32-bit whatever the table is stored in (for a stream that is kept so).  `side_name`: a
    second table [vocab, side_width] whose rows for the step's tokens are handed to the layers (`TokenSideSpec`)."""
    vocab_size: int
    hidden: int
    name: str
    kind: str = "embedding"
    scale: float = 1.0
    wide: bool = False
    side_name: Optional[str] = None
    side_width: int = 0


@dataclass(frozen=True)
class CappedHeadSpec:
    """A logits head whose logits are capped: cap * tanh(logits / cap) (`cap` None: not capped)."""
    vocab_size: int
    hidden: int
    name: Optional[str]
    cap: Optional[float] = None
    required: bool = True
    kind: str = "capped_lm_head"


@dataclass(frozen=True)
class HeadSpec:
    """Normed rows -> logits.  kind "lm_head": a product with a [vocab, hidden] matrix stored under
    `name`; when the file has no such tensor (or `name` is None) the embedding table serves.
    `required`: a random model is written with a matrix of its own.  `scale`: a factor on the logits."""
    vocab_size: int
    hidden: int
    name: Optional[str]
    required: bool = True
    kind: str = "lm_head"
    scale: float = 1.0


@dataclass(frozen=True)
class ScheduleEntry:
    """One stop in the run order: run `layer` (its weights); its mixer uses a cache.

    By default a stop owns a cache of its own and writes it, so a layer that is named at two
    stops keeps two caches and a request's results do not depend on how its tokens were cut
    into steps.  `cache_of = j` (an earlier stop's index in the schedule) makes this stop
    read stop j's cache and write none.
    """
    layer: int
    cache_of: Optional[int] = None
    pass_index: Optional[int] = None    # this stop begins pass t of a looped range: `ModelSpec.pass_input` enters before it


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: Optional[NormSpec]      # None: the head reads the stream as it is
    final_norm_name: Optional[str]
    embed_name: str
    head_name: Optional[str]            # None: logits use the embedding table
    max_position: int
    head_required: bool = True          # False: use `head_name` if the file has it, else the table
    eos_token_ids: Tuple[int, ...] = field(default_factory=tuple)
    embedding: Any = None               # a spec whose `kind` names a registered embedding part; None: EmbeddingSpec
    head: Any = None                    # likewise for the logits head; None: HeadSpec
    pass_input: Any = None              # a spec whose `kind` names a registered pass-input part (stops with a `pass_index`)

    def __post_init__(self):
        if self.embedding is None:
            object.__setattr__(self, "embedding", EmbeddingSpec(self.vocab_size, self.hidden, self.embed_name))
        if self.head is None:
            object.__setattr__(self, "head", HeadSpec(self.vocab_size, self.hidden, self.head_name, self.head_required))

    def validate(self) -> None:
        n = len(self.layers)
        if n == 0:
            raise SpecError("a model needs at least one layer")
        if not self.schedule:
            raise SpecError("the schedule is empty")
        if (self.final_norm is None) != (self.final_norm_name is None):
            raise SpecError("a final norm and the name of its weight come together")
        for i, layer in enumerate(self.layers):
            if len(layer.norms) != len(layer.norm_names):
                raise SpecError(f"layer {i}: {len(layer.norms)} norms but {len(layer.norm_names)} names for their weights")
        for i, e in enumerate(self.schedule):
            if not (0 <= e.layer < n):
                raise SpecError(f"schedule stop {i} names layer {e.layer}, outside 0..{n - 1}")
            if e.cache_of is not None:
                if not (0 <= e.cache_of < i):
                    raise SpecError(f"schedule stop {i} reads the cache of stop {e.cache_of}, which is not an earlier stop")
                if self.schedule[e.cache_of].cache_of is not None:
                    raise SpecError(f"schedule stop {i} reads the cache of stop {e.cache_of}, which owns none")

    def cache_stop(self, stop: int) -> int:
        """The schedule stop whose cache stop `stop` uses (itself unless it reads another's)."""
        e = self.schedule[stop]
        return stop if e.cache_of is None else e.cache_of


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    return tuple(ScheduleEntry(i) for i in range(n_layers))
