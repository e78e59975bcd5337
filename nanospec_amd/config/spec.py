"""Typed descriptions of a model as data: which parts each layer is made of, with every size
and constant as a field, and the order in which the layers run.

A ``ModelSpec`` is what an architecture's configuration is turned into (see
``config/registry.py``); ``parts/`` builds the runnable model from it.  No part reads an
architecture's configuration: it sees only its own spec.  A spec class carries a ``kind``
string; ``parts/registry.py`` maps (role, kind) to the class that implements it, so a new
mixer, feed-forward, norm or position encoding is one spec dataclass plus one implementation
registered under a new kind.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import ClassVar


@dataclass(frozen=True)
class RMSNormSpec:
    """y = w * x / sqrt(mean(x^2) + eps) over the last axis.  ``unit_offset``: the stored weight is the factor minus one: the
    factor is 1 + w, formed in 32-bit."""

    kind: ClassVar[str] = "rmsnorm"
    dim: int
    eps: float
    unit_offset: bool = False


@dataclass(frozen=True)
class NoNormSpec:
    """No norm: y = x.  In front of a sublayer of a block over a 32-bit stream it means that the sublayer reads the stream
    itself (rounded to the model's precision)."""

    kind: ClassVar[str] = "none"
    dim: int


@dataclass(frozen=True)
class RopeSpec:
    """Rotary position encoding over the first ``rotary_dim`` elements of a head; pair j is elements j and
    j + rotary_dim/2 (``interleaved``: 2j and 2j + 1).  ``scaling`` is None or the llama3 frequency scaling as
    (factor, low_freq_factor, high_freq_factor, original_max_position_embeddings).  ``cos_sin_factor`` multiplies
    cosine and sine.  ``yarn`` is None or (factor, original, fast, slow): with d(t) = rotary_dim ln(original / (2 pi t)) /
    (2 ln theta), lo = max(floor(d(fast)), 0), hi = min(ceil(d(slow)), rotary_dim - 1) and ramp_j = clamp((j - lo) /
    max(hi - lo, 0.001), 0, 1), pair j turns at f_j / factor * ramp_j + f_j (1 - ramp_j), and cosine and sine are
    multiplied by 0.1 ln(factor) + 1 (on top of ``cos_sin_factor``)."""

    kind: ClassVar[str] = "rope"
    rotary_dim: int
    theta: float
    scaling: tuple[float, float, float, int] | None = None
    yarn: tuple[float, float, float, float] | None = None
    max_positions: int | None = None  # None = unbounded
    interleaved: bool = False
    cos_sin_factor: float = 1.0


@dataclass(frozen=True)
class NoPositionSpec:
    kind: ClassVar[str] = "none"


@dataclass(frozen=True)
class AttentionSpec:
    """Soft-max attention over a key/value cache with grouped query heads.  ``window`` = 0 sees
    all earlier keys; ``window`` = w sees the last w positions (its own included)."""

    kind: ClassVar[str] = "attention"
    hidden: int
    heads: int
    kv_heads: int
    head_dim: int
    position: object  # a position spec (RopeSpec, NoPositionSpec, ...)
    softmax_scale: float  # multiplies q.k before the soft-max
    window: int = 0
    # Options, each off at its default.  A layer that sets any of them runs the general attention path.
    value_dim: int = 0  # size of a value head if it is not ``head_dim``
    qk_norm_eps: float | None = None  # q and k of every head are divided by sqrt(mean(x^2) + eps), no weight, before the scores
    score_cap: float = 0.0  # > 0: a score s (after the scale) becomes cap * tanh(s / cap)
    chunk: int = 0  # > 0: a query sees a key only inside its own chunk of this many positions, counted from position 0
    sink: bool = False  # the soft-max's denominator holds one more term of score 0, which has no value
    own_kv: bool = True  # False: no key/value projections; the layer reads the cache of the run-order entry it names
    names: tuple[str, str, str, str] = ("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight")  # after the prefix
    bias: bool = False  # the four projections have biases, named as their matrices plus ``bias_suffix``
    bias_suffix: str = ".b"
    # q (and k) pass an RMS norm over the WHOLE projection, all heads at once, with a weight per channel and this eps;
    # the weights are named as the q and k matrices plus ``whole_norm_suffix``
    whole_norm_eps: float | None = None
    whole_norm_suffix: str = ".norm"
    slope_exp: float = 0.0  # > 0: head h of H loses 2^(-slope_exp (h + 1) / H) * (query position - key position) from its score
    # values across layers: "source" keeps this layer's values of the step's tokens for later layers; "mix" turns this
    # layer's values into (1 - m) v + m v_source before they are cached, m one stored value named ``value_mix_name``
    # (a "source" layer may hold that tensor too; it is not read)
    value_mix: str = ""
    value_mix_name: str = "vmix"
    # q and k of every head pass an RMS norm over the head with a weight [head_dim] that all heads share and this eps,
    # before the rotation; the weights are named as the q and k matrices plus ``head_norm_suffix``
    head_norm_eps: float | None = None
    head_norm_suffix: str = ".norm"
    # the key projection's raw output (bias added, no norm, no rotation) serves as the values too; the layer has no value matrix
    value_is_key: bool = False
    # a learned sink: the soft-max's denominator holds one more term exp(sink_h), one stored value per head (the tensor
    # ``sink_name`` [heads] after the prefix), which has no key and no value and is not scaled
    sink_name: str = ""
    # an output gate: the concatenated heads' outputs are multiplied, channel by channel, by sigmoid(W_g h) before the output
    # projection; W_g [heads * value size, hidden] is the tensor ``gate_name`` after the prefix and reads the mixer's input
    out_gate: bool = False
    gate_name: str = "g"

    @property
    def v_dim(self) -> int:
        return self.value_dim or self.head_dim

    @property
    def general(self) -> bool:
        return bool(self.value_dim not in (0, self.head_dim) or self.qk_norm_eps is not None or self.score_cap or self.chunk or self.sink
                    or not self.own_kv or self.bias or self.whole_norm_eps is not None or self.slope_exp or self.value_mix
                    or self.head_norm_eps is not None or self.value_is_key or self.sink_name or self.out_gate)


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Soft-max attention whose keys and values come from one cached latent per token.  With h the input:
    c_q = norm(W_dq h); q = W_uq c_q (``q_rank`` = 0: q = W_uq h, no query latent), per head [dim unrotated | rot rotated];  W_dkv h = [latent | rot]: c = norm(first part),
    the rest is one rotated key part for all heads;  per head k = [W_uk c | rotated part], v = W_uv c;
    score = q . k * softmax_scale over the last ``window`` positions (0: all);  head outputs times sigmoid(W_g h) per head
    if ``gate``;  then W_o.  The two norms are RMS norms with plain weights.  Only c and the rotated part are cached.
    ``sink_name``: a learned sink as in ``AttentionSpec`` (one value per head, "" for none)."""

    kind: ClassVar[str] = "latent_attention"
    hidden: int
    heads: int
    head_dim: int  # unrotated query/key channels of a head
    rot_dim: int  # rotated ones
    value_dim: int
    q_rank: int
    kv_rank: int
    position: object  # a RopeSpec over rot_dim channels
    softmax_scale: float
    norm_eps: float
    window: int = 0
    gate: bool = True
    # after the prefix: W_dq, its norm, W_uq, W_dkv, its norm, W_uk, W_uv, W_g, W_o
    names: tuple = ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "g", "o")
    sink_name: str = ""


@dataclass(frozen=True)
class ChannelDeltaSpec:
    """The gated delta rule with one decay per head and key channel, behind short causal convolutions of q, k and v.
    Per head, S [key_dim, value_dim] in 32-bit: S = g_t * S (by key channel); u = beta_t (v_t - S^T k_t); S = S + k_t u^T;
    o_t = S^T q_t; then o / rms(o) * weight * sigmoid(gate), and the output projection.  The decay's and the gate's
    projections are products of two matrices whose inner sizes (``decay_rank``, ``gate_rank``) are read from the
    checkpoint when None; random weights need them given."""

    kind: ClassVar[str] = "channel_delta"
    hidden: int
    heads: int
    kv_heads: int
    key_dim: int
    value_dim: int
    conv: int  # taps of the convolutions, the current token's included
    norm_eps: float
    decay_rank: int | None = None
    gate_rank: int | None = None


@dataclass(frozen=True)
class MatrixMemorySpec:
    """A matrix memory with exponential gates (the mLSTM of xLSTM).  With h the input, per head: q = W_q h key_dim^(-1/2),
    k = W_k h [key_dim], v = W_v h [value_dim], and two gates in the logarithm, i = cap tanh((W_i h + b_i) / cap) and
    f = logsigmoid(cap tanh((W_f h + b_f) / cap)).  S [key_dim, value_dim], n [key_dim] and a running maximum m start at zero:
        m' = max(f + m, i);  S <- exp(f + m - m') S + exp(i - m') k v^T;  n likewise with k alone;
        o = S^T q / (max(|n . q|, exp(-m')) + den_eps)
    then o / rms(o) per head (``norm_eps``) times a weight over all heads' channels, times sigmoid(W_g h), through W_o.
    Gates, state and read-out are 32-bit.  ``names``: q, k, v, the output gate, o, the norm weight, the two gate
    projections (their biases are these names plus ``bias_suffix``), after the prefix."""

    kind: ClassVar[str] = "matrix_memory"
    hidden: int
    heads: int
    key_dim: int
    value_dim: int
    gate_cap: float
    norm_eps: float
    den_eps: float = 1e-6
    names: tuple = ("q", "k", "v", "g", "o", "norm", "i", "f")
    bias_suffix: str = ".b"


@dataclass(frozen=True)
class RetentionSpec:
    """Retention: linear attention with one fixed decay per head, no soft-max and no denominator.  With h the input, per
    head: q = W_q h, k = W_k h [key_dim], v = W_v h [value_dim]; q and k are rotated by their position (``position``), k is
    then multiplied by ``key_scale``;  S [key_dim, value_dim] starts at zero:
        S_t = decay_h S_(t-1) + k_t v_t^T;   o_t = S_t^T q_t
    then o / rms(o) per head (``norm_eps``, no weight), times silu(W_g h), through W_o.  Rotation, decay, state and read-out
    are 32-bit.  ``names``: q, k, v, the gate, o after the prefix."""

    kind: ClassVar[str] = "retention"
    hidden: int
    heads: int
    key_dim: int
    value_dim: int
    decay: tuple[float, ...]  # one per head
    position: object
    key_scale: float
    norm_eps: float
    names: tuple = ("q", "k", "v", "g", "o")


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers side by side that read the same input: left_scale * left(h) + right_scale * right(h).  Each keeps what it
    keeps (pages, state); their tensors lie under the two prefixes."""

    kind: ClassVar[str] = "parallel"
    left: object
    right: object
    left_scale: float = 1.0
    right_scale: float = 1.0
    prefixes: tuple[str, str] = ("left.", "right.")


@dataclass(frozen=True)
class ClippedGLUSpec:
    """One gated feed-forward with clipped inputs: g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit);
    W_down (g sigmoid(alpha g) (u + shift)).  No biases.  An infinite ``limit`` clips nothing; with alpha = 1 and shift = 0
    that is the gated SiLU form, W_down (silu(W_gate h) * W_up h)."""

    intermediate: int
    limit: float = float("inf")
    alpha: float = 1.702
    shift: float = 1.0


@dataclass(frozen=True)
class ClippedGLUFFSpec:
    """A dense feed-forward of the ``ClippedGLUSpec`` form.  ``names``: gate, up, down after the prefix."""

    kind: ClassVar[str] = "clipped_glu"
    hidden: int
    glu: ClippedGLUSpec
    names: tuple[str, str, str] = ("gate", "up", "down")


@dataclass(frozen=True)
class MoESpec:
    """A mixture of ``experts`` clipped-GLU feed-forwards of which each token uses ``top``: router logits z = W_r h + b in
    32-bit, the ``top`` largest are chosen and weighted by the soft-max over the chosen logits alone; ``shared`` (or None)
    is one more expert that every token uses with weight 1.  Tensor names after the prefix: ``expert_prefix`` + index + "."
    + gate / up / down, ``router`` and its bias ("" for none), ``shared_prefix`` + gate / up / down.
    ``score`` = "sigmoid": the scores are s = sigmoid(z); the choice goes by s + correction (the tensor ``correction_name``
    [experts], "" for none) and the weights are the chosen experts' s themselves, not renormalized.  ``groups`` > 1: the
    experts form that many equal groups of neighbours; a group's score is the sum of its two largest choice scores, and only
    experts of the ``keep_groups`` best groups can be chosen."""

    kind: ClassVar[str] = "moe"
    hidden: int
    experts: int
    top: int
    expert: ClippedGLUSpec
    shared: ClippedGLUSpec | None = None
    names: tuple[str, str, str] = ("gate", "up", "down")
    expert_prefix: str = "e"
    router_name: str = "router"
    router_bias_name: str = "router.b"
    shared_prefix: str = "shared."
    score: str = "softmax"
    correction_name: str = ""
    groups: int = 1
    keep_groups: int = 1


@dataclass(frozen=True)
class TokenSideSpec:
    """A per-layer input chosen by the token: e = table[token][offset : offset + dim] of a table [vocab, table_dim] that the
    layers share; y = W_proj (gelu_tanh(W_gate x) * e).  ``table_name`` is the whole tensor name of the table; ``names``: the
    gate and the projection after the prefix."""

    kind: ClassVar[str] = "token_side"
    hidden: int
    vocab: int
    dim: int
    offset: int
    table_dim: int
    table_name: str = "side.embed"
    names: tuple[str, str] = ("gate", "proj")


@dataclass(frozen=True)
class DenseFFSpec:
    """down(act(up(x))), dense, no bias.  ``names``: the two matrices after the prefix."""

    kind: ClassVar[str] = "dense"
    hidden: int
    intermediate: int
    activation: str = "gelu_tanh"
    names: tuple[str, str] = ("up", "down")


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(silu(gate(x)) * up(x)), dense.  ``bias``: the three projections have biases, named as their matrices plus
    ``bias_suffix``.  ``names``: the three matrices after the prefix."""

    kind: ClassVar[str] = "swiglu"
    hidden: int
    intermediate: int
    bias: bool = False
    names: tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")
    bias_suffix: str = ".b"


@dataclass(frozen=True)
class PreNormBlockSpec:
    """x = x + mixer(norm1(x)); x = x + feed_forward(norm2(x)).  ``prefix`` is the layer's
    tensor-name prefix in the checkpoint, e.g. ``model.layers.3.``; the four names that follow it are the
    architecture's own and are appended to it: the two norms' weight tensors and the prefixes under which
    the mixer and the feed-forward find their tensors (None: the part's ``kind`` and a dot)."""

    kind: ClassVar[str] = "prenorm"
    prefix: str
    mixer_norm: object
    mixer: object
    ffn_norm: object
    ffn: object
    mixer_norm_name: str = "mixer_norm.weight"
    mixer_prefix: str | None = None
    ffn_norm_name: str = "ffn_norm.weight"
    ffn_prefix: str | None = None


@dataclass(frozen=True)
class StreamBlockSpec:
    """A pre-norm block over a residual stream that is kept in 32-bit and may be ``streams`` parallel streams x_1 .. x_S
    (hyper-connections).  For sublayer q (the mixer, then the feed-forward, which may be None):
        u = sum_s in_q[s] x_s;  y = sublayer(norm_q(u));  x_t <- sum_s mix_q[s, t] x_s + mult * out_q[t] * y   (all t at once)
    with the tensors ``prefix + hc_names[q] + "in" | "out" | "mix"``.  ``streams`` = 0: one stream and no such tensors,
    x <- x + mult * sublayer(norm(x)).  ``mixer_post_norm`` / ``ffn_post_norm`` (norm specs or None): a second norm behind
    the sublayer, y = post_norm(sublayer(norm(u))), in 32-bit on the way into the streams.  A norm in front may be a
    ``NoNormSpec``: the sublayer then reads u itself.  ``extra`` (or None): a third sublayer behind the feed-forward, a part
    of the "ffn" role with a norm in front (``extra_norm``) and optionally behind (``extra_post_norm``)."""

    kind: ClassVar[str] = "streams"
    prefix: str
    mixer_norm: object
    mixer: object
    ffn_norm: object | None
    ffn: object | None
    streams: int = 0
    mult: float = 1.0
    mixer_norm_name: str = "norm1"
    mixer_prefix: str = "mix."
    ffn_norm_name: str = "norm2"
    ffn_prefix: str = "mlp."
    hc_names: tuple[str, str] = ("hc1.", "hc2.")
    mixer_post_norm: object | None = None
    ffn_post_norm: object | None = None
    mixer_post_norm_name: str = "norm1b"
    ffn_post_norm_name: str = "norm2b"
    extra: object | None = None
    extra_norm: object | None = None
    extra_post_norm: object | None = None
    extra_prefix: str = "side."
    extra_norm_name: str = "norm3"
    extra_post_norm_name: str = "norm3b"


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.  ``layer`` indexes ``ModelSpec.layers`` (a layer may be named
    by several entries: its weights are used again, each entry with a cache of its own).
    ``cache_from`` names an EARLIER entry of the run order whose cache this entry reads instead
    of writing one of its own.  ``enters``: this entry is the first of pass number ``enters`` over a range of layers
    (``ModelSpec.passes``): what the pass adds to the stream is added right before the entry runs."""

    layer: int
    cache_from: int | None = None
    enters: int | None = None


@dataclass(frozen=True)
class PassSpec:
    """What is added to the residual stream in front of each pass over a range of layers that runs several times with the
    same weights: row t of the tensor ``name`` [times, hidden] in front of pass t, and, in front of every pass but the
    first if ``add_embedding``, the embedding's output (the stream as it was before the first layer)."""

    name: str
    times: int
    add_embedding: bool = True


@dataclass(frozen=True)
class PairEmbeddingSpec:
    """A second embedding table, added to the first: row (previous token * mul_prev + token * mul_cur) mod buckets, and
    row ``buckets`` (the last of its buckets + 1 rows) for a sequence's first token.  The previous token of a request is
    kept in its state slot between steps."""

    name: str  # tensor name of the [buckets + 1, hidden] table
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class ModelSpec:
    vocab_size: int
    hidden: int
    embed_name: str  # tensor name of the [vocab, hidden] table
    layers: tuple  # block specs
    run_order: tuple[LayerCall, ...]
    final_norm: object
    final_norm_name: str
    head_name: str  # tensor name of the [vocab, hidden] output matrix
    tie_head: bool  # a missing head tensor is the embedding table
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)
    # what an architecture may do at the two ends of the stack; the defaults do nothing and launch nothing
    embed_scale: float = 1.0  # the embedding rows are multiplied by this as they enter the stream
    logit_scale: float = 1.0  # the head's 32-bit logits are multiplied by this ...
    logit_softcap: float = 0.0  # ... and then, if > 0, become softcap * tanh(logit / softcap)
    # the residual stream between the blocks: 0 = one stream in the model's precision; S >= 1 = S copies in 32-bit, all
    # equal to the embedding's output at the start and added up before the last norm (blocks of kind "streams")
    streams: int = 0
    # tensor-name prefixes that a checkpoint may hold although the model reads nothing under them (the tensors of a
    # sublayer that a layer does not have); anything else that is unexpected is an error
    unread_prefixes: tuple[str, ...] = field(default_factory=tuple)
    pair_embedding: PairEmbeddingSpec | None = None  # models that carry 32-bit streams only
    passes: PassSpec | None = None  # models that carry 32-bit streams only; see ``LayerCall.enters``

    def __post_init__(self) -> None:
        for pos, call in enumerate(self.run_order):
            if not 0 <= call.layer < len(self.layers):
                raise ValueError(f"run order entry {pos} names layer {call.layer}, but there are {len(self.layers)} layers")
            if call.enters is not None and (self.passes is None or not 0 <= call.enters < self.passes.times):
                raise ValueError(f"run order entry {pos} starts pass {call.enters}, which the model does not have")
            if call.cache_from is not None:
                if not 0 <= call.cache_from < pos:
                    raise ValueError(f"run order entry {pos} reads the cache of entry {call.cache_from}, which is not an earlier entry")
                if self.run_order[call.cache_from].cache_from is not None:
                    raise ValueError(f"run order entry {pos} reads the cache of entry {call.cache_from}, which has no cache of its own")
