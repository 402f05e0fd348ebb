"""Descriptions of a model as data: which parts each layer is made of, with every
size and constant as a field, and the order in which layers run.

A specification names a part kind (the key of a registry in
`wllm_amd.parts.registry`) and carries that part's parameters and the names of
its tensors in the checkpoint.  No part, and nothing in here, knows which model
it belongs to: an architecture is a function from its configuration to a
`ModelPlan`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class NormSpec:
    """kind "rms": y = x * rsqrt(mean(x^2) + eps) * (weight_offset + w); kind "layer": y = (x - mean(x)) *
    rsqrt(mean((x - mean(x))^2) + eps) * (weight_offset + w), a layer norm without a bias.  Computed in float32."""
    size: int
    eps: float
    weight: str                    # tensor name
    weight_offset: float = 0.0     # 1.0: the weight is stored as an offset from one
    kind: str = "rms"


@dataclass(frozen=True)
class PositionSpec:
    """How positions enter a mixer.  kind "rope": rotation of query and key by
    angles position * theta^(-2j/rotary_dim) / scaling_factor, pairing element j with
    j + rotary_dim/2 ("half") or element 2j with 2j + 1 ("interleaved"); elements of a head
    beyond rotary_dim pass unchanged.  kind "none": nothing.
    `ramp` = (factor, original, fast, slow) interpolates the frequencies pair by pair between their plain values
    and those divided by `factor`: with pair(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta),
    lo = max(floor(pair(fast)), 0), hi = min(ceil(pair(slow)), rotary_dim - 1) and
    r_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1), pair j turns by f_j / factor * r_j + f_j * (1 - r_j): pairs
    that make many turns within `original` positions keep their frequency, slow ones are stretched.
    `magnitude`: sine and cosine are both multiplied by it."""
    kind: str = "rope"
    rotary_dim: int = 0
    theta: float = 10000.0
    pairing: str = "half"
    scaling_factor: float = 1.0     # linear scaling: every frequency is divided by it
    ramp: Optional[tuple] = None
    magnitude: float = 1.0


@dataclass(frozen=True)
class MixerSpec:
    """Base of token-mixer specifications; `kind` selects the implementation."""
    kind: str = ""


@dataclass(frozen=True)
class AttentionSpec(MixerSpec):
    """Softmax attention of each query over the earlier keys of its request,
    read from the paged cache.  Query head h uses key/value head
    h // (num_heads // num_kv_heads).  `window` = W limits a query at position p
    to keys p-W+1..p; None is all keys.

    Options beyond the plain form, each off by default.  `softcap` c: the scaled score s becomes
    c * tanh(s / c) before the softmax.  `qk_norm_eps`: after the rotation every query and key
    head is divided by sqrt(mean of its squares + eps) (a norm without a weight).
    `values_are_keys`: there is no value projection; a key head as projected (with its bias,
    before rotation and norm) is also the value head.  `gate_weight`: the concatenated heads are
    multiplied by sigmoid(W_gate h) before the output projection.  `o_bias`: a bias of the output
    projection.  `weights_in_float32`: the softmax weights are not rounded to the values' type before
    they weigh the values (a design that wants its attention weights in 32-bit).
    `value_dim`: the size of a value head where it is not head_dim.  `chunk` c (instead of a window): a
    query sees the earlier keys of its own chunk of c positions counted from 0.  `release_chunk`: the
    chunk by which the cache gives pages back (the owner of a cache that layers with other masks read
    keeps what the widest of them needs; None with `chunk` set: keep everything).  `q_norm_weight` /
    `k_norm_weight` with `band_norm_eps`: an RMS norm with a weight over the whole query projection
    (all heads at once) and over the whole key projection, before the heads are split.
    `gate_per_head`: the gate's projection has one row a head, and its sigmoid multiplies the whole head.
    `owns_cache` False: the layer has no key and value projections (nor their norms); it reads the cache
    of the schedule entry its run names.  `sink`: the softmax's denominator holds exp(sink) once more for
    every head, a term with no key and no value (0.0: one is added to the sum of exponentials).
    `bias_before_norm`: the biases of the query and key projections are added before the norm over the
    whole projection, not behind it.  `output_scale`: the concatenated heads are multiplied by it before
    the output projection (a mixer whose result enters a weighted sum with another's).
    `q_head_norm_weight` / `k_head_norm_weight` with `head_norm_eps`: before the rotation every query head and
    every key head passes an RMS norm over its own elements with a weight of head_dim numbers that the heads
    share.  `sink_weight`: the term in the softmax's denominator is exp(sink_h) of a learned number a head
    (a tensor [num_heads]) instead of the constant `sink`."""
    kind: str = "attention"
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    window: Optional[int] = None
    position: PositionSpec = field(default_factory=PositionSpec)
    q_weight: str = ""
    k_weight: str = ""
    v_weight: str = ""
    o_weight: str = ""
    q_bias: Optional[str] = None
    k_bias: Optional[str] = None
    v_bias: Optional[str] = None
    softcap: Optional[float] = None
    qk_norm_eps: Optional[float] = None
    values_are_keys: bool = False
    gate_weight: Optional[str] = None
    o_bias: Optional[str] = None
    weights_in_float32: bool = False
    value_dim: Optional[int] = None
    chunk: Optional[int] = None
    release_chunk: Optional[int] = None
    q_norm_weight: Optional[str] = None
    k_norm_weight: Optional[str] = None
    band_norm_eps: Optional[float] = None
    gate_per_head: bool = False
    owns_cache: bool = True
    sink: Optional[float] = None
    bias_before_norm: bool = False
    output_scale: float = 1.0
    q_head_norm_weight: Optional[str] = None
    k_head_norm_weight: Optional[str] = None
    head_norm_eps: Optional[float] = None
    sink_weight: Optional[str] = None


@dataclass(frozen=True)
class LatentAttentionSpec(MixerSpec):
    """Causal softmax attention whose keys and values are expanded from one compressed vector a token
    (`kv_rank` numbers, the only thing cached), without positions: c_q = rms(W_dq h) * w_dqn, q = W_uq c_q;
    c = rms(W_dkv h) * w_dkvn; per head k = W_uk c, v = W_uv c; score = q.k * scale; with `sink_weight` the
    softmax's denominator holds exp(sink_h) once more; the concatenated heads are multiplied by
    sigmoid(W_g h) and projected by W_o.
    `q_weight` (then `q_rank` is 0 and the three tensors of the queries' latent are not named): q = W_q h.
    `rope_dim` r > 0 with `position`: a query head is [head_dim elements | r elements], W_dkv has kv_rank + r rows of
    which the last r (not normed) are one more part of the key that all heads share; the r elements of the query heads
    and of that key part turn by the position, and the score is (q . k + q_r . k_r) * scale.  Cached: c and the turned
    key part.  `gate_weight` None: no gate.  `weights_in_float32`: the softmax weights are not rounded to the values' type
    before they weigh the values."""
    kind: str = "latent_attention"
    hidden_size: int = 0
    num_heads: int = 0
    head_dim: int = 0           # query/key size of a head
    value_dim: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    norm_eps: float = 1e-6
    dq_weight: str = ""
    dq_norm_weight: str = ""
    uq_weight: str = ""
    dkv_weight: str = ""
    dkv_norm_weight: str = ""
    uk_weight: str = ""
    uv_weight: str = ""
    sink_weight: Optional[str] = None
    gate_weight: Optional[str] = None
    o_weight: str = ""
    q_weight: Optional[str] = None
    rope_dim: int = 0
    position: PositionSpec = field(default_factory=lambda: PositionSpec(kind="none"))
    weights_in_float32: bool = False


@dataclass(frozen=True)
class StateSpaceSpec(MixerSpec):
    """The selective state-space mixer of Mamba-2.  W_in h is [z: inner | x: inner | B: groups*N | C: groups*N |
    dt: heads] with inner = heads * head_dim; x, B and C pass a causal convolution per channel (`conv_taps`
    taps, a bias) and silu; dt = softplus(dt + dt_bias); per head S = exp(-exp(A_log) dt) S + dt B x^T,
    y = S^T C + D x; y * silu(z) is RMS-normed in `norm_groups` equal parts, times a weight, and projected.
    A request carries S (float32) and the convolution's last taps - 1 inputs."""
    kind: str = "state_space"
    hidden_size: int = 0
    num_heads: int = 0
    head_dim: int = 0
    state_size: int = 0
    groups: int = 1
    conv_taps: int = 4
    norm_groups: int = 1
    norm_eps: float = 1e-6
    in_weight: str = ""
    conv_weight: str = ""
    conv_bias: str = ""
    dt_bias: str = ""
    a_log: str = ""
    d_skip: str = ""
    norm_weight: str = ""
    o_weight: str = ""


@dataclass(frozen=True)
class MatrixMemorySpec(MixerSpec):
    """A recurrent mixer whose state is a matrix a head, S [head_dim, value_dim] in float32, written by outer
    products of keys and values and read by queries (linear attention in its recurrent form):
        q = q_scale * rot(W_q h),  k = k_scale * rot(W_k h),  v = W_v h            (rot: `position`, or none)
        S_t = a_t S_(t-1) + b_t k_t v_t^T,        o_t = S_t^T q_t / den_t
    `gating` "decay": a_t is the head's fixed number of `decays`, b_t = den_t = 1 (retention).
    `gating` "exponential": per head a log input gate i = cap tanh((W_i h + b_i) / cap) and a log forget gate
    f = logsigmoid(cap tanh((W_f h + b_f) / cap)) (`gate_cap` None: no cap), held in range by a running maximum
    m_t = max(f + m_(t-1), i) that starts at 0: a_t = exp(f + m_(t-1) - m_t), b_t = exp(i - m_t); a normaliser
    n_t = a_t n_(t-1) + b_t k_t; den_t = max(|n_t . q_t|, exp(-m_t)) + `den_eps` (the matrix memory of an mLSTM).
    Then every head's o is divided by its root mean square (`norm_eps` inside the root), the heads are
    concatenated, multiplied by `norm_weight` (if named), by act(W_g h) with `gate_activation` "sigmoid" or
    "silu", by `output_scale`, and projected by W_o.  A request carries S (and n, m) from token to token.
    `gating` "forget": a forget gate a channel that also decides what is written (HGRN2).  There is no key
    projection: f = l + (1 - l) * sigmoid(W_f h + b_f) with a lower bound l a channel (`lower_bound`, a tensor
    [heads * head_dim]; not named: 0), S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, den_t = 1; f multiplies the
    rows of S, those of q's channels.  `q_activation` "silu": q = silu(W_q h).  `gate_weight` None: no gate
    behind the norm.  `norm_weight_per_head` False: `norm_weight` has value_dim numbers that the heads share."""
    kind: str = "matrix_memory"
    hidden_size: int = 0
    num_heads: int = 0
    head_dim: int = 0
    value_dim: int = 0
    gating: str = "decay"
    decays: tuple = ()
    gate_cap: Optional[float] = None
    den_eps: float = 1e-6
    q_scale: float = 1.0
    k_scale: float = 1.0
    position: PositionSpec = field(default_factory=lambda: PositionSpec(kind="none"))
    norm_eps: float = 1e-6
    norm_weight: Optional[str] = None
    gate_activation: str = "sigmoid"
    output_scale: float = 1.0
    q_weight: str = ""
    k_weight: str = ""
    v_weight: str = ""
    gate_weight: str = ""
    o_weight: str = ""
    i_weight: Optional[str] = None
    i_bias: Optional[str] = None
    f_weight: Optional[str] = None
    f_bias: Optional[str] = None
    lower_bound: Optional[str] = None
    q_activation: str = "none"
    norm_weight_per_head: bool = True


@dataclass(frozen=True)
class SideBySideSpec(MixerSpec):
    """Two mixers that read the same input; the result is the sum of theirs (each weighs its own with its
    `output_scale`).  At most one of the two pages a cache and at most one carries a state."""
    kind: str = "side_by_side"
    left: MixerSpec = field(default_factory=MixerSpec)
    right: MixerSpec = field(default_factory=MixerSpec)


@dataclass(frozen=True)
class TokenSideSpec:
    """A per-layer token input behind the feed-forward: e = table[token][offset : offset + dim];
    g = act(W_gate x) * e; y = W_proj g; x += rms(y) * w_norm.  The table [vocab, D] is shared by
    the layers, each reading its own band of columns."""
    hidden_size: int = 0
    vocab_size: int = 0
    dim: int = 0
    table: str = ""
    table_width: int = 0
    offset: int = 0
    activation: str = "gelu_tanh"
    gate_weight: str = ""
    proj_weight: str = ""
    norm: Optional[NormSpec] = None


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str = ""


@dataclass(frozen=True)
class GatedMLPSpec(FeedForwardSpec):
    """down(act(gate(x)) * up(x)) without biases; `activation` names the
    nonlinearity ("gelu_tanh")."""
    kind: str = "gated_mlp"
    hidden_size: int = 0
    intermediate_size: int = 0
    activation: str = "gelu_tanh"
    gate_weight: str = ""
    up_weight: str = ""
    down_weight: str = ""


@dataclass(frozen=True)
class MixtureOfExpertsSpec(FeedForwardSpec):
    """`num_experts` gated feed-forwards without biases, down_e(act(gate_e(x)) * up_e(x)), of which a token
    uses `top`.  Router: z = W_router x in float32, s = softmax(z) over all experts.  The experts form
    `num_groups` equal groups of neighbours; a group's score is its largest s, and only experts of the
    `keep_groups` best groups can be chosen (one group, one kept: no limit).  The `top` allowed experts with
    the largest s are chosen, their weights are their s divided by the sum of the chosen (+ `weight_eps`),
    and the result is the weighted sum of their outputs.  `expert_prefix` + "<e>." + `gate_name` ... name an
    expert's tensors.  `scoring` "sigmoid": s = sigmoid(z), every expert by itself.  `normalize` False: the
    weights are the chosen s themselves.  `weight_on_input`: the weight multiplies the expert's input instead of
    its output, y = sum of expert_e(w_e x).  `shared`: one more gated feed-forward that every token uses, added to
    the experts' sum."""
    kind: str = "mixture_of_experts"
    hidden_size: int = 0
    intermediate_size: int = 0
    num_experts: int = 0
    top: int = 1
    num_groups: int = 1
    keep_groups: int = 1
    weight_eps: float = 1e-20
    activation: str = "silu"
    router_weight: str = ""
    expert_prefix: str = ""
    gate_name: str = "gate"
    up_name: str = "up"
    down_name: str = "down"
    scoring: str = "softmax"
    normalize: bool = True
    weight_on_input: bool = False
    shared: Optional[GatedMLPSpec] = None


@dataclass(frozen=True)
class InputConvSpec:
    """A short causal convolution over time on each channel of what a sublayer reads: h_t becomes
    h_t + sum_j w[:, j] * h_(t - taps + 1 + j) with zeros before the sequence's start; `weight` [size, taps],
    no bias.  A request carries its last taps - 1 inputs."""
    size: int
    taps: int
    weight: str


@dataclass(frozen=True)
class BlockSpec:
    """One layer: a mixer and a feed-forward with their norms, and how they are
    arranged around the residual stream.  "pre_norm": x += mixer(norm(x));
    x += ffn(norm(x)) (`feed_forward` and its norm may be None: then the layer is its mixer alone).  "parallel": h = mixer_norm(x); x += mixer(h) + ffn(h): one norm, both
    sublayers read it (`feed_forward_norm` is None, and `feed_forward` may be None: then the
    layer is its mixer alone).  "sandwich": x += post(mixer(pre(x))); x += post(ffn(pre(x))) with the
    two norms behind the sublayers in `mixer_post_norm` and `feed_forward_post_norm` (a layer without a
    feed-forward has neither of its norms), then the layer's token input (`side`), if it has one.
    "post_norm": x += post(mixer(x)); x += post(ffn(x)): the sublayers read the stream itself and the only norms
    stand behind them (`mixer_norm` and `feed_forward_norm` are None).  With `mixer_input_conv` /
    `feed_forward_input_conv` what a sublayer reads first passes a short convolution over time (`InputConvSpec`)."""
    mixer: MixerSpec
    feed_forward: Optional[FeedForwardSpec]
    mixer_norm: Optional[NormSpec]
    feed_forward_norm: Optional[NormSpec]
    arrangement: str = "pre_norm"
    mixer_post_norm: Optional[NormSpec] = None
    feed_forward_post_norm: Optional[NormSpec] = None
    side: Optional[TokenSideSpec] = None
    mixer_input_conv: Optional[InputConvSpec] = None
    feed_forward_input_conv: Optional[InputConvSpec] = None


@dataclass(frozen=True)
class EmbeddingSpec:
    """x = table[id] * scale.  `scale_in_model_dtype`: the factor is rounded to
    the model's dtype before use, as a buffer cast with the model would be."""
    vocab_size: int
    hidden_size: int
    weight: str
    scale: float = 1.0
    scale_in_model_dtype: bool = False


@dataclass(frozen=True)
class HeadSpec:
    """logits = hidden @ W^T; W is the embedding table when `weight` is None.  `tied_checkpoint_name`:
    the name under which a checkpoint of tied weights may still store the head; such a tensor is
    accepted if it equals the table.  `logit_scale`: the logits are multiplied by it (in float32)."""
    vocab_size: int
    hidden_size: int
    weight: Optional[str] = None
    tied_checkpoint_name: Optional[str] = None
    logit_scale: float = 1.0


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `layer` indexes ModelPlan.layers (the same layer may
    be named by several entries: its weights are shared, each run has a cache
    of its own).  `reads_cache_of` = index of an earlier schedule entry whose
    cache this run reads instead of writing one.  `adds_embedding`: before this run the
    embedding output (the stream as it was before the first run) is added to the stream, as
    a model does that sends the stream through a span of its layers several times."""
    layer: int
    reads_cache_of: Optional[int] = None
    adds_embedding: bool = False


@dataclass(frozen=True)
class ModelPlan:
    embedding: EmbeddingSpec
    layers: tuple
    schedule: tuple
    final_norm: NormSpec
    head: HeadSpec
    max_positions: int
    # tensor names that may appear in a checkpoint and are ignored
    ignored_tensor_suffixes: tuple = ()

    def __post_init__(self):
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ValueError(f"schedule entry {i} names layer {e.layer}, the plan has {n}")
            if e.reads_cache_of is not None:
                j = e.reads_cache_of
                if not 0 <= j < i:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {j}, which is not an earlier entry")
                if self.schedule[j].reads_cache_of is not None:
                    raise ValueError(f"schedule entry {i} reads the cache of entry {j}, which owns none")
