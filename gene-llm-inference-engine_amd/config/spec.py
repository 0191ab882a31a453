"""Architecture-neutral description of a model: what the engine builds from.

An architecture's own configuration class (for instance `LlamaConfig`) reads config.json and
translates itself into a `ModelSpec`: a list of layers, each naming its mixer, feed-forward,
norms and position encoding with all sizes, constants and tensor names as fields, and a run
order.  Nothing below this file knows which architecture a spec came from.

Every part spec is a frozen dataclass with a class attribute `kind`; the parts registry maps
`kind` to the class that implements it, so a new kind of part needs a spec class, an
implementation and one `register_*` call.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, ClassVar, Optional, Tuple


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of the pairs (k, k + head_dim/2) of every head by pos * f_k, with f_k = theta^(-2k/head_dim) unless the
    architecture gives its own `frequencies` (head_dim/2 numbers: whatever rule stretches or blends them is the
    architecture's, applied where it builds this spec).  `magnitude` multiplies every cosine and sine (rules that stretch the
    frequencies for longer contexts may lengthen the turned vectors a little)."""
    kind: ClassVar[str] = "rotary_half_split"
    head_dim: int
    theta: float
    frequencies: Optional[Tuple[float, ...]] = None
    magnitude: float = 1.0

    def __post_init__(self):
        if self.frequencies is not None and len(self.frequencies) != self.head_dim // 2:
            raise ValueError(f"a rotation of heads of {self.head_dim} channels needs {self.head_dim // 2} frequencies, not {len(self.frequencies)}")


@dataclass(frozen=True)
class PartialRotarySpec:
    """Rotation of the pairs (k, k + rotary_dim/2) of the first `rotary_dim` channels of every head by pos * f_k; the other
    channels of the head pass unchanged.  f_k = theta^(-2k/rotary_dim) unless the architecture gives its own `frequencies`;
    `magnitude` multiplies every cosine and sine."""
    kind: ClassVar[str] = "rotary_partial"
    head_dim: int
    rotary_dim: int
    theta: float
    frequencies: Optional[Tuple[float, ...]] = None
    magnitude: float = 1.0

    def __post_init__(self):
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= self.head_dim:
            raise ValueError(f"a rotation of {self.rotary_dim} of a head's {self.head_dim} channels: an even number within the head is needed")
        if self.frequencies is not None and len(self.frequencies) != self.rotary_dim // 2:
            raise ValueError(f"a rotation of {self.rotary_dim} channels needs {self.rotary_dim // 2} frequencies, not {len(self.frequencies)}")


@dataclass(frozen=True)
class InterleavedRotarySpec:
    """Rotation of the neighbouring pairs (2k, 2k + 1) of `rotary_dim` channels by pos * f_k, f_k = theta^(-2k/rotary_dim) unless
    the architecture gives its own `frequencies`.  It only makes the cosines and sines; the mixer that names it says which
    channels they turn."""
    kind: ClassVar[str] = "rotary_interleaved"
    rotary_dim: int
    theta: float
    frequencies: Optional[Tuple[float, ...]] = None
    magnitude: float = 1.0

    def __post_init__(self):
        if self.rotary_dim % 2 or self.rotary_dim <= 0:
            raise ValueError(f"a rotation of pairs needs an even number of channels, not {self.rotary_dim}")
        if self.frequencies is not None and len(self.frequencies) != self.rotary_dim // 2:
            raise ValueError(f"a rotation of {self.rotary_dim} channels needs {self.rotary_dim // 2} frequencies, not {len(self.frequencies)}")


@dataclass(frozen=True)
class RmsNormSpec:
    """x / sqrt(mean(x^2) + eps) * (weight + weight_offset): an architecture that stores its norm weights around zero says
    weight_offset = 1."""
    kind: ClassVar[str] = "rmsnorm"
    size: int
    eps: float
    weight: str                      # tensor name
    weight_offset: float = 0.0


@dataclass(frozen=True)
class AttentionSpec:
    """Causal attention with grouped key/value heads over a paged cache."""
    kind: ClassVar[str] = "attention"
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    q_proj: str
    k_proj: str
    v_proj: str
    o_proj: str
    position: Optional[Any] = None   # a position-encoding spec, or None for no rotation
    window: Optional[int] = None     # keys further back than this many positions are not seen
    # What follows is absent (None) in the plain attention of a Llama layer; a layer that names any of it takes the general kernels.
    value_dim: Optional[int] = None  # channels of a value head, where they differ from those of a query/key head
    scale: Optional[float] = None    # what the scores are multiplied by; head_dim^(-1/2) if not given
    chunk: Optional[int] = None      # position i sees j <= i only if floor(i / chunk) = floor(j / chunk), counted from the sequence's start
    sinks: Optional[str] = None      # tensor [heads]: a learned score per head that joins the softmax's denominator and has no value
    q_norm: Optional[str] = None     # tensors [head_dim]: RMS norm of every query (key) head with these weights, before the rotation
    k_norm: Optional[str] = None
    qk_norm_eps: float = 1e-6
    head_gate: Optional[str] = None  # tensor [heads, hidden]: head h's output is multiplied by sigmoid(row h of it . the mixer's input)
    keep_chunk: Optional[int] = None # the pages of chunks gone by are given back: set where this entry and every reader of its pages cut their masks alike
    q_bias: Optional[str] = None     # tensors [heads*head_dim], [kv_heads*head_dim], [kv_heads*value_dim]: added to the projections
    k_bias: Optional[str] = None
    v_bias: Optional[str] = None
    # Values blended across layers: the layers that name one `value_family` share the values of the family's first layer in
    # the run order (the one without `value_blend`); each other one caches and attends over (1 - w) v + w v_first, with w the
    # number in its tensor `value_blend` and v_first the first layer's values of the same row.
    value_family: Optional[str] = None
    value_blend: Optional[str] = None
    # Every query and key head divided by its root mean square over the head (eps `qk_norm_eps` inside the root), without weights and
    # behind the rotation (q_norm and k_norm must then be absent).
    qk_unit_rms: bool = False
    # q_norm and k_norm taken over all heads of the projection at once (tensors [heads*head_dim], [kv_heads*head_dim]) instead of
    # head by head.
    qk_norm_whole: bool = False
    score_cap: Optional[float] = None    # a scaled score s becomes cap * tanh(s / cap) before the softmax


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose queries and keys/values pass through low-rank latents.  c_q = norm(W_dq x), q = W_uq c_q, per head
    [head_dim unrotated | rotary_dim rotated]; W_dkv x = [kv_rank | rotary_dim]: the first part, normed, is the latent c, the
    second one rotated key part for all heads; per head the unrotated key is W_uk c and the value W_uv c, so that only c and
    the rotated part are cached.  score = (q_plain . k_plain + q_rot . k_rot) * scale; causal, optionally windowed."""
    kind: ClassVar[str] = "latent_attention"
    hidden_size: int
    n_heads: int
    head_dim: int                    # unrotated channels of a query/key head
    rotary_dim: int                  # rotated channels
    value_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    norm_eps: float
    dq_proj: str
    dq_norm: str
    uq_proj: str
    dkv_proj: str
    dkv_norm: str
    uk_proj: str
    uv_proj: str
    o_proj: str
    position: Optional[Any] = None   # a spec that gives cosines and sines for rotary_dim / 2 neighbouring pairs
    window: Optional[int] = None
    head_gate: Optional[str] = None  # tensor [heads, hidden]: head h's output is multiplied by sigmoid(row h of it . the mixer's input)


@dataclass(frozen=True)
class TokenShiftSpec:
    """A mixer whose input h is first blended, channel by channel, with the input of the token before: h + (h_before - h) * w, with
    `weight` [hidden] and h_before the row the request's previous token brought, before its own blending (zeros for a request's
    first token).  `inner` is the spec of the mixer that reads the blended rows; it keeps the cache it would keep alone, and the
    last row's h is kept per request beside it."""
    kind: ClassVar[str] = "token_shift"
    hidden_size: int
    weight: str
    inner: Any


@dataclass(frozen=True)
class SwiGluSpec:
    """down( act(gate(x)) * up(x) ), no biases; act is SiLU, or the tanh form of GELU (`activation` = "gelu_tanh"), or, as
    "swish_clamped" with `activation_limit` L: g <- min(gate(x), L), u <- clamp(up(x), -L, L), down(g sigmoid(1.702 g) (u + 1))."""
    kind: ClassVar[str] = "swiglu"
    hidden_size: int
    intermediate_size: int
    gate_proj: str
    up_proj: str
    down_proj: str
    activation: str = "silu"
    activation_limit: float = 0.0


@dataclass(frozen=True)
class DenseMlpSpec:
    """down(act(up(x))), no gate, no biases.  `activation` "xielu": with the two numbers (p, q) of the tensor `activation_params`,
    and a = softplus(p), b = 1/2 + softplus(q): act(z) = z/2 + a z^2 on the right of zero and z/2 + b (e^z - 1 - z) on the left."""
    kind: ClassVar[str] = "dense_mlp"
    hidden_size: int
    intermediate_size: int
    up_proj: str
    down_proj: str
    activation: str = "xielu"
    activation_params: Optional[str] = None


@dataclass(frozen=True)
class GatedDeltaSpec:
    """The gated delta rule: per head a memory M [key_dim, value_dim], zero at a sequence's start.  A token first lets it decay,
    M <- d M; then corrects what it holds along the token's key towards the token's value, M <- M + k e^T with e = s (v - M^T k);
    then reads it with the query, y = M^T q (so the read-out sees the token's own correction).  Per head the decay is
    d = exp(-exp(a_log) softplus(a(x) + dt_bias)) and the step size s = sigmoid(b(x)).  q and k (n_kv_heads heads, head h of
    the memory uses q/k head h // (n_heads / n_kv_heads)) and v pass a causal convolution of `conv_taps` taps per channel
    (tensors [channels, taps], the last tap the token's own) and SiLU; q and k are then divided by sqrt(sum of squares + 1e-6),
    q also by sqrt(key_dim).  Every head's y is divided by its root mean square (`norm_eps`), multiplied by `out_norm`
    [value_dim], one for all heads, and by SiLU(gate(x)), and goes through `o_proj`."""
    kind: ClassVar[str] = "gated_delta"
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    key_dim: int
    value_dim: int
    conv_taps: int
    norm_eps: float
    q_proj: str
    k_proj: str
    v_proj: str
    q_conv: str
    k_conv: str
    v_conv: str
    a_proj: str
    a_log: str
    dt_bias: str
    b_proj: str
    gate_proj: str
    out_norm: str
    o_proj: str


@dataclass(frozen=True)
class SelectiveScanSpec:
    """A selective scan (the Mamba recurrence).  `in_proj` [2 inner, hidden] gives [x | z].  x passes a causal convolution per channel
    (`conv` [inner, conv_taps], the last tap the token's own, bias `conv_bias`, zeros before a sequence's start) and SiLU.  `x_proj`
    [dt_rank + 2 state, inner] of that gives [dt | B | C]; dt <- softplus(`dt_proj` [inner, dt_rank] dt + `dt_bias`), one step size per
    channel; A = -exp(`a_log`) [inner, state].  Per channel c and state n, S zero at a sequence's start:
        S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n        y_c = sum_n S[c, n] C_n + D_c x_c
    and the mixer's result is `o_proj` (y * SiLU(z)).  A request's state is S and the convolution's last conv_taps - 1 inputs."""
    kind: ClassVar[str] = "selective_scan"
    hidden_size: int
    inner: int
    state: int
    dt_rank: int
    conv_taps: int
    in_proj: str
    conv: str
    conv_bias: str
    x_proj: str
    dt_proj: str
    dt_bias: str
    a_log: str
    d_skip: str
    o_proj: str


@dataclass(frozen=True)
class SideBySideSpec:
    """Several mixers that read the same rows; the layer's mixer output is sum_i weights[i] * members[i](h).  Each member keeps the
    cache or state it would keep alone."""
    kind: ClassVar[str] = "side_by_side"
    hidden_size: int
    members: Tuple[Any, ...]
    weights: Tuple[float, ...]

    def __post_init__(self):
        if not self.members or len(self.members) != len(self.weights):
            raise ValueError("mixers side by side: one weight per member, and at least one member")


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """A mixture of gated feed-forwards: `router` [experts, hidden] gives a logit per expert in 32-bit; the scores are their sigmoids
    (`score` = "sigmoid") or a softmax over all experts ("softmax"); the `top` experts with the largest scores serve the row.  The
    chosen scores, divided by their sum if `renormalize`, weigh each chosen expert's input (`weigh` = "input": the sum of
    expert(w h)) or its output ("output": the sum of w expert(h)).  An expert is down(act(gate(a)) * up(a)) without biases (the
    activations of `SwiGluSpec`, `activation_limit` with them).  `shared`, a feed-forward spec of any kind, serves every row and is
    added; with `shared_gate` [1, hidden] it is multiplied by sigmoid(shared_gate . h) first, one number a row.  With `n_groups` > 1 the
    experts form that many equal groups of neighbours, a group scores what its best expert scores, and only experts of the
    `groups_kept` best groups can be chosen.  `renormalize_floor` is added to the sum the chosen scores are divided by."""
    kind: ClassVar[str] = "routed_experts"
    hidden_size: int
    intermediate_size: int
    n_experts: int
    top: int
    router: str
    gate_projs: Tuple[str, ...]
    up_projs: Tuple[str, ...]
    down_projs: Tuple[str, ...]
    score: str = "sigmoid"
    renormalize: bool = False
    weigh: str = "input"
    activation: str = "silu"
    shared: Optional[Any] = None
    activation_limit: float = 0.0
    shared_gate: Optional[str] = None
    n_groups: int = 1
    groups_kept: int = 1
    renormalize_floor: float = 0.0

    def __post_init__(self):
        if not (len(self.gate_projs) == len(self.up_projs) == len(self.down_projs) == self.n_experts) or not 1 <= self.top <= self.n_experts:
            raise ValueError("routed experts: three matrices per expert, and 1 <= top <= experts")
        if (self.n_groups < 1 or self.n_experts % self.n_groups or not 1 <= self.groups_kept <= self.n_groups
                or self.top > self.groups_kept * (self.n_experts // self.n_groups)):
            raise ValueError("routed experts: equal groups, of which 1 .. all are kept, with at least `top` experts in the kept ones")
        if self.shared_gate is not None and self.shared is None:
            raise ValueError("routed experts: a gate on the shared feed-forward needs a shared feed-forward")


@dataclass(frozen=True)
class TokenSideInputSpec:
    """A second input from the token itself, added to the residual stream x behind a layer: with e the columns
    [first_column, first_column + dim) of the token's row of `table` [vocab, table_width],
        g = act(`gate_proj` x) * e;   y = `out_proj` g;   x <- x + norm(y)
    gate_proj [dim, hidden], out_proj [hidden, dim], `norm` a norm spec over hidden."""
    kind: ClassVar[str] = "token_side_input"
    hidden_size: int
    vocab_size: int
    dim: int
    table: str
    table_width: int
    first_column: int
    gate_proj: str
    out_proj: str
    norm: Any
    activation: str = "gelu_tanh"


@dataclass(frozen=True)
class RejoinSpec:
    """The residual stream mixed with the token rows again: x <- `weight` [x; x0] + row `row` of `offsets`, with x0 the rows of the
    token table as the first layer got them, weight [hidden, 2 hidden] (x's columns first), offsets [rows, hidden] (None: nothing
    added)."""
    kind: ClassVar[str] = "rejoin"
    hidden_size: int
    weight: str
    offsets: Optional[str] = None
    offsets_rows: int = 0
    row: int = 0


@dataclass(frozen=True)
class MlstmSpec:
    """A matrix memory per head (the mLSTM of xLSTM) with exponential gating kept stable by a running maximum:
        m_t = max(f_t + m_(t-1), i_t)
        S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t the same with k_t alone
        o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
    with q scaled by key_dim^(-1/2), i = cap * tanh(pre_i / cap), f = logsigmoid(cap * tanh(pre_f / cap)), S, n, m zero at a
    sequence's start.  Every head's o is divided by its root mean square; the heads side by side are multiplied by `out_norm`
    and by sigmoid(gate(x)) and go through `o_proj`."""
    kind: ClassVar[str] = "mlstm"
    hidden_size: int
    n_heads: int
    key_dim: int
    value_dim: int
    gate_cap: float
    norm_eps: float
    q_proj: str
    k_proj: str
    v_proj: str
    gate_proj: str
    o_proj: str
    out_norm: str
    i_proj: str
    i_bias: str
    f_proj: str
    f_bias: str


@dataclass(frozen=True)
class ScaleSpec:
    """Rows multiplied by a constant (for instance a token table that is stored unscaled)."""
    kind: ClassVar[str] = "scale"
    factor: float


@dataclass(frozen=True)
class SoftCapSpec:
    """x <- cap * tanh(x / cap): values kept within (-cap, cap)."""
    kind: ClassVar[str] = "softcap"
    cap: float


@dataclass(frozen=True)
class StreamAccessSpec:
    """How one half of a layer uses the n copies x_0 .. x_(n-1) of the residual stream: it reads u = sum_s read[s] x_s, and with its
    result y every copy becomes x_t <- sum_s mix[s, t] x_s + c * write[t] * y, all copies at once from the old ones (c the layer's
    `residual_scale`).  Tensors `read` [n], `write` [n], `mix` [n, n], the matrix indexed [from, to]."""
    kind: ClassVar[str] = "stream_access"
    n_streams: int
    read: str
    write: str
    mix: str


@dataclass(frozen=True)
class LayerSpec:
    """One layer: which parts, and in which arrangement (`block`) they are wired."""
    mixer: Any
    feed_forward: Any                # None: the layer has no feed-forward half (blocks that allow it)
    mixer_norm: Any
    feed_forward_norm: Any
    block: str = "prenorm"
    mixer_post_norm: Any = None      # "sandwich" blocks: a norm on what each half puts out, before it joins the residual stream
    feed_forward_post_norm: Any = None
    after: Tuple[Any, ...] = ()      # specs of parts that change the residual stream in place behind the block, in order (stream parts)
    # "multistream" blocks (models that carry several copies of the residual stream): how each half reads and writes the copies,
    # and what a half's result is multiplied by on its way into the stream
    mixer_streams: Any = None
    feed_forward_streams: Any = None
    residual_scale: float = 1.0


@dataclass(frozen=True)
class RunEntry:
    """One position of the run order.  `layer` indexes `ModelSpec.layers` (a layer may be named by
    several entries).  `cache_of` is None when the entry keeps a cache of its own, or the index of
    an earlier entry whose cache it reads without writing.  Entries that name one layer share its weights and keep a cache
    each."""
    layer: int
    cache_of: Optional[int] = None
    before: Optional[Any] = None     # spec of a part that changes the residual stream in place before this entry's layer runs (a stream part)


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: str                       # tensor name of the token table [vocab, hidden]
    final_norm: Any
    lm_head: str                         # tensor name; the embedding's name when tied
    layers: Tuple[LayerSpec, ...]
    run_order: Tuple[RunEntry, ...]
    ignorable_tensors: Tuple[str, ...] = field(default=())   # regular expressions of names a file may hold unused
    after_embedding: Tuple[Any, ...] = field(default=())     # row-transform specs applied, in order, to the rows of the token table
    after_head: Tuple[Any, ...] = field(default=())          # ... and to the logits
    # Copies of the residual stream that the layers carry side by side (rows [n_streams * hidden]): all equal to the token rows at the
    # start, added up before the final norm.  More than one needs blocks that know of them (`stream_aware`).
    n_streams: int = 1

    def __post_init__(self):
        for i, e in enumerate(self.run_order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run order entry {i} names layer {e.layer}, but there are {len(self.layers)} layers")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"run order entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if self.run_order[e.cache_of].cache_of is not None:
                    raise ValueError(f"run order entry {i} reads the cache of entry {e.cache_of}, which has none of its own")
