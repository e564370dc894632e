"""Architecture-independent description of a decoder: what the engine builds from.

An architecture's own configuration (for example `Qwen3Config`) is translated
into a `ModelSpec`: a tuple of `LayerSpec`s, each naming its block arrangement,
norm, mixer and feed-forward with every size and constant as a field, plus a
`schedule` that says in which order layers run and which cache each run uses.
Parts are selected by the `kind` strings through `parts.registry`; nothing in
this file knows a model family.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


@dataclass(frozen=True)
class NormSpec:
    """kind "rmsnorm": x / sqrt(mean(x^2) + eps) * w; kind "layernorm":
    (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b, with a weight and a bias."""
    kind: str = "rmsnorm"
    eps: float = 1e-6


@dataclass(frozen=True)
class FrequencyScaling:
    """Long wavelengths of a rotation are stretched: with l = 2 pi / f, a frequency stays where
    l < original / high, becomes f / factor where l > original / low, and in between the blend
    (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class PositionSpec:
    """Position encoding of a mixer.  kind "rope": rotate-half pairs (i, i+dim/2)
    with angle = position / theta^(2i/dim), from a table of `max_positions` rows; kind
    "rope_pairs": neighbouring pairs (2i, 2i+1) with the same angles, worked out by the kernels
    from the frequencies theta^(-2i/dim), so no position is too far; kind "rope_half": the pairs
    of "rope" with the angles worked out by the kernels as for "rope_pairs", the frequencies
    optionally rescaled (`scaling`); kind "none": no encoding."""
    kind: str = "rope"
    theta: float = 10000.0
    dim: int = 0
    max_positions: int = 0
    scaling: Optional[FrequencyScaling] = None      # kind "rope_half" only


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a key/value cache."""
    kind: str = "attention"
    n_heads: int = 0
    n_kv_heads: int = 0
    head_dim: int = 0
    qk_norm: bool = False          # per-head RMSNorm of q and k before the rotation
    qk_norm_eps: float = 1e-6
    window: Optional[int] = None   # None: every earlier key; w: the last w keys
    scale: Optional[float] = None  # None: 1/sqrt(head_dim)
    position: PositionSpec = field(default_factory=PositionSpec)
    value_dim: Optional[int] = None     # None: values as wide as keys
    # biases of the q, k and v projections: None: taken when the checkpoint holds them,
    # True: the checkpoint must hold them, False: it must not
    qkv_bias: Optional[bool] = None
    # "head": RMSNorm of every head with one weight [head_dim]; "projection": one RMSNorm
    # over all heads of q (and of k) together, weights [heads * head_dim]
    qk_norm_scope: str = "head"
    # positions i >= j see each other only if i // chunk == j // chunk, counted from the
    # sequence's position 0 (None: no such blocks)
    chunk: Optional[int] = None
    # r: the score of query i and key j is lowered by 2^(-r (h + 1) / heads) * (i - j) for
    # head h (None: no distance term)
    distance_slope_range: Optional[float] = None
    # a learned number per head that joins the softmax's denominator as exp(sink), with no
    # key and no value
    sink: bool = False
    # the softmax's denominator holds a 1 besides the keys' terms (a sink of score 0 that is
    # not learned); not together with `sink`
    unit_sink: bool = False
    # a learned matrix T [heads, heads] mixes the scaled scores of a (query, key) pair over the
    # heads before the softmax: score_h <- sum_g T[h, g] score_g
    talking_heads: bool = False
    # the output projection's bias: None: taken when the checkpoint holds it, True: it must
    # hold it, False: it must not
    o_bias: Optional[bool] = None
    # values shared across layers of a step: "source": this layer's values (before anything is
    # mixed into them) are kept for the step's later layers; "mix": what this layer caches and
    # attends to is (1 - lambda) v + lambda v_source, v_source the source layer's values of the
    # same token and lambda a learned number; "off": the layer's values are its own, but its
    # checkpoint may hold the (unused) number; None: no such thing
    value_mix: Optional[str] = None
    # the concatenated heads are multiplied, element by element, by sigmoid(W_g x), x the
    # mixer's input, before the output projection; "head": W_g has one row a head, and every
    # element of a head's output is multiplied by that head's sigmoid
    output_gate: object = False
    # P: besides the tokens of its window a query at position i sees one key and value for
    # every block b of P positions that lies wholly before the window (b P + P - 1 <= i -
    # window): the means of the block's cached keys and of its values; tokens and blocks share
    # one softmax.  Needs a window.
    pool: Optional[int] = None
    # (coef, every): the query at position p is multiplied by
    # 1 + coef ln(floor((p + 1) / every) + 1)
    query_temperature: Optional[Tuple[float, int]] = None
    # the part has no key and value projections: every run of it reads keys and values that
    # another run has cached (its schedule entries never write the cache)
    shared_kv: bool = False
    # positions behind the newest one that the cache keeps for other runs that read it with a
    # wider mask than this layer's own: None: what the own window and pool need; 0: all
    cache_span: Optional[int] = None

    @property
    def q_width(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_width(self) -> int:
        return self.n_kv_heads * self.head_dim

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def v_width(self) -> int:
        return self.n_kv_heads * self.v_dim

    @property
    def out_width(self) -> int:
        return self.n_heads * self.v_dim


@dataclass(frozen=True)
class GatedMLPSpec:
    """down(act(gate(x)) * up(x))."""
    kind: str = "gated_mlp"
    intermediate_size: int = 0
    # of the gate: "silu" or "gelu_tanh"; or "clamped_swish": with g = min(gate x, limit) and
    # u = clamp(up x, -limit, limit) the product is g sigmoid(alpha g) (u + 1)
    activation: str = "silu"
    # biases of the three projections: None: taken when the checkpoint holds them, True: it
    # must hold them, False: it must not
    bias: Optional[bool] = None
    limit: float = 0.0            # "clamped_swish" only
    alpha: float = 1.0            # "clamped_swish" only


@dataclass(frozen=True)
class RoutedMLPSpec:
    """Mixture of experts: a router chooses `top` of `n_experts` gated feed-forwards
    down(silu(gate x) * up x) for every token, by the largest float32 logits W_router x, and
    adds their outputs weighted by the softmax over the chosen logits alone.

    `scoring` "softmax_all": the scores are the softmax over all router outputs, the choice is
    by the largest score (plus a learned per-output `correction` where the spec says so), and
    the weights are the chosen scores themselves, not renormalised.  `identity`: the router
    has that many outputs beyond `n_experts`; one of them chosen adds the input row itself,
    times its weight (such experts have no matrices)."""
    kind: str = "routed_mlp"
    n_experts: int = 0
    top: int = 0
    intermediate_size: int = 0    # of one expert
    scoring: str = "softmax_chosen"
    correction: bool = False
    identity: int = 0

    @property
    def router_outputs(self) -> int:
        return self.n_experts + self.identity


@dataclass(frozen=True)
class StateSpaceSpec:
    """Selective state-space mixer with one decay per head (Mamba-2): a recurrent mixer whose
    state is one [state, head_dim] matrix per head, fed through a short causal convolution.
    See `parts.ssm`."""
    kind: str = "mamba2"
    n_heads: int = 0
    head_dim: int = 0             # columns of a head's state (its share of the inner width)
    state: int = 0                # rows of a head's state: the size of B and C
    groups: int = 1               # pairs of B and C, each shared by n_heads / groups heads
    conv_taps: int = 4
    norm_parts: int = 1           # the gated read-out is RMS-normed in this many equal parts
    norm_eps: float = 1e-6

    @property
    def inner(self) -> int:
        return self.n_heads * self.head_dim


@dataclass(frozen=True)
class LinearAttentionSpec:
    """Linear attention with a fixed decay per head: q = silu(W_q x), k = silu(W_k x) (heads x
    key_dim), v = silu(W_v x) (heads x value_dim); per head S_t = decay_h S_(t-1) + k_t v_t^T
    and o_t = S_t^T q_t; the concatenated heads pass an RMS norm with a weight, are multiplied
    by sigmoid(W_g x), and projected.  See `parts.linear_attention`."""
    kind: str = "linear_attention"
    n_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    decay: Tuple[float, ...] = ()     # one per head
    norm_eps: float = 1e-6

    @property
    def qk_width(self) -> int:
        return self.n_heads * self.key_dim

    @property
    def v_width(self) -> int:
        return self.n_heads * self.value_dim


@dataclass(frozen=True)
class ParallelSpec:
    """Several mixers side by side that read the same rows: the result is the mean of their
    outputs, each first RMS-normed over the model's width with a weight of its own.  See
    `parts.parallel`."""
    kind: str = "parallel"
    branches: Tuple[object, ...] = ()     # mixer specs
    names: Tuple[str, ...] = ()           # parameter prefix of every branch
    norm_eps: float = 1e-6


@dataclass(frozen=True)
class DenseMLPSpec:
    """down(act(up(x))); activation "relu2" (the square of relu), "relu", "silu" or
    "gelu_tanh"."""
    kind: str = "dense_mlp"
    intermediate_size: int = 0
    activation: str = "relu2"


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Causal attention whose keys and values are up-projections of one latent vector a
    position, which is all the cache holds besides one rotated key part that every head
    shares.  Queries pass a normed latent of their own.  A head's query and key are
    [head_dim unrotated | rot_dim rotated].  See `parts.latent`."""
    kind: str = "latent_attention"
    n_heads: int = 0
    head_dim: int = 0             # unrotated query/key elements of a head
    rot_dim: int = 0              # rotated elements of a head; the key's are shared by all heads
    value_dim: int = 0
    kv_rank: int = 0              # width of the cached latent
    q_rank: int = 0               # width of the queries' latent
    scale: Optional[float] = None         # None: 1/sqrt(head_dim + rot_dim)
    norm_eps: float = 1e-6                # eps of the RMS norms of the two latents
    position: PositionSpec = field(default_factory=lambda: PositionSpec(kind="rope_pairs"))
    sink: bool = False            # a learned number per head in the softmax's denominator
    output_gate: bool = False     # a head's output is multiplied by sigmoid(w_h . x), x the input

    @property
    def q_width(self) -> int:
        return self.n_heads * (self.head_dim + self.rot_dim)

    @property
    def cache_width(self) -> int:
        return self.kv_rank + self.rot_dim

    @property
    def out_width(self) -> int:
        return self.n_heads * self.value_dim


@dataclass(frozen=True)
class MatrixMemorySpec:
    """Matrix memory with exponential gates (mLSTM): a recurrent mixer whose state is one
    [key_dim, value_dim] matrix, a normaliser [key_dim] and a running maximum per head.  See
    `parts.mlstm`."""
    kind: str = "mlstm"
    n_heads: int = 0
    key_dim: int = 0
    value_dim: int = 0
    gate_cap: float = 15.0        # the gates' pre-activations pass cap * tanh(x / cap)
    out_norm_eps: float = 1e-6    # eps of the RMS norm of each head's read-out
    bottom_eps: float = 1e-6      # added to the read-out's denominator

    @property
    def qk_width(self) -> int:
        return self.n_heads * self.key_dim

    @property
    def v_width(self) -> int:
        return self.n_heads * self.value_dim


@dataclass(frozen=True)
class GatedDeltaSpec:
    """Gated delta rule: a recurrent mixer whose state is one [key_dim, value_dim] matrix per
    head, fed through short causal convolutions.  See `parts.delta`."""
    kind: str = "gated_delta"
    n_heads: int = 0              # value heads (one state each)
    n_kv_heads: int = 0           # query/key heads, shared by n_heads / n_kv_heads value heads
    key_dim: int = 0
    value_dim: int = 0
    conv_taps: int = 4            # taps of the causal convolution of q, k and v
    out_norm_eps: float = 1e-6    # eps of the RMS norm of each head's read-out
    unit_eps: float = 1e-6        # q and k become x / sqrt(sum(x^2) + unit_eps) per head

    @property
    def qk_width(self) -> int:
        return self.n_kv_heads * self.key_dim

    @property
    def v_width(self) -> int:
        return self.n_heads * self.value_dim


@dataclass(frozen=True)
class LayerSpec:
    block: str            # arrangement, e.g. "prenorm"
    norm: NormSpec
    mixer: object         # a spec with a .kind (AttentionSpec, or one a test registers)
    feed_forward: object  # a spec with a .kind (GatedMLPSpec, ...), or None: no feed-forward
    # what a sublayer adds to the stream is multiplied by this (arrangements that know it)
    residual_scale: float = 1.0
    # what a sublayer adds is multiplied, element by element, by a learned vector of the
    # model's width, one for the mixer and one for the feed-forward (arrangements that know it)
    layer_scale: bool = False
    # taps T > 0: what a sublayer reads, h, is replaced by h + conv(h), a causal convolution
    # over time on every channel with a learned filter [width, T] per sublayer and no bias:
    # conv(h)_t = sum_j w[:, j] h_(t - T + 1 + j), zeros before the sequence's start; the last
    # T - 1 inputs of both sublayers are state of the sequence (arrangements that know it)
    input_conv: int = 0
    # the model's width, for arrangements that ask for state of that width (None: not needed)
    width: Optional[int] = None


@dataclass(frozen=True)
class LoopSpec:
    """Layers start .. stop - 1 run `times` times in a row with the same weights, each pass
    with cache entries of its own.  Before a pass the stream x is made anew from itself and the
    embedding output x0: x <- W [x ; x0] + step[pass], with W [hidden, 2 hidden] and step
    [times, hidden] parameters of the model."""
    start: int
    stop: int
    times: int


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer.  `cache` is the id of the cache entry the mixer uses;
    `writes_cache` False means it only reads an entry that another run wrote.  `own` is the id
    under which the run keeps what is its own whatever `cache` says (the state of its block,
    what its mixer derives from keys that another run wrote); None: the same as `cache`."""
    layer: int
    cache: int
    writes_cache: bool = True
    own: Optional[int] = None

    @property
    def own_id(self) -> int:
        return self.cache if self.own is None else self.own


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: NormSpec
    tie_word_embeddings: bool
    max_position_embeddings: int
    bos_token_id: Optional[int]   # None: the architecture names no such token
    eos_token_id: Optional[int]
    embedding_scale: float = 1.0         # the embedding rows are multiplied by this
    loop: Optional[LoopSpec] = None      # the schedule then has to be `looped_schedule`'s
    embedding_norm: Optional[NormSpec] = None    # a norm on the embedding rows (None: none)
    logit_scale: float = 1.0             # the head's products are multiplied by this,
    logit_softcap: Optional[float] = None    # and then capped: c tanh(logit / c) (None: no cap)

    def validate(self) -> None:
        if not self.layers or not self.schedule:
            raise ValueError("a model needs at least one layer and one schedule entry")
        writers = {}
        for entry in self.schedule:
            if not 0 <= entry.layer < len(self.layers):
                raise ValueError(f"schedule names layer {entry.layer} of {len(self.layers)}")
            if entry.writes_cache:
                if entry.cache in writers:
                    raise ValueError(f"cache entry {entry.cache} has two writers")
                writers[entry.cache] = entry.layer
        owners = {}
        for run, entry in enumerate(self.schedule):
            if entry.own is None:
                continue
            # what a run keeps under `own` must not be another run's
            if entry.own in owners or (entry.own in writers and entry.own != entry.cache) \
                    or any(other.cache == entry.own or other.own == entry.own
                           for index, other in enumerate(self.schedule) if index != run):
                raise ValueError(f"the id {entry.own} under which run {run} keeps its own "
                                 "state is also another run's")
            owners[entry.own] = run
        if self.loop is not None:
            loop = self.loop
            if not (0 <= loop.start < loop.stop <= len(self.layers)) or loop.times < 1:
                raise ValueError(f"a loop over layers {loop.start}..{loop.stop - 1}, {loop.times} "
                                 f"times, does not fit {len(self.layers)} layers")
            if self.schedule != looped_schedule(len(self.layers), loop):
                raise ValueError("the schedule of a model with a loop must be looped_schedule's")
        seen = set()
        for entry in self.schedule:
            if entry.writes_cache:
                seen.add(entry.cache)
            elif entry.cache not in seen:
                raise ValueError(
                    f"layer {entry.layer} reads cache entry {entry.cache} before it is written")


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    """Every layer once, in order, each with a cache entry of its own."""
    return tuple(ScheduleEntry(layer=i, cache=i) for i in range(n_layers))


def looped_schedule(n_layers: int, loop: LoopSpec) -> Tuple[ScheduleEntry, ...]:
    """The layers before the loop, the looped layers `times` times, the rest; every run has a
    cache entry of its own."""
    order = list(range(loop.start))
    for _ in range(loop.times):
        order += list(range(loop.start, loop.stop))
    order += list(range(loop.stop, n_layers))
    return tuple(ScheduleEntry(layer=layer, cache=run) for run, layer in enumerate(order))


def pass_starts(n_layers: int, loop: LoopSpec):
    """Index in `looped_schedule` of the first run of every pass."""
    return tuple(loop.start + t * (loop.stop - loop.start) for t in range(loop.times))
