"""Descriptions of a model as data: which parts each layer is made of, with
every size and constant as a field, and the order in which layers run.

A spec is a frozen dataclass with a class attribute ``kind``; the part class
registered under that kind (``shrike_amd.parts.registry``) is built from it.
An architecture turns its config.json into a :class:`ModelSpec`; nothing below
this level knows which architecture it came from.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import ClassVar

# Every part finds its tensors under its own name plus a sub-name per role ("weight",
# "q_proj.weight", ...).  A spec's `names` replaces those sub-names for architectures whose
# files spell them otherwise: pairs (role, sub-name); an empty sub-name stands for the
# part's own name.
Names = tuple


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * (offset + weight): offset 0 for a weight that is
    stored as it is applied, 1 for one that is stored around zero."""

    kind: ClassVar[str] = "rmsnorm"
    eps: float
    offset: float = 0.0
    names: Names = ()


@dataclass(frozen=True)
class LayerNormSpec:
    """y = (x - mean(x)) / sqrt(var(x) + eps) * weight + bias, var the mean of the squared
    deviations; ``bias`` False: no bias tensor."""

    kind: ClassVar[str] = "layernorm"
    eps: float
    bias: bool = True
    names: Names = ()


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of element pairs (i, i + rotary_dim/2) by position * theta**(-2i/rotary_dim)."""

    kind: ClassVar[str] = "rotary_half"
    theta: float
    rotary_dim: int


@dataclass(frozen=True)
class RotaryAdjacentSpec:
    """Rotation of neighbouring elements (2i, 2i + 1), i < rotary_dim / 2, by
    position * theta**(-2i/rotary_dim); elements from rotary_dim on stay as they are."""

    kind: ClassVar[str] = "rotary_adjacent"
    theta: float
    rotary_dim: int


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a paged key/value cache.

    ``window``: a query at position p reads keys j with p - window < j <= p;
    None reads every key.  ``chunk``: a query reads only the keys j <= p of its own
    block of `chunk` positions, floor(j / chunk) == floor(p / chunk), blocks counted
    from position 0 of the sequence; None sets no such bound.  ``position`` is
    applied to queries and keys after the projections; None leaves them as they
    are.  ``values_from_keys``: there is no value projection; a token's values are
    its keys as projected, before ``position`` is applied.
    ``value_dim``: size of a head's value where it differs from ``head_dim`` (the
    size of queries and keys).  ``softcap``: scaled scores become cap * tanh(score /
    cap).  ``sinks``: a learned number per query head whose exponential joins the
    softmax's denominator; it has no key and no value.  ``query_temperature`` =
    (coef, every): the queries at position p are multiplied by 1 + coef *
    ln(floor((p + 1) / every) + 1).  ``value_norm_eps``: each head's value is divided
    by sqrt(mean(v^2) + eps), without a weight, before it is cached.
    ``distance_bias``: two learned numbers per query head (r1, r2); r1 * ln(1 + r2 * (i - j))
    is taken off the scaled score of query i and key j.  ``fixed_sink``: a sink of this fixed
    score (no tensor) in every head's denominator.  ``talking_heads``: a learned [heads, heads]
    matrix T mixes the softmax weights across heads, w_h = sum_g T[h, g] p_g, before head h
    applies them to the values of its own key/value head (the sink's share is not mixed).
    ``qk_norm`` = (eps, weighted): every head of the queries and of the keys is divided by
    sqrt(mean(x^2) + eps) after the projection (queries before their temperature); with
    `weighted` also multiplied by a learned weight of the head's size that all heads share (one
    for the queries, one for the keys).  ``bucket_bias`` = (rows, reach): a learned table [rows,
    heads] whose row bucket(i - j) is added to the (capped) score of head h; the first rows // 2
    rows stand for one distance each, the others are spread evenly over ln(distance) up to
    `reach`, and the last row serves every distance beyond (parts/attention.py:
    distance_buckets); rows None: as many as the file's tensor has.  ``shared_kv``: the layer has no key and value projections (and none of
    their norms' weights); it reads the cache of another run (ScheduleEntry.cache_of) with its
    own queries and mask.  ``cache_window``: what the layer's cache keeps where that is not its
    own window, because a run that reads this cache looks further back ("own": the window;
    None: everything).
    """

    kind: ClassVar[str] = "paged_attention"
    num_heads: int
    num_kv_heads: int
    head_dim: int
    qkv_bias: bool
    out_bias: bool
    scale: float
    window: int | None = None
    position: object = None
    chunk: int | None = None
    values_from_keys: bool = False
    names: Names = ()
    value_dim: int | None = None
    softcap: float | None = None
    sinks: bool = False
    query_temperature: tuple | None = None
    value_norm_eps: float | None = None
    distance_bias: bool = False
    fixed_sink: float | None = None
    talking_heads: bool = False
    qk_norm: tuple | None = None
    bucket_bias: tuple | None = None
    shared_kv: bool = False
    cache_window: object = "own"


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose queries, keys and values come through low-rank latents.

    c_q = norm(W_dq x) (q_rank), q = W_uq c_q: per head ``head_dim`` unrotated and
    ``rot_dim`` rotated elements.  W_dkv x has kv_rank + rot_dim rows: the first
    kv_rank, normed, are the key/value latent c; the rest, not normed, are one rotated
    key part that all heads share.  Per head the unrotated key is W_uk c and the value
    W_uv c (``value_dim``); score = (q_plain . k_plain + q_rot . k_rot) * scale.  The
    rotation turns neighbouring pairs (2i, 2i + 1) of the rotated part by position *
    rot_theta ** (-2i / rotated), for the first ``rotated`` elements of the part (None: all
    of it; the rest pass unchanged).  Both norms are RMS norms with a weight and ``eps``.
    ``window`` / ``chunk`` bound the keys as in AttentionSpec.  Only c and the rotated key
    part are cached.  ``output_gate``: the heads' outputs side by side are multiplied by
    sigmoid(W_g x) before the output matrix."""

    kind: ClassVar[str] = "latent_attention"
    num_heads: int
    head_dim: int
    rot_dim: int
    value_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    eps: float
    rot_theta: float = 10000.0
    window: int | None = None
    chunk: int | None = None
    names: Names = ()
    rotated: int | None = None
    output_gate: bool = False


@dataclass(frozen=True)
class MLSTMSpec:
    """A matrix memory with exponential gates (the mLSTM of xLSTM).  Per head: q = W_q x *
    head_dim ** -0.5, k = W_k x, v = W_v x (``value_dim``); log gates i = cap tanh((W_i x
    + b_i) / cap), f = logsigmoid(cap tanh((W_f x + b_f) / cap)); state S [head_dim,
    value_dim], n [head_dim], running maximum m (all zero before the first token):
        m' = max(f + m, i);  S' = exp(f + m - m') S + exp(i - m') k v^T;  n' likewise with k;
        o = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6).
    Each head's o is divided by its root mean square (``eps``), the heads side by side are
    multiplied by a weight and by sigmoid(W_g x), then W_o."""

    kind: ClassVar[str] = "mlstm"
    num_heads: int
    head_dim: int
    value_dim: int
    gate_cap: float
    eps: float
    names: Names = ()


@dataclass(frozen=True)
class SelectiveScanSpec:
    """The selective scan of Mamba.  W_in x is [u: inner | z: inner]; u passes a causal
    convolution per channel (``conv`` taps, the last meets the current token, with a bias) and
    SiLU; W_x u is [dt: dt_rank | B: state | C: state]; dt <- softplus(W_dt dt + b) per channel;
    A = -exp(A_log) [inner, state];  S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c u_c B_n;
    y_c = sum_n S[c, n] C_n + D_c u_c;  out = W_o (y * silu(z)).  Per request: S (float32) and
    the convolution's last conv - 1 inputs."""

    kind: ClassVar[str] = "selective_scan"
    inner: int
    state: int
    dt_rank: int
    conv: int
    names: Names = ()


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with a fixed decay per head, no softmax and no denominator.  q = W_q x,
    k = W_k x ([heads, head_dim]), v = W_v x ([heads, value_dim]); ``position`` (a rotation
    spec or None) is applied to q and k; k is multiplied by head_dim ** -0.5;
    S_t = decay[h] S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  Each head's o is divided by its root
    mean square (``eps``, no weight), the heads side by side are multiplied by silu(W_g x),
    then W_o.  Per request: S (float32)."""

    kind: ClassVar[str] = "retention"
    num_heads: int
    head_dim: int
    value_dim: int
    decay: tuple
    eps: float
    position: object = None
    names: Names = ()


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Several mixers side by side on the same input: ``branches`` = ((sub-name, mixer spec),
    ...).  Each output is brought to unit root mean square over the model width (``eps``) and
    multiplied by its own weight (tensor "<sub-name>.out" of the mixer, as it is stored); the
    result is ``scale`` times their sum."""

    kind: ClassVar[str] = "parallel_mixers"
    branches: tuple
    eps: float
    scale: float = 0.5
    out_name: str = "out"


@dataclass(frozen=True)
class MoESpec:
    """A routed mixture of gated experts ("e0", "e1", ...), each down(act(gate x) * up x) of
    ``expert_size`` features.  Router logits W_router x in float32; scores = softmax over all
    experts; the ``top`` experts with the largest score + correction (a tensor of one number
    per expert, with ``correction``) are chosen; their weights are their scores over the
    chosen ones' sum (+ 1e-20), which is the softmax over the chosen experts' logits alone.
    ``shared_size``: an expert of that many features that every token passes and whose output is
    added (None: none).  ``gated`` False: experts (the shared one too) are down(act(up x)) and
    have no gate matrix; their activation is then "relu_squared".  ``router_bias``: a learned
    number per expert is added to the logits (a tensor).  ``shared_gate``: the shared expert's
    output is multiplied by sigmoid(w . x), one number per token (a tensor [1, width])."""

    kind: ClassVar[str] = "moe"
    experts: int
    top: int
    expert_size: int
    shared_size: int | None = None
    correction: bool = True
    activation: str = "silu"
    names: Names = ()
    gated: bool = True
    router_bias: bool = False
    shared_gate: bool = False


@dataclass(frozen=True)
class DenseFFNSpec:
    """down(act(up(x))) without biases.  ``activation`` "xielu": for z > 0, softplus(p) z^2
    + z / 2; else (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2, with the layer's own two
    numbers (p, q) in a tensor of two elements."""

    kind: ClassVar[str] = "dense_act"
    intermediate_size: int
    activation: str = "xielu"
    names: Names = ()


@dataclass(frozen=True)
class SwiGLUSpec:
    """down(act(gate(x)) * up(x)) without biases; act is "silu" (SwiGLU proper),
    "gelu_tanh" (the tanh form of GELU) or "quick_gelu" (g * sigmoid(1.702 g)).  With
    ``limit`` the gate is bounded from above, g <- min(g, limit), and the other factor from
    both sides, u <- clamp(u, -limit, limit), before the activation; ``up_shift`` is added to
    that factor: down(act(g) * (u + up_shift))."""

    kind: ClassVar[str] = "swiglu"
    intermediate_size: int
    activation: str = "silu"
    names: Names = ()
    limit: float | None = None
    up_shift: float = 0.0


@dataclass(frozen=True)
class TokenSideSpec:
    """A second input per token and layer, gated by the stream:
    y = proj(act(gate(x)) * table[token, index*dim : (index+1)*dim]);
    x += y * rsqrt(mean(y^2) + eps) * weight.  ``table_name`` is the full name of the
    table [vocab, slices * dim], which all layers share."""

    kind: ClassVar[str] = "token_side"
    vocab_size: int
    dim: int
    index: int
    slices: int
    eps: float
    activation: str = "gelu_tanh"
    table_name: str = "side.embed"
    names: Names = ()


@dataclass(frozen=True)
class BlockSpec:
    """x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x)).  ``ffn`` may be None: the
    layer then has no feed-forward and no second norm.

    ``name`` is the prefix of the block's tensors in the weight file; the
    ``*_name`` fields are the sub-names of its parts below that prefix.
    """

    kind: ClassVar[str] = "prenorm_residual"
    name: str
    mixer: object
    ffn: object
    mixer_norm: object
    ffn_norm: object
    mixer_name: str = "self_attn"
    ffn_name: str = "mlp"
    mixer_norm_name: str = "input_layernorm"
    ffn_norm_name: str = "post_attention_layernorm"


@dataclass(frozen=True)
class SandwichBlockSpec:
    """A norm before and after each sublayer: x += mixer_post(mixer(mixer_norm(x)));
    x += ffn_post(ffn(ffn_norm(x))).  ``ffn`` may be None: the layer then has no feed-forward
    and neither of its norms."""

    kind: ClassVar[str] = "sandwich_residual"
    name: str
    mixer: object
    ffn: object
    mixer_norm: object
    mixer_post: object
    ffn_norm: object = None
    ffn_post: object = None
    mixer_name: str = "mix"
    ffn_name: str = "mlp"
    mixer_norm_name: str = "norm1"
    mixer_post_name: str = "norm1b"
    ffn_norm_name: str = "norm2"
    ffn_post_name: str = "norm2b"


@dataclass(frozen=True)
class PostNormBlockSpec:
    """The norm stands after the sum, and the stream is what the norm leaves:
    x <- mixer_norm(alpha * x + s1 * mixer(x)); x <- ffn_norm(alpha * x + s2 * ffn(x)), the
    sublayers reading x itself.  ``layer_scale``: s1 and s2 are learned vectors of the model's
    width (tensors ``mixer_scale_name`` / ``ffn_scale_name`` below the block's name); else ones.
    ``ffn`` may be None: the layer then has no feed-forward and no second scale; it has a second
    norm only if ``ffn_norm`` is given and the weight file holds its tensor, and the stream then
    passes it with nothing added, x <- ffn_norm(alpha * x)."""

    kind: ClassVar[str] = "postnorm_residual"
    name: str
    mixer: object
    ffn: object
    mixer_norm: object
    ffn_norm: object = None
    alpha: float = 1.0
    layer_scale: bool = False
    mixer_name: str = "mix"
    ffn_name: str = "mlp"
    mixer_norm_name: str = "norm1"
    ffn_norm_name: str = "norm2"
    mixer_scale_name: str = "ls1"
    ffn_scale_name: str = "ls2"


@dataclass(frozen=True)
class ParallelBlockSpec:
    """h = norm(x); x += mixer(h) + ffn(h); then x = side(x, tokens) where there is one.
    One norm feeds both sublayers; ``ffn`` and ``side`` may be None."""

    kind: ClassVar[str] = "parallel_residual"
    name: str
    norm: object
    mixer: object
    ffn: object = None
    side: object = None
    norm_name: str = "norm1"
    mixer_name: str = "mix"
    ffn_name: str = "mlp"
    side_name: str = "side"


@dataclass(frozen=True)
class TokenEmbeddingSpec:
    """x = table[token id] * scale; with ``norm`` (a norm spec, its tensors under
    ``norm_name``), x = norm(x) after that."""

    kind: ClassVar[str] = "token_lookup"
    vocab_size: int
    scale: float = 1.0
    names: Names = ()
    norm: object = None
    norm_name: str = "embed.norm"


@dataclass(frozen=True)
class PairHashEmbeddingSpec:
    """x = table[token] + pairs[(previous token * mul_prev + token * mul_cur) mod buckets];
    a sequence's first token, which has no previous one, takes row `buckets` (the last of
    the buckets + 1 rows).  ``pair_name`` is the full name of the pair table."""

    kind: ClassVar[str] = "token_pair_hash"
    vocab_size: int
    buckets: int
    mul_prev: int
    mul_cur: int
    pair_name: str = "bigram"
    names: Names = ()


@dataclass(frozen=True)
class LinearHeadSpec:
    """logits = (x @ W.T) * scale, no bias; with ``softcap``, logits <- softcap * tanh(logits /
    softcap) after that."""

    kind: ClassVar[str] = "linear"
    vocab_size: int
    names: Names = ()
    scale: float = 1.0
    softcap: float | None = None


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a block.  ``cache_of`` names an earlier schedule position whose
    cache this run reads instead of owning one; None means it owns its cache.
    Before the run, ``add_embedding`` adds the embedding's output (the stream as it
    was before the first block) to the stream, and ``add_vector`` = (tensor, row)
    adds row `row` of a tensor that the model declares in ``stream_vectors``.
    ``depth_average`` names a tensor of (position + 2) numbers c: with X_0 the embedding's
    output and X_(k+1) what run k leaves, the stream that goes on after this run (position i)
    is sum_j c[j] X_j, j = 0 .. i + 1; X_(i+1) itself is the run's result before that sum.
    Either every entry of a schedule has one or none has."""

    block: int
    cache_of: int | None = None
    add_embedding: bool = False
    add_vector: tuple | None = None
    depth_average: str | None = None


@dataclass(frozen=True)
class ModelSpec:
    """Token ids -> embedding -> schedule of blocks -> final norm -> head.

    ``embedding`` and ``head`` are part specs like the others; left as None they
    are the plain table lookup and the plain output matrix over ``vocab_size``.
    """

    architecture: str
    hidden_size: int
    vocab_size: int
    blocks: tuple[BlockSpec, ...]
    final_norm: object
    tie_word_embeddings: bool
    schedule: tuple[ScheduleEntry, ...] = ()
    embed_name: str = "model.embed_tokens"
    final_norm_name: str = "model.norm"
    head_name: str = "lm_head"
    eos_token_ids: tuple[int, ...] = ()
    max_position_embeddings: int | None = None
    stored_dtype: str = "bfloat16"
    extra: dict = field(default_factory=dict, compare=False)
    embedding: object = None
    head: object = None
    # (tensor name, rows): float32 tensors [rows, hidden_size] whose rows schedule
    # entries add to the stream (ScheduleEntry.add_vector)
    stream_vectors: tuple = ()

    def __post_init__(self):
        if self.embedding is None:
            object.__setattr__(self, "embedding", TokenEmbeddingSpec(self.vocab_size))
        if self.head is None:
            object.__setattr__(self, "head", LinearHeadSpec(self.vocab_size))
        if not self.schedule:
            object.__setattr__(
                self, "schedule", tuple(ScheduleEntry(i) for i in range(len(self.blocks)))
            )
        averaged = [e.depth_average is not None for e in self.schedule]
        if any(averaged) and not all(averaged):
            raise ValueError("a depth average needs every run's result: every schedule entry must name one")
        for pos, entry in enumerate(self.schedule):
            if not 0 <= entry.block < len(self.blocks):
                raise ValueError(f"schedule[{pos}] names block {entry.block}, which does not exist")
            if entry.add_vector is not None:
                rows = dict(self.stream_vectors).get(entry.add_vector[0])
                if rows is None or not 0 <= entry.add_vector[1] < rows:
                    raise ValueError(f"schedule[{pos}] adds {entry.add_vector}, which stream_vectors does not hold")
            if entry.cache_of is not None:
                if not 0 <= entry.cache_of < pos:
                    raise ValueError(
                        f"schedule[{pos}] reads the cache of position {entry.cache_of}, "
                        "which is not an earlier position"
                    )
                if self.schedule[entry.cache_of].cache_of is not None:
                    raise ValueError(
                        f"schedule[{pos}] reads the cache of position {entry.cache_of}, "
                        "which does not own one"
                    )
