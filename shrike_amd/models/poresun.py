"""Poresun: a decoder whose norms stand after the sums (the stream is what a norm leaves, and
each sublayer's output is scaled by a learned vector before it joins), whose mixers are two
kinds of attention without rotation (positions enter through a learned bias by distance) and
an attention through latents with an output gate, and whose feed-forward is a bounded gated
one or a routed mixture of experts without gates.

config.json (every size and every constant that can differ between models):

    architecture   "Poresun"
    vocab, width
    embedding      {scale}
    norm           {eps}                     all norms
    postln_alpha                             x <- norm(alpha * x + ls * sublayer(x))
    layers[i]      {type, mixer: {...}, mlp: {...} | null}

    type "attention"         mixer {heads, kv_heads, dim, vdim, scale, softcap, bias_max, mask: {size}}
        grouped-query attention; queries and keys brought to unit root mean square per head
        (no weight); scaled scores capped, cap * tanh(s / cap); a learned bias by distance added
        after that (table `rel` [rows, heads], the rows spread as parts/attention.py:
        distance_buckets says, up to the distance bias_max; the tensor's shape gives the rows,
        and a config.json written for random weights names them as bias_rows); sliding window.
    type "attention_2"       mixer {heads, kv_heads, dim, vdim, scale, bias_max, q_temp: {coef, every},
                                    kv_from}
        grouped-query attention; queries and keys normed per head with a weight that the heads
        share (`q.norm`, `k.norm`); queries multiplied by 1 + coef * ln(floor((p + 1) / every) + 1);
        the same bias by distance; causal.  With kv_from: j the layer has no keys and values of
        its own and reads layer j's.
    type "latent_attention"  mixer {heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot: {base, dims}}
        queries and keys/values through normed latents, a rotated key part shared by the heads
        (neighbouring pairs), causal, heads' outputs times sigmoid(W_g x).

    mlp {kind: "dense", ff, limit}           g = min(W_gate x, limit), u = clamp(W_up x, +-limit),
                                             W_down (g sigmoid(1.702 g) (u + 1))
    mlp {kind: "moe", expert: {ff}, router: {experts, top}, shared: {ff} | absent}
        experts W_down relu(W_up x)^2; router logits W_router x + b in float32, the `top` largest
        chosen, weights their softmax; the shared expert's output times sigmoid(w_sg . x).

Tensors: embed (also the output matrix), final.norm, and per layer l<i>.norm1, norm2, ls1, ls2,
l<i>.mix.* (by mixer), l<i>.mlp.{gate, up, down} or l<i>.mlp.{e<k>.{up, down}, router, router.b,
shared.{up, down, sg}}.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..config.engine_config import canonical_dtype
from ..config.registry import ConfigError, register_architecture
from ..config.specs import (
    AttentionSpec,
    LatentAttentionSpec,
    LinearHeadSpec,
    MoESpec,
    ModelSpec,
    PostNormBlockSpec,
    RMSNormSpec,
    ScheduleEntry,
    SwiGLUSpec,
    TokenEmbeddingSpec,
)

ARCHITECTURE = "Poresun"
MIXERS = ("attention", "attention_2", "latent_attention")
DENSE_ACTIVATION = "quick_gelu"  # g * sigmoid(1.702 g)
DENSE_UP_SHIFT = 1.0  # the gate multiplies (u + 1)
EXPERT_ACTIVATION = "relu_squared"


def _get(raw, key: str, kind, where: str = "config.json"):
    if not isinstance(raw, dict) or key not in raw or raw[key] is None:
        raise ConfigError(f"{where} lacks the key {key!r}, which {ARCHITECTURE} needs")
    value = raw[key]
    if kind is int:
        if isinstance(value, bool) or not isinstance(value, int):
            raise ConfigError(f"{where}: {key} must be an integer, got {value!r}")
    elif kind is float:
        if isinstance(value, bool) or not isinstance(value, (int, float)):
            raise ConfigError(f"{where}: {key} must be a number, got {value!r}")
        value = float(value)
    elif kind is dict and not isinstance(value, dict):
        raise ConfigError(f"{where}: {key} must be an object, got {value!r}")
    return value


def _positive(where: str, **values) -> None:
    for name, value in values.items():
        if not value > 0:
            raise ConfigError(f"{where}: {name} must be positive, got {value}")


@dataclass(frozen=True)
class BucketAttention:
    """Both kinds of attention without rotation; `weighted_norm` tells them apart."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: int
    weighted_norm: bool
    window: int | None = None
    softcap: float | None = None
    q_temp: tuple | None = None
    kv_from: int | None = None
    bias_rows: int | None = None  # rows of the bias table; None: as many as the file's tensor has

    @classmethod
    def from_dict(cls, raw: dict, where: str, weighted_norm: bool) -> "BucketAttention":
        dim = _get(raw, "dim", int, where)
        mask, qt = raw.get("mask"), raw.get("q_temp")
        out = cls(heads=_get(raw, "heads", int, where), kv_heads=_get(raw, "kv_heads", int, where), dim=dim,
                  vdim=_get(raw, "vdim", int, where) if raw.get("vdim") is not None else dim,
                  scale=_get(raw, "scale", float, where), bias_max=_get(raw, "bias_max", int, where),
                  weighted_norm=weighted_norm,
                  window=None if mask is None else _get(mask, "size", int, where + ".mask"),
                  softcap=None if raw.get("softcap") is None else _get(raw, "softcap", float, where),
                  q_temp=None if qt is None else (_get(qt, "coef", float, where + ".q_temp"),
                                                  _get(qt, "every", int, where + ".q_temp")),
                  kv_from=None if raw.get("kv_from") is None else _get(raw, "kv_from", int, where),
                  bias_rows=None if raw.get("bias_rows") is None else _get(raw, "bias_rows", int, where))
        _positive(where, heads=out.heads, kv_heads=out.kv_heads, dim=out.dim, vdim=out.vdim, bias_max=out.bias_max)
        if out.window is not None:
            _positive(where + ".mask", size=out.window)
        if out.softcap is not None:
            _positive(where, softcap=out.softcap)
        if out.q_temp is not None:
            _positive(where + ".q_temp", every=out.q_temp[1])
        if out.bias_rows is not None:
            _positive(where, bias_rows=out.bias_rows)
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads are not a multiple of {out.kv_heads} kv_heads")
        return out

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
               "bias_max": self.bias_max}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        if self.softcap is not None:
            out["softcap"] = self.softcap
        if self.q_temp is not None:
            out["q_temp"] = {"coef": self.q_temp[0], "every": self.q_temp[1]}
        if self.kv_from is not None:
            out["kv_from"] = self.kv_from
        if self.bias_rows is not None:
            out["bias_rows"] = self.bias_rows
        return out


@dataclass(frozen=True)
class GatedLatentAttention:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "GatedLatentAttention":
        rot_dim = _get(raw, "rot_dim", int, where)
        rot = raw.get("rot") or {}
        out = cls(heads=_get(raw, "heads", int, where), dim=_get(raw, "dim", int, where), rot_dim=rot_dim,
                  vdim=_get(raw, "vdim", int, where), q_rank=_get(raw, "q_rank", int, where),
                  kv_rank=_get(raw, "kv_rank", int, where), scale=_get(raw, "scale", float, where),
                  rot_base=_get(rot, "base", float, where + ".rot") if rot_dim else 1.0,
                  rot_dims=(_get(rot, "dims", int, where + ".rot") if rot.get("dims") is not None else rot_dim))
        _positive(where, heads=out.heads, dim=out.dim, vdim=out.vdim, q_rank=out.q_rank, kv_rank=out.kv_rank,
                  rot_base=out.rot_base)
        if out.rot_dim < 0 or out.rot_dim % 2 or out.rot_dims < 0 or out.rot_dims % 2 or out.rot_dims > out.rot_dim:
            raise ConfigError(f"{where}: rot_dim ({out.rot_dim}) and rot.dims ({out.rot_dims}) must be even, and "
                              "rot.dims at most rot_dim")
        return out

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}


@dataclass(frozen=True)
class BoundedDense:
    ff: int
    limit: float

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "BoundedDense":
        out = cls(ff=_get(raw, "ff", int, where), limit=_get(raw, "limit", float, where))
        _positive(where, ff=out.ff, limit=out.limit)
        return out

    def to_dict(self) -> dict:
        return {"kind": "dense", "ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class UngatedMixture:
    experts: int
    top: int
    ff: int
    shared_ff: int | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "UngatedMixture":
        router = _get(raw, "router", dict, where)
        shared = raw.get("shared")
        out = cls(experts=_get(router, "experts", int, where + ".router"), top=_get(router, "top", int, where + ".router"),
                  ff=_get(_get(raw, "expert", dict, where), "ff", int, where + ".expert"),
                  shared_ff=None if shared is None else _get(shared, "ff", int, where + ".shared"))
        _positive(where, experts=out.experts, top=out.top, ff=out.ff)
        if out.shared_ff is not None:
            _positive(where + ".shared", ff=out.shared_ff)
        if out.top > out.experts:
            raise ConfigError(f"{where}: top {out.top} is more than the {out.experts} experts")
        return out

    def to_dict(self) -> dict:
        out = {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


def _mlp_from_dict(raw, where: str):
    if raw is None:
        return None
    kind = _get(raw, "kind", str, where)
    if kind == "dense":
        return BoundedDense.from_dict(raw, where)
    if kind == "moe":
        return UngatedMixture.from_dict(raw, where)
    raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (known: dense, moe)")


@dataclass(frozen=True)
class PoresunLayer:
    type: str
    mixer: object
    mlp: object

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class PoresunConfig:
    vocab: int
    width: int
    norm_eps: float
    alpha: float
    layers: tuple[PoresunLayer, ...]
    embedding_scale: float = 1.0
    torch_dtype: str = "bfloat16"

    def __post_init__(self):
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be > 0, got {self.norm_eps}")
        for i, layer in enumerate(self.layers):
            source = getattr(layer.mixer, "kv_from", None)
            if source is None:
                continue
            where = f"config.json layers[{i}].mixer"
            if not 0 <= source < i:
                raise ConfigError(f"{where}: kv_from {source} must name an earlier layer")
            other = self.layers[source]
            if other.type not in ("attention", "attention_2") or other.mixer.kv_from is not None:
                raise ConfigError(f"{where}: kv_from {source} names a layer without keys and values of its own")
            a, b = layer.mixer, other.mixer
            if (a.kv_heads, a.dim, a.vdim) != (b.kv_heads, b.dim, b.vdim):
                raise ConfigError(f"{where}: layer {source}'s keys and values have other sizes than this layer's")

    @classmethod
    def from_dict(cls, raw: dict) -> "PoresunConfig":
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: layers must be a non-empty list")
        layers = []
        for i, entry in enumerate(listed):
            where = f"config.json layers[{i}]"
            kind = _get(entry, "type", str, where)
            mixer = _get(entry, "mixer", dict, where)
            if kind == "latent_attention":
                mixer = GatedLatentAttention.from_dict(mixer, where + ".mixer")
            elif kind in ("attention", "attention_2"):
                mixer = BucketAttention.from_dict(mixer, where + ".mixer", weighted_norm=kind == "attention_2")
            else:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXERS)})")
            layers.append(PoresunLayer(kind, mixer, _mlp_from_dict(entry.get("mlp"), where + ".mlp")))
        dtype = raw.get("torch_dtype") or "bfloat16"
        try:
            dtype = canonical_dtype(dtype)
        except ValueError as e:
            raise ConfigError(f"config.json: {e}") from None
        embedding = raw.get("embedding") or {}
        return cls(vocab=_get(raw, "vocab", int), width=_get(raw, "width", int),
                   norm_eps=_get(_get(raw, "norm", dict), "eps", float, "config.json norm"),
                   alpha=_get(raw, "postln_alpha", float) if raw.get("postln_alpha") is not None else 1.0,
                   layers=tuple(layers),
                   embedding_scale=_get(embedding, "scale", float, "config.json embedding")
                   if embedding.get("scale") is not None else 1.0, torch_dtype=dtype)

    def to_dict(self) -> dict:
        """A config.json that `from_dict` reads back to the same configuration."""
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
                "postln_alpha": self.alpha, "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers], "torch_dtype": self.torch_dtype}


_ATTENTION_NAMES = (("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("q_norm", "q.norm"), ("k_norm", "k.norm"),
                    ("rel", "rel"))


def cache_windows(cfg: PoresunConfig) -> dict:
    """For every attention layer that owns a cache, how many keys it has to keep: its own window,
    or more where a layer that reads its cache looks further back (None: everything)."""
    kept = {}
    for i, layer in enumerate(cfg.layers):
        if layer.type == "latent_attention":
            continue
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        window = layer.mixer.window
        if owner not in kept:
            kept[owner] = window
        elif kept[owner] is not None:
            kept[owner] = None if window is None else max(kept[owner], window)
    return kept


def mixer_spec(layer: PoresunLayer, eps: float, cache_window="own"):
    m = layer.mixer
    if layer.type == "latent_attention":
        return LatentAttentionSpec(num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim,
                                   q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=eps, rot_theta=m.rot_base,
                                   rotated=m.rot_dims, output_gate=True)
    return AttentionSpec(num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, qkv_bias=False, out_bias=False,
                         scale=m.scale, window=m.window, value_dim=m.vdim, softcap=m.softcap,
                         query_temperature=m.q_temp, qk_norm=(eps, m.weighted_norm), bucket_bias=(m.bias_rows, m.bias_max),
                         shared_kv=m.kv_from is not None, cache_window=cache_window, names=_ATTENTION_NAMES)


def ffn_spec(mlp):
    if mlp is None:
        return None
    if isinstance(mlp, BoundedDense):
        return SwiGLUSpec(intermediate_size=mlp.ff, activation=DENSE_ACTIVATION, limit=mlp.limit,
                          up_shift=DENSE_UP_SHIFT, names=(("gate", "gate"), ("up", "up"), ("down", "down")))
    return MoESpec(experts=mlp.experts, top=mlp.top, expert_size=mlp.ff, shared_size=mlp.shared_ff, correction=False,
                   activation=EXPERT_ACTIVATION, gated=False, router_bias=True, shared_gate=mlp.shared_ff is not None)


def build_spec(cfg: PoresunConfig) -> ModelSpec:
    norm = RMSNormSpec(eps=cfg.norm_eps, names=(("weight", ""),))
    kept = cache_windows(cfg)
    blocks, schedule = [], []
    for i, layer in enumerate(cfg.layers):
        own = layer.type != "latent_attention" and layer.mixer.kv_from is None
        window = kept[i] if own and kept[i] != layer.mixer.window else "own"
        blocks.append(PostNormBlockSpec(name=f"l{i}", mixer=mixer_spec(layer, cfg.norm_eps, window),
                                        ffn=ffn_spec(layer.mlp), mixer_norm=norm, ffn_norm=norm, alpha=cfg.alpha,
                                        layer_scale=True))
        schedule.append(ScheduleEntry(i, cache_of=getattr(layer.mixer, "kv_from", None)))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        blocks=tuple(blocks),
        final_norm=norm,
        tie_word_embeddings=True,
        schedule=tuple(schedule),
        embed_name="embed",
        final_norm_name="final.norm",
        head_name="head",
        stored_dtype=cfg.torch_dtype,
        embedding=TokenEmbeddingSpec(cfg.vocab, scale=cfg.embedding_scale, names=(("weight", ""),)),
        head=LinearHeadSpec(cfg.vocab, names=(("weight", ""),)),
    )


register_architecture(ARCHITECTURE, PoresunConfig, build_spec)
