"""Ligipel: a decoder whose layers have a norm before and after each sublayer, whose stream
between layers is a learned weighted sum of every earlier layer's result, whose mixer is
either an attention and a selective scan side by side or retention, and whose feed-forward
is a routed mixture of experts.

config.json (every size and every constant that can differ between models):

    architecture   "Ligipel"
    vocab, width
    norm           {eps}                     all norms
    logit_scale, logit_softcap               logits = cap * tanh(head x * scale / cap)
    layers[i]      {type, mixer: {...}, mlp: {kind: "moe", expert: {ff}, router: {experts, top},
                                               shared: {ff}} | null}

    type "parallel"    mixer {left: {heads, kv_heads, dim, vdim, scale, mask: {size}},
                              right: {inner, state, dt_rank, conv}}
        left: grouped-query attention without rotation; r1 ln(1 + r2 distance) is taken off the
        scores (two learned numbers per head); sliding window; a sink of score 0 in the
        softmax's denominator; the weights are mixed across heads by a learned matrix.
        right: the selective scan of Mamba.  Each output is brought to unit root mean square
        and weighted; the mixer's result is half their sum.
    type "retention"   mixer {heads, dim, vdim, decay: [per head], rot: {base, dims}}
        linear attention with a fixed decay per head; rotation of the first rot.dims elements
        of a head, pairs (i, i + dims / 2)

Tensors: embed, embed.norm(.b), head, final.norm(.b), and per layer l<i>.norm1, norm1b, norm2,
norm2b (each with .b), l<i>.mix.* (by mixer), l<i>.mlp.{e<k>.{gate,up,down}, router, correction,
shared.{gate,up,down}}, l<i>.dwa (i + 2 numbers).  All norms are layer norms with weight and
bias.  A layer is x += norm1b(mixer(norm1(x))); x += norm2b(mlp(norm2(x))); what goes on after
layer i is sum_j dwa[j] X_j over the embedding's output X_0 and the layers' results X_1 ..
X_(i+1).  The embedding's output is the normed lookup.
"""

from __future__ import annotations

from dataclasses import dataclass

from ..config.engine_config import canonical_dtype
from ..config.registry import ConfigError, register_architecture
from ..config.specs import (
    AttentionSpec,
    LayerNormSpec,
    LinearHeadSpec,
    MoESpec,
    ModelSpec,
    ParallelMixerSpec,
    RetentionSpec,
    RotarySpec,
    SandwichBlockSpec,
    ScheduleEntry,
    SelectiveScanSpec,
    TokenEmbeddingSpec,
)

ARCHITECTURE = "Ligipel"
MIXERS = ("parallel", "retention")
SINK_SCORE = 0.0  # the design's sink: one more term exp(0) in every head's denominator
BRANCH_SCALE = 0.5  # the mixer's result is half the sum of its two normed outputs


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
class BiasedAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "BiasedAttention":
        dim = _get(raw, "dim", int, where)
        mask = raw.get("mask")
        out = cls(heads=_get(raw, "heads", int, where), kv_heads=_get(raw, "kv_heads", int, where), dim=dim,
                  vdim=_get(raw, "vdim", int, where) if raw.get("vdim") is not None else dim,
                  scale=_get(raw, "scale", float, where),
                  window=None if mask is None else _get(mask, "size", int, where + ".mask"))
        _positive(where, heads=out.heads, kv_heads=out.kv_heads, dim=out.dim, vdim=out.vdim)
        if out.window is not None:
            _positive(where + ".mask", size=out.window)
        if out.heads % out.kv_heads:
            raise ConfigError(f"{where}: {out.heads} heads are not a multiple of {out.kv_heads} kv_heads")
        return out

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.window is not None:
            out["mask"] = {"size": self.window}
        return out


@dataclass(frozen=True)
class Scan:
    inner: int
    state: int
    dt_rank: int
    conv: int

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "Scan":
        out = cls(inner=_get(raw, "inner", int, where), state=_get(raw, "state", int, where),
                  dt_rank=_get(raw, "dt_rank", int, where), conv=_get(raw, "conv", int, where))
        _positive(where, inner=out.inner, state=out.state, dt_rank=out.dt_rank, conv=out.conv)
        return out

    def to_dict(self) -> dict:
        return {"inner": self.inner, "state": self.state, "dt_rank": self.dt_rank, "conv": self.conv}


@dataclass(frozen=True)
class SideBySide:
    left: BiasedAttention
    right: Scan

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "SideBySide":
        return cls(left=BiasedAttention.from_dict(_get(raw, "left", dict, where), where + ".left"),
                   right=Scan.from_dict(_get(raw, "right", dict, where), where + ".right"))

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class DecayedRetention:
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot_base: float
    rot_dims: int

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "DecayedRetention":
        dim = _get(raw, "dim", int, where)
        rot = raw.get("rot") or {}
        dims = _get(rot, "dims", int, where + ".rot") if rot.get("dims") is not None else 0
        if dims < 0 or dims % 2 or dims > dim:
            raise ConfigError(f"{where}: rot.dims ({dims}) must be even and at most dim ({dim})")
        decay = raw.get("decay")
        if not isinstance(decay, (list, tuple)) or any(isinstance(d, bool) or not isinstance(d, (int, float))
                                                       for d in decay):
            raise ConfigError(f"{where}: decay must be a list of one number per head")
        out = cls(heads=_get(raw, "heads", int, where), dim=dim,
                  vdim=_get(raw, "vdim", int, where) if raw.get("vdim") is not None else dim,
                  decay=tuple(float(d) for d in decay),
                  rot_base=_get(rot, "base", float, where + ".rot") if dims else 1.0, rot_dims=dims)
        _positive(where, heads=out.heads, dim=out.dim, vdim=out.vdim, rot_base=out.rot_base)
        if len(out.decay) != out.heads:
            raise ConfigError(f"{where}: {len(out.decay)} decays for {out.heads} heads")
        return out

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rot_dims:
            out["rot"] = {"base": self.rot_base, "dims": self.rot_dims}
        return out


@dataclass(frozen=True)
class Mixture:
    experts: int
    top: int
    ff: int
    shared_ff: int | None

    @classmethod
    def from_dict(cls, raw: dict, where: str) -> "Mixture":
        if raw.get("kind") != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {raw.get('kind')!r} (known: moe)")
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


_MIXER_CONFIGS = {"parallel": SideBySide, "retention": DecayedRetention}


@dataclass(frozen=True)
class LigipelLayer:
    type: str
    mixer: object
    mlp: Mixture | None

    def to_dict(self) -> dict:
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class LigipelConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: tuple[LigipelLayer, ...]
    logit_scale: float = 1.0
    logit_softcap: float | None = None
    torch_dtype: str = "bfloat16"

    def __post_init__(self):
        if self.vocab < 1 or self.width < 1 or not self.layers:
            raise ConfigError("config.json: vocab, width and the number of layers must be positive")
        if not self.norm_eps > 0:
            raise ConfigError(f"config.json: norm.eps must be > 0, got {self.norm_eps}")
        if self.logit_softcap is not None and not self.logit_softcap > 0:
            raise ConfigError(f"config.json: logit_softcap must be > 0, got {self.logit_softcap}")

    @classmethod
    def from_dict(cls, raw: dict) -> "LigipelConfig":
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: layers must be a non-empty list")
        layers = []
        for i, entry in enumerate(listed):
            where = f"config.json layers[{i}]"
            kind = _get(entry, "type", str, where)
            if kind not in _MIXER_CONFIGS:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} (known: {', '.join(MIXERS)})")
            mlp = entry.get("mlp")
            mixer = _MIXER_CONFIGS[kind].from_dict(_get(entry, "mixer", dict, where), where + ".mixer")
            layers.append(LigipelLayer(kind, mixer, None if mlp is None else Mixture.from_dict(mlp, where + ".mlp")))
        dtype = raw.get("torch_dtype") or "bfloat16"
        try:
            dtype = canonical_dtype(dtype)
        except ValueError as e:
            raise ConfigError(f"config.json: {e}") from None
        cap = raw.get("logit_softcap")
        return cls(vocab=_get(raw, "vocab", int), width=_get(raw, "width", int),
                   norm_eps=_get(_get(raw, "norm", dict), "eps", float, "config.json norm"), layers=tuple(layers),
                   logit_scale=_get(raw, "logit_scale", float) if raw.get("logit_scale") is not None else 1.0,
                   logit_softcap=None if cap is None else _get(raw, "logit_softcap", float), torch_dtype=dtype)

    def to_dict(self) -> dict:
        """A config.json that `from_dict` reads back to the same configuration."""
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "logit_scale": self.logit_scale, "layers": [layer.to_dict() for layer in self.layers],
               "torch_dtype": self.torch_dtype}
        if self.logit_softcap is not None:
            out["logit_softcap"] = self.logit_softcap
        return out


_SAME = lambda *roles: tuple((r, r) for r in roles)  # noqa: E731  (tensor sub-names equal to their roles)


def mixer_spec(layer: LigipelLayer, eps: float):
    m = layer.mixer
    if layer.type == "parallel":
        left = AttentionSpec(
            num_heads=m.left.heads, num_kv_heads=m.left.kv_heads, head_dim=m.left.dim, qkv_bias=False,
            out_bias=False, scale=m.left.scale, window=m.left.window, value_dim=m.left.vdim, distance_bias=True,
            fixed_sink=SINK_SCORE, talking_heads=True, names=_SAME("q", "k", "v", "o", "r1", "r2", "talk"))
        right = SelectiveScanSpec(inner=m.right.inner, state=m.right.state, dt_rank=m.right.dt_rank, conv=m.right.conv)
        return ParallelMixerSpec(branches=(("left", left), ("right", right)), eps=eps, scale=BRANCH_SCALE)
    position = RotarySpec(theta=m.rot_base, rotary_dim=m.rot_dims) if m.rot_dims else None
    return RetentionSpec(num_heads=m.heads, head_dim=m.dim, value_dim=m.vdim, decay=m.decay, eps=eps,
                         position=position)


def build_spec(cfg: LigipelConfig) -> ModelSpec:
    norm = LayerNormSpec(eps=cfg.norm_eps, names=(("weight", ""), ("bias", "b")))
    blocks = []
    for i, layer in enumerate(cfg.layers):
        ffn = None
        if layer.mlp is not None:
            ffn = MoESpec(experts=layer.mlp.experts, top=layer.mlp.top, expert_size=layer.mlp.ff,
                          shared_size=layer.mlp.shared_ff, correction=True, activation="silu")
        blocks.append(SandwichBlockSpec(name=f"l{i}", mixer=mixer_spec(layer, cfg.norm_eps), ffn=ffn, mixer_norm=norm,
                                        mixer_post=norm, ffn_norm=norm, ffn_post=norm))
    return ModelSpec(
        architecture=ARCHITECTURE,
        hidden_size=cfg.width,
        vocab_size=cfg.vocab,
        blocks=tuple(blocks),
        final_norm=norm,
        tie_word_embeddings=False,
        schedule=tuple(ScheduleEntry(i, depth_average=f"l{i}.dwa") for i in range(len(blocks))),
        embed_name="embed",
        final_norm_name="final.norm",
        head_name="head",
        stored_dtype=cfg.torch_dtype,
        embedding=TokenEmbeddingSpec(cfg.vocab, names=(("weight", ""),), norm=norm, norm_name="embed.norm"),
        head=LinearHeadSpec(cfg.vocab, names=(("weight", ""),), scale=cfg.logit_scale, softcap=cfg.logit_softcap),
    )


register_architecture(ARCHITECTURE, LigipelConfig, build_spec)
