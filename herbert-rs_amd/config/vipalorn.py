"""Typed configuration of the Vipalorn decoder: layers listed one by one, each with a mixer (a gated
delta rule or an attention over a shared latent) beside an optional feed-forward of routed experts.

config.json names the design under "architecture"; every size and every constant that can differ
between models is a key here, nothing is defaulted from another key, and an unknown layer type or
feed-forward kind is an error.
"""
from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import ConfigError
from .base import Reader

# The design names no longest sequence: positions are bounded by what the cache holds.
MAX_POSITIONS = 1 << 20


def _section(raw, key, where):
    v = raw.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}{key} must be an object")
    return Reader(v)


@dataclass(frozen=True)
class DeltaMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int

    @staticmethod
    def from_reader(r, where):
        c = DeltaMixerConfig(*(r.integer(k, required=True) for k in ("heads", "kv_heads", "dim", "vdim", "conv")))
        if min(c.heads, c.kv_heads, c.dim, c.vdim, c.conv) <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"config.json: {where}: sizes must be positive and heads a multiple of kv_heads")
        return c

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot_base: float
    rot_dims: int

    @staticmethod
    def from_reader(r, where):
        rot = _section(r.raw, "rot", where + ".")
        c = LatentMixerConfig(r.integer("heads", required=True), r.integer("dim", required=True),
                              r.integer("rot_dim", required=True), r.integer("vdim", required=True),
                              r.integer("kv_rank", required=True), r.number("scale", required=True),
                              rot.number("base", required=True), rot.integer("dims", required=True))
        if min(c.heads, c.dim, c.vdim, c.kv_rank) <= 0 or c.rot_dim < 0:
            raise ConfigError(f"config.json: {where}: sizes must be positive")
        if c.rot_dims % 2 or not 0 <= c.rot_dims <= c.rot_dim:
            raise ConfigError(f"config.json: {where}: rot.dims must be even and at most rot_dim")
        return c

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": {"base": self.rot_base, "dims": self.rot_dims}}


@dataclass(frozen=True)
class ExpertsConfig:
    experts: int
    top: int
    ff: int
    limit: float

    @staticmethod
    def from_reader(r, where):
        kind = r.raw.get("kind")
        if kind != "moe":
            raise ConfigError(f"config.json: {where}: unknown feed-forward kind {kind!r} (known: 'moe')")
        expert, router = _section(r.raw, "expert", where + "."), _section(r.raw, "router", where + ".")
        c = ExpertsConfig(router.integer("experts", required=True), router.integer("top", required=True),
                          expert.integer("ff", required=True), expert.number("limit", required=True))
        if not 0 < c.top <= c.experts or c.ff <= 0:
            raise ConfigError(f"config.json: {where}: top must be within 1..experts and ff positive")
        return c

    def to_dict(self):
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top}}


MIXERS = {"delta": DeltaMixerConfig, "latent_attention": LatentMixerConfig}


@dataclass(frozen=True)
class VipalornLayer:
    type: str
    mixer: object
    mlp: Optional[ExpertsConfig]

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class VipalornConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[VipalornLayer, ...]
    norm_eps: float
    residual_mult: float
    logit_scale: float
    eos_token_id: Optional[int] = None
    max_position_embeddings: int = MAX_POSITIONS

    @property
    def num_hidden_layers(self):
        return len(self.layers)

    @staticmethod
    def from_dict(raw):
        r = Reader(raw)
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: layers must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(listed):
            where = f"layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"config.json: {where} must be an object")
            kind = entry.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r} (known: {', '.join(sorted(MIXERS))})")
            mixer = MIXERS[kind].from_reader(_section(entry, "mixer", where + "."), where + ".mixer")
            mlp = None
            if entry.get("mlp") is not None:
                mlp = ExpertsConfig.from_reader(_section(entry, "mlp", where + "."), where + ".mlp")
            layers.append(VipalornLayer(kind, mixer, mlp))
        cfg = VipalornConfig(r.integer("vocab", required=True), r.integer("width", required=True), tuple(layers),
                             _section(raw, "norm", "").number("eps", required=True),
                             r.number("residual_mult", required=True), r.number("logit_scale", required=True))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        return cfg

    def to_dict(self):
        return {"architecture": "Vipalorn", "vocab": self.vocab_size, "width": self.hidden_size,
                "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "logit_scale": self.logit_scale}
