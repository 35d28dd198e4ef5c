"""Typed configuration of the Modasun decoder: layers listed one by one, each a mixer (a softmax attention
without rotation, or a gated delta rule with a decay a key channel) and an optional feed-forward (dense, or
a mixture of experts beside a shared expert), with the norm after each sum. A layer may run an earlier
layer's weights with a cache or state of its own.

config.json names the design under "architecture"; every size and every constant that can differ between
models is a key here, an unknown layer type or feed-forward kind is an error, and the sizes that only the
stored tensors give (the narrow middles of a delta layer's two-step projections) stay open unless the
optional key "low_rank" names them (a random model needs them named).
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
class AttentionMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp_coef: float
    q_temp_every: int

    @staticmethod
    def from_reader(r, where):
        # (a mixer without "q_temp", or with null there, has queries that do not grow: coef 0)
        coef, every = 0.0, 1
        if r.raw.get("q_temp") is not None:
            t = _section(r.raw, "q_temp", where + ".")
            coef, every = t.number("coef", required=True), t.integer("every", required=True)
        c = AttentionMixerConfig(*(r.integer(k, required=True) for k in ("heads", "kv_heads", "dim", "vdim")),
                                 r.number("scale", required=True), coef, every)
        if min(c.heads, c.kv_heads, c.dim, c.vdim, c.q_temp_every) <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"config.json: {where}: sizes must be positive and heads a multiple of kv_heads")
        return c

    def to_dict(self):
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "q_temp": {"coef": self.q_temp_coef, "every": self.q_temp_every}}


@dataclass(frozen=True)
class ChannelDeltaMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    decay_rank: Optional[int] = None       # None: whatever the stored tensors have
    gate_rank: Optional[int] = None

    @staticmethod
    def from_reader(r, where):
        ranks = (None, None)
        if r.has("low_rank"):
            lr = _section(r.raw, "low_rank", where + ".")
            ranks = (lr.integer("decay", required=True), lr.integer("gate", required=True))
        c = ChannelDeltaMixerConfig(*(r.integer(k, required=True) for k in ("heads", "kv_heads", "dim", "vdim", "conv")),
                                    *ranks)
        if min(c.heads, c.kv_heads, c.dim, c.vdim, c.conv) <= 0 or c.heads % c.kv_heads:
            raise ConfigError(f"config.json: {where}: sizes must be positive and heads a multiple of kv_heads")
        if any(v is not None and v <= 0 for v in ranks):
            raise ConfigError(f"config.json: {where}.low_rank: sizes must be positive")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}
        if self.decay_rank is not None and self.gate_rank is not None:
            d["low_rank"] = {"decay": self.decay_rank, "gate": self.gate_rank}
        return d


@dataclass(frozen=True)
class DenseConfig:
    ff: int

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class ExpertsConfig:
    experts: int
    top: int
    groups: int
    keep: int
    ff: int
    shared_ff: Optional[int]         # None: no shared expert

    def to_dict(self):
        d = {"kind": "moe", "expert": {"ff": self.ff},
             "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.keep}}}
        if self.shared_ff is not None:
            d["shared"] = {"ff": self.shared_ff}
        return d


def _mlp(r, where):
    kind = r.raw.get("kind")
    if kind == "dense":
        c = DenseConfig(r.integer("ff", required=True))
        if c.ff <= 0:
            raise ConfigError(f"config.json: {where}: ff must be positive")
        return c
    if kind != "moe":
        raise ConfigError(f"config.json: {where}: unknown feed-forward kind {kind!r} (known: 'dense', 'moe')")
    expert, router = _section(r.raw, "expert", where + "."), _section(r.raw, "router", where + ".")
    # (a router without "groups" has one group of all experts; a feed-forward without "shared" no shared expert)
    count, keep, shared_ff = 1, 1, None
    if router.raw.get("groups") is not None:
        groups = _section(router.raw, "groups", where + ".router.")
        count, keep = groups.integer("count", required=True), groups.integer("keep", required=True)
    if r.raw.get("shared") is not None:
        shared_ff = _section(r.raw, "shared", where + ".").integer("ff", required=True)
    c = ExpertsConfig(router.integer("experts", required=True), router.integer("top", required=True), count, keep,
                      expert.integer("ff", required=True), shared_ff)
    if not 0 < c.top <= c.experts or c.ff <= 0 or (c.shared_ff is not None and c.shared_ff <= 0):
        raise ConfigError(f"config.json: {where}: top must be within 1..experts and the widths positive")
    if c.groups <= 0 or c.experts % c.groups or not 0 < c.keep <= c.groups or c.top > c.keep * (c.experts // c.groups):
        raise ConfigError(f"config.json: {where}: {c.top} experts cannot come from {c.keep} of {c.groups} equal "
                          f"groups of {c.experts} experts")
    return c


MIXERS = {"attention": AttentionMixerConfig, "channel_delta": ChannelDeltaMixerConfig}


@dataclass(frozen=True)
class ModasunLayer:
    type: str
    mixer: object
    mlp: object                      # DenseConfig, ExpertsConfig or None
    weights_of: Optional[int] = None  # the layer whose tensors this one runs (None: its own)

    def to_dict(self):
        d = {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}
        if self.weights_of is not None:
            d["weights_of"] = self.weights_of
        return d


@dataclass(frozen=True)
class ModasunConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[ModasunLayer, ...]
    norm_eps: float
    postln_alpha: float
    embedding_scale: float
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
                mlp = _mlp(_section(entry, "mlp", where + "."), where + ".mlp")
            layers.append(ModasunLayer(kind, mixer, mlp, Reader(entry).integer("weights_of")))
        for i, layer in enumerate(layers):
            if layer.weights_of is None:
                continue
            # the layer whose tensors are run: the end of the chain, if the named layer runs another's itself
            source, seen = layer.weights_of, {i}
            while True:
                if not 0 <= source < len(layers) or source in seen:
                    raise ConfigError(f"config.json: layers[{i}].weights_of must name another layer that has tensors "
                                      "of its own")
                if layers[source].weights_of is None:
                    break
                seen.add(source)
                source = layers[source].weights_of
            theirs = layers[source]
            if (theirs.type, theirs.mixer, theirs.mlp) != (layer.type, layer.mixer, layer.mlp):
                raise ConfigError(f"config.json: layers[{i}] runs the weights of layer {source} but differs from it")
            layers[i] = ModasunLayer(layer.type, layer.mixer, layer.mlp, source)
        cfg = ModasunConfig(r.integer("vocab", required=True), r.integer("width", required=True), tuple(layers),
                            _section(raw, "norm", "").number("eps", required=True),
                            r.number("postln_alpha", required=True),
                            _section(raw, "embedding", "").number("scale", required=True))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        if cfg.postln_alpha == 0.0:
            raise ConfigError("config.json: postln_alpha must not be zero")
        return cfg

    def to_dict(self):
        return {"architecture": "Modasun", "vocab": self.vocab_size, "width": self.hidden_size,
                "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps},
                "postln_alpha": self.postln_alpha, "embedding": {"scale": self.embedding_scale}}
