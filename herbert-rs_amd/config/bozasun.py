"""Typed configuration of the Bozasun decoder: pre-norm layers listed one by one, each a mixer (a softmax attention
over the keys of the query's own chunk of positions, an attention over one shared latent a token, or a state-space
layer with one decay a head) and an optional feed-forward (dense, or a mixture of experts among which some are the
identity), and, where the model has one, a per-layer input from a table of the tokens' ids.

config.json names the design under "architecture"; every size and every constant that can differ between models is
a key here, and an unknown layer type or feed-forward kind is an error. A section that a model leaves out switches
its mechanism off: "mask" (the attention then sees every earlier key), "rot", "rot.scaling", "softcap", the
router's "groups" and "identity", "norm_groups" (one group), "mlp", "token_side".
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


def _positive(where, **values):
    for name, v in values.items():
        if v is None or v <= 0:
            raise ConfigError(f"config.json: {where}.{name} must be positive")


@dataclass(frozen=True)
class Rotation:
    """Neighbouring pairs of a head's first `dims` entries turn by position x base^(-2i / dims) / factor."""
    dims: int
    base: float
    factor: Optional[float] = None          # of the linear scaling; None: none

    @staticmethod
    def from_raw(raw, where):
        if raw.get("rot") is None:
            return None
        r = _section(raw, "rot", where + ".")
        factor = None
        if r.raw.get("scaling") is not None:
            factor = _section(r.raw, "scaling", where + ".rot.").number("factor", required=True)
        rot = Rotation(r.integer("dims", required=True), r.number("base", required=True), factor)
        if rot.dims <= 0 or rot.dims % 2 or rot.base <= 0 or (factor is not None and factor <= 0):
            raise ConfigError(f"config.json: {where}.rot: dims must be even and positive, base and scaling.factor positive")
        return rot

    def to_dict(self):
        d = {"dims": self.dims, "base": self.base}
        if self.factor is not None:
            d["scaling"] = {"factor": self.factor}
        return d


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation] = None
    chunk: Optional[int] = None             # mask.size; None: every earlier key is seen
    softcap: Optional[float] = None

    @staticmethod
    def from_reader(r, where):
        chunk = None
        if r.raw.get("mask") is not None:
            chunk = _section(r.raw, "mask", where + ".").integer("size", required=True)
        c = AttentionConfig(*(r.integer(k, required=True) for k in ("heads", "kv_heads", "dim", "vdim")),
                            r.number("scale", required=True), Rotation.from_raw(r.raw, where), chunk, r.number("softcap"))
        _positive(where, heads=c.heads, kv_heads=c.kv_heads, dim=c.dim, vdim=c.vdim, scale=c.scale)
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: {where}: heads must be a multiple of kv_heads")
        if c.rot is not None and c.rot.dims > c.dim:
            raise ConfigError(f"config.json: {where}.rot.dims exceeds the keys' size")
        if (c.chunk is not None and c.chunk <= 0) or (c.softcap is not None and c.softcap <= 0):
            raise ConfigError(f"config.json: {where}: mask.size and softcap must be positive")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        if self.chunk is not None:
            d["mask"] = {"size": self.chunk}
        if self.softcap is not None:
            d["softcap"] = self.softcap
        return d


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: Rotation

    @staticmethod
    def from_reader(r, where):
        rot = Rotation.from_raw(r.raw, where)
        c = LatentAttentionConfig(*(r.integer(k, required=True) for k in ("heads", "dim", "rot_dim", "vdim", "kv_rank")),
                                  r.number("scale", required=True), rot)
        _positive(where, heads=c.heads, dim=c.dim, rot_dim=c.rot_dim, vdim=c.vdim, kv_rank=c.kv_rank, scale=c.scale)
        if rot is None or rot.dims != c.rot_dim:
            raise ConfigError(f"config.json: {where}.rot.dims must be rot_dim: the whole rotated part turns")
        return c

    def to_dict(self):
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class StateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1

    @staticmethod
    def from_reader(r, where):
        c = StateSpaceConfig(*(r.integer(k, required=True) for k in ("heads", "vdim", "state", "groups", "conv")),
                             r.integer("norm_groups", 1))
        _positive(where, heads=c.heads, vdim=c.vdim, state=c.state, groups=c.groups, conv=c.conv, norm_groups=c.norm_groups)
        if c.heads % c.groups or (c.heads * c.vdim) % c.norm_groups:
            raise ConfigError(f"config.json: {where}: heads must be a multiple of groups, and norm_groups divide heads x vdim")
        return c

    def to_dict(self):
        return {"heads": self.heads, "vdim": self.vdim, "state": self.state, "groups": self.groups, "conv": self.conv,
                "norm_groups": self.norm_groups}


@dataclass(frozen=True)
class DenseConfig:
    ff: int

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff}


@dataclass(frozen=True)
class ExpertsConfig:
    ff: int
    experts: int
    top: int
    identity: int = 0                       # further outputs of the router whose "expert" is the identity
    groups: Optional[Tuple[int, int]] = None    # (count, keep); None: every expert can be chosen

    @property
    def routed(self):
        return self.experts + self.identity

    @staticmethod
    def from_reader(m, where):
        e = _section(m.raw, "expert", where + ".")
        r = _section(m.raw, "router", where + ".")
        groups = None
        if r.raw.get("groups") is not None:
            g = _section(r.raw, "groups", where + ".router.")
            groups = (g.integer("count", required=True), g.integer("keep", required=True))
        c = ExpertsConfig(e.integer("ff", required=True), r.integer("experts", required=True),
                          r.integer("top", required=True), r.integer("identity", 0), groups)
        _positive(where, ff=c.ff, experts=c.experts, top=c.top)
        if c.identity < 0 or c.top > c.routed:
            raise ConfigError(f"config.json: {where}.router: {c.top} of {c.experts} + {c.identity} experts")
        if groups is not None:
            count, keep = groups
            if count <= 0 or c.routed % count or not 0 < keep <= count or c.top > keep * (c.routed // count):
                raise ConfigError(f"config.json: {where}.router.groups: {c.top} experts cannot come from {keep} of "
                                  f"{count} groups of {c.routed} experts")
        return c

    def to_dict(self):
        router = {"experts": self.experts, "top": self.top}
        if self.identity:
            router["identity"] = self.identity
        if self.groups is not None:
            router["groups"] = {"count": self.groups[0], "keep": self.groups[1]}
        return {"kind": "moe", "expert": {"ff": self.ff}, "router": router}


MIXERS = {"attention": AttentionConfig, "latent_attention": LatentAttentionConfig, "mamba2": StateSpaceConfig}


@dataclass(frozen=True)
class BozasunLayer:
    type: str
    mixer: object
    mlp: object                              # DenseConfig, ExpertsConfig or None

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class BozasunConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[BozasunLayer, ...]
    norm_eps: float
    side_dim: Optional[int] = None           # token_side.dim; None: the model has no per-layer token input
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
                m = _section(entry, "mlp", where + ".")
                if m.raw.get("kind") == "dense":
                    mlp = DenseConfig(m.integer("ff", required=True))
                    if mlp.ff <= 0:
                        raise ConfigError(f"config.json: {where}.mlp.ff must be positive")
                elif m.raw.get("kind") == "moe":
                    mlp = ExpertsConfig.from_reader(m, where + ".mlp")
                else:
                    raise ConfigError(f"config.json: {where}.mlp: unknown feed-forward kind {m.raw.get('kind')!r} "
                                      "(known: 'dense', 'moe')")
            layers.append(BozasunLayer(kind, mixer, mlp))
        side = None
        if raw.get("token_side") is not None:
            side = _section(raw, "token_side", "").integer("dim", required=True)
            if side <= 0:
                raise ConfigError("config.json: token_side.dim must be positive")
        cfg = BozasunConfig(r.integer("vocab", required=True), r.integer("width", required=True), tuple(layers),
                            _section(raw, "norm", "").number("eps", required=True), side, r.integer("eos_token_id"))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        return cfg

    def to_dict(self):
        d = {"architecture": "Bozasun", "vocab": self.vocab_size, "width": self.hidden_size,
             "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps}}
        if self.side_dim is not None:
            d["token_side"] = {"dim": self.side_dim}
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d
