"""Typed configuration of the Mefatar decoder: pre-norm layers listed one by one, each a mixer (a real-gated
linear recurrent unit, or two mixers side by side: a filtered, rotated softmax attention with a sink and a
linear attention whose state decays channel by channel) and an optional dense feed-forward, every branch
times a learned scale a channel; a run of adjacent layers may be repeated with the same weights.

config.json names the design under "architecture"; every size and every constant that can differ between
models is a key here, and an unknown layer type or feed-forward kind is an error. Sizes that only the stored
tensors give (the narrow middle of the linear attention's decay) stay open unless the optional key "rank"
names them (a random model needs it named).
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
class RotationScaling:
    """Long wavelengths turn slower: beyond original / low by `factor`, under original / high not at all."""
    factor: float
    low: float
    high: float
    original: float

    def to_dict(self):
        return {"factor": self.factor, "low": self.low, "high": self.high, "original": self.original}


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    scaling: Optional[RotationScaling] = None

    @staticmethod
    def from_reader(r, where):
        scaling = None
        if r.raw.get("scaling") is not None:
            s = _section(r.raw, "scaling", where + ".")
            scaling = RotationScaling(*(s.number(k, required=True) for k in ("factor", "low", "high", "original")))
            if scaling.factor <= 0 or scaling.original <= 0 or scaling.low <= 0 or scaling.high <= scaling.low:
                raise ConfigError(f"config.json: {where}.scaling: factor, original and low must be positive and high above low")
        rot = Rotation(r.integer("dims", required=True), r.number("base", required=True), scaling)
        if rot.dims <= 0 or rot.dims % 2 or rot.base <= 0:
            raise ConfigError(f"config.json: {where}: dims must be even and positive, base positive")
        return rot

    def to_dict(self):
        d = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            d["scaling"] = self.scaling.to_dict()
        return d


@dataclass(frozen=True)
class LeftConfig:
    """The softmax attention of a "parallel" layer."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: Optional[int]              # taps of the filter on queries, keys and values; None: no filter
    rot: Optional[Rotation]          # None: no rotation

    @staticmethod
    def from_reader(r, where):
        rot = None
        if r.raw.get("rot") is not None:
            rot = Rotation.from_reader(_section(r.raw, "rot", where + "."), where + ".rot")
        c = LeftConfig(*(r.integer(k, required=True) for k in ("heads", "kv_heads", "dim", "vdim")),
                       r.number("scale", required=True), r.integer("conv"), rot)
        _positive(where, heads=c.heads, kv_heads=c.kv_heads, dim=c.dim, vdim=c.vdim)
        if c.heads % c.kv_heads:
            raise ConfigError(f"config.json: {where}: heads must be a multiple of kv_heads")
        if c.conv is not None and c.conv <= 0:
            raise ConfigError(f"config.json: {where}.conv must be positive")
        if rot is not None and rot.dims > c.dim:
            raise ConfigError(f"config.json: {where}.rot.dims exceeds the keys' size")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.conv is not None:
            d["conv"] = self.conv
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        return d


@dataclass(frozen=True)
class RightConfig:
    """The linear attention of a "parallel" layer."""
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: Optional[int] = None       # the decay's narrow middle; None: whatever the stored tensors have

    @staticmethod
    def from_reader(r, where):
        c = RightConfig(*(r.integer(k, required=True) for k in ("heads", "dim", "vdim")), r.number("tau", required=True),
                        r.integer("rank"))
        _positive(where, heads=c.heads, dim=c.dim, vdim=c.vdim, tau=c.tau)
        if c.rank is not None and c.rank <= 0:
            raise ConfigError(f"config.json: {where}.rank must be positive")
        return c

    def to_dict(self):
        d = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "tau": self.tau}
        if self.rank is not None:
            d["rank"] = self.rank
        return d


@dataclass(frozen=True)
class ParallelMixerConfig:
    left: LeftConfig
    right: RightConfig

    @staticmethod
    def from_reader(r, where):
        return ParallelMixerConfig(LeftConfig.from_reader(_section(r.raw, "left", where + "."), where + ".left"),
                                   RightConfig.from_reader(_section(r.raw, "right", where + "."), where + ".right"))

    def to_dict(self):
        return {"left": self.left.to_dict(), "right": self.right.to_dict()}


@dataclass(frozen=True)
class RecurrentMixerConfig:
    """The real-gated linear recurrent unit between its two branches."""
    width: int
    blocks: int
    conv: int

    @staticmethod
    def from_reader(r, where):
        c = RecurrentMixerConfig(*(r.integer(k, required=True) for k in ("width", "blocks", "conv")))
        _positive(where, width=c.width, blocks=c.blocks, conv=c.conv)
        if c.width % c.blocks:
            raise ConfigError(f"config.json: {where}: width must be a multiple of blocks")
        return c

    def to_dict(self):
        return {"width": self.width, "blocks": self.blocks, "conv": self.conv}


@dataclass(frozen=True)
class DenseConfig:
    ff: int

    def to_dict(self):
        return {"kind": "dense", "ff": self.ff}


MIXERS = {"rglru": RecurrentMixerConfig, "parallel": ParallelMixerConfig}


@dataclass(frozen=True)
class MefatarLayer:
    type: str
    mixer: object
    mlp: Optional[DenseConfig]

    def to_dict(self):
        return {"type": self.type, "mixer": self.mixer.to_dict(), "mlp": None if self.mlp is None else self.mlp.to_dict()}


@dataclass(frozen=True)
class Loop:
    """Layers start .. stop - 1 run `times` times in a row with the same weights."""
    start: int
    stop: int
    times: int

    def to_dict(self):
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclass(frozen=True)
class MefatarConfig:
    vocab_size: int
    hidden_size: int
    layers: Tuple[MefatarLayer, ...]
    norm_eps: float
    loop: Optional[Loop] = None
    eos_token_id: Optional[int] = None
    max_position_embeddings: int = MAX_POSITIONS

    @property
    def num_hidden_layers(self):
        return len(self.layers)

    def layer_runs(self):
        """The layers in the order they run."""
        n = len(self.layers)
        if self.loop is None:
            return list(range(n))
        lp = self.loop
        return list(range(lp.start)) + list(range(lp.start, lp.stop)) * lp.times + list(range(lp.stop, n))

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
                if m.raw.get("kind") != "dense":
                    raise ConfigError(f"config.json: {where}.mlp: unknown feed-forward kind {m.raw.get('kind')!r} (known: 'dense')")
                mlp = DenseConfig(m.integer("ff", required=True))
                if mlp.ff <= 0:
                    raise ConfigError(f"config.json: {where}.mlp.ff must be positive")
            layers.append(MefatarLayer(kind, mixer, mlp))
        loop = None
        if raw.get("loop") is not None:
            lp = _section(raw, "loop", "")
            loop = Loop(*(lp.integer(k, required=True) for k in ("start", "stop", "times")))
            if not (0 <= loop.start <= loop.stop <= len(layers)) or loop.times < 1:
                raise ConfigError(f"config.json: loop: layers {loop.start} .. {loop.stop} x {loop.times} of {len(layers)} layers")
        cfg = MefatarConfig(r.integer("vocab", required=True), r.integer("width", required=True), tuple(layers),
                            _section(raw, "norm", "").number("eps", required=True), loop, r.integer("eos_token_id"))
        if cfg.vocab_size <= 0 or cfg.hidden_size <= 0:
            raise ConfigError("config.json: vocab and width must be positive")
        return cfg

    def to_dict(self):
        d = {"architecture": "Mefatar", "vocab": self.vocab_size, "width": self.hidden_size,
             "layers": [l.to_dict() for l in self.layers], "norm": {"eps": self.norm_eps}}
        if self.loop is not None:
            d["loop"] = self.loop.to_dict()
        if self.eos_token_id is not None:
            d["eos_token_id"] = self.eos_token_id
        return d
