"""Typed configuration of Fazezen, read from the design's own config.json keys.

A Fazezen file names its design under ``architecture`` (one string), gives ``vocab``, ``width``, ``norm.eps`` and a
list ``layers``; each entry has a ``type`` (the kind of its mixer), the mixer's sizes and constants under ``mixer``
and its feed-forward under ``mlp`` (null: none).  Every size and constant is read from there; a layer may differ from
its neighbours in all of them.

    mixer  (type "lightning"): heads, dim, vdim, decay [one per head]
    mixer  (type "parallel"):  left_scale, right_scale,
           left  {heads, kv_heads, dim, vdim, scale, rot {base, dims, scaling {factor, low, high, original} | null},
                  mask {size} | null}
           right {heads, dim, vdim, decay [one per head], rot {base, dims, scaling ... | null} | null}
    mlp    (kind "dense"): ff

As with the other architectures an unknown key is an error that names the key (a key this reader does not know
would be a mechanism it does not compute); a key whose value is null counts as left out.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..errors import ConfigError

ARCHITECTURE = "Fazezen"
LIGHTNING = "lightning"
PARALLEL = "parallel"
DENSE = "dense"

# the most positions a request may hold when nothing else bounds it: the file has no such key, the rotation tables
# are made for this many, the engine's own context length is what limits a request
DEFAULT_MAX_POSITION = 1 << 15

# keys that describe provenance, read by nobody
_IGNORED = frozenset({"seed", "name", "description", "comment", "dtype", "torch_dtype"})


def _section(raw, where: str, required, optional=()):
    """``raw`` as a dictionary holding exactly the ``required`` keys and any of the ``optional`` ones."""
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object, found {raw!r}", key=where)
    known = set(required) | set(optional) | _IGNORED
    for k, v in raw.items():
        if k not in known and v is not None:
            raise ConfigError(f"unsupported key {k!r} in {where} (no Fazezen feature declares it)", key=f"{where}.{k}")
    for k in required:
        if raw.get(k) is None:
            raise ConfigError(f"{where} lacks the required key {k!r}", key=f"{where}.{k}")
    return raw


def _int(raw, key, where, least=1) -> int:
    v = raw[key]
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"{where}.{key} must be an integer of at least {least}, found {v!r}", key=f"{where}.{key}")
    return v


def _num(raw, key, where, positive=False) -> float:
    v = raw[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)) or (positive and not v > 0):
        raise ConfigError(f"{where}.{key} must be a {'positive ' if positive else ''}number, found {v!r}", key=f"{where}.{key}")
    return float(v)


def _decays(raw, where, heads) -> Tuple[float, ...]:
    v = raw["decay"]
    if not isinstance(v, list) or len(v) != heads:
        raise ConfigError(f"{where}.decay must list one factor per head ({heads})", key=f"{where}.decay")
    out = []
    for i, d in enumerate(v):
        if isinstance(d, bool) or not isinstance(d, (int, float)) or not 0.0 <= d <= 1.0:
            raise ConfigError(f"{where}.decay[{i}] must be a number in [0, 1], found {d!r}", key=f"{where}.decay")
        out.append(float(d))
    return tuple(out)


@dataclass(frozen=True)
class Stretch:
    """How rotation frequencies are stretched for long contexts (by wavelength against ``original``)."""

    factor: float
    low: float
    high: float
    original: float

    def to_json(self) -> dict:
        return {"factor": self.factor, "high": self.high, "low": self.low, "original": self.original}


@dataclass(frozen=True)
class Rotation:
    base: float
    dims: int
    scaling: Optional[Stretch] = None

    @staticmethod
    def from_dict(raw, where: str, most: int) -> "Rotation":
        _section(raw, where, ("base", "dims"), ("scaling",))
        dims = _int(raw, "dims", where, least=0)
        if dims % 2 or dims > most:
            raise ConfigError(f"{where}.dims must be even and at most the head's width {most}, found {dims}", key=f"{where}.dims")
        scaling = None
        if raw.get("scaling") is not None:
            w = where + ".scaling"
            s = _section(raw["scaling"], w, ("factor", "low", "high", "original"))
            scaling = Stretch(_num(s, "factor", w, True), _num(s, "low", w, True), _num(s, "high", w, True),
                              _num(s, "original", w, True))
            if not scaling.high > scaling.low:
                raise ConfigError(f"{w}.high must exceed {w}.low", key=w)
        return Rotation(_num(raw, "base", where, positive=True), dims, scaling)

    def to_json(self) -> dict:
        return {"base": self.base, "dims": self.dims, "scaling": None if self.scaling is None else self.scaling.to_json()}


@dataclass(frozen=True)
class LightningConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]

    @staticmethod
    def from_dict(raw, where: str) -> "LightningConfig":
        _section(raw, where, ("heads", "dim", "vdim", "decay"))
        heads = _int(raw, "heads", where)
        return LightningConfig(heads, _int(raw, "dim", where), _int(raw, "vdim", where), _decays(raw, where, heads))

    def to_json(self) -> dict:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ChunkedAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation]
    chunk: Optional[int]             # mask.size

    def __post_init__(self):
        if self.heads % self.kv_heads:
            raise ConfigError("query heads must be a multiple of key/value heads", heads=self.heads, kv_heads=self.kv_heads)
        if self.rot is not None and self.vdim % 2:
            raise ConfigError("values are turned in pairs: vdim must be even", vdim=self.vdim)

    @staticmethod
    def from_dict(raw, where: str) -> "ChunkedAttentionConfig":
        _section(raw, where, ("heads", "kv_heads", "dim", "vdim", "scale"), ("rot", "mask"))
        dim = _int(raw, "dim", where)
        rot = None if raw.get("rot") is None else Rotation.from_dict(raw["rot"], where + ".rot", dim)
        chunk = None
        if raw.get("mask") is not None:
            chunk = _int(_section(raw["mask"], where + ".mask", ("size",)), "size", where + ".mask")
        return ChunkedAttentionConfig(_int(raw, "heads", where), _int(raw, "kv_heads", where), dim, _int(raw, "vdim", where),
                                      _num(raw, "scale", where), rot, chunk)

    def to_json(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                "mask": None if self.chunk is None else {"size": self.chunk},
                "rot": None if self.rot is None else self.rot.to_json(), "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class RetentionConfig:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[Rotation]

    @staticmethod
    def from_dict(raw, where: str) -> "RetentionConfig":
        _section(raw, where, ("heads", "dim", "vdim", "decay"), ("rot",))
        heads, dim = _int(raw, "heads", where), _int(raw, "dim", where)
        rot = None if raw.get("rot") is None else Rotation.from_dict(raw["rot"], where + ".rot", dim)
        return RetentionConfig(heads, dim, _int(raw, "vdim", where), _decays(raw, where, heads), rot)

    def to_json(self) -> dict:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads,
                "rot": None if self.rot is None else self.rot.to_json(), "vdim": self.vdim}


@dataclass(frozen=True)
class ParallelConfig:
    left: ChunkedAttentionConfig
    right: RetentionConfig
    left_scale: float
    right_scale: float

    @staticmethod
    def from_dict(raw, where: str) -> "ParallelConfig":
        _section(raw, where, ("left", "right", "left_scale", "right_scale"))
        return ParallelConfig(ChunkedAttentionConfig.from_dict(raw["left"], where + ".left"),
                              RetentionConfig.from_dict(raw["right"], where + ".right"),
                              _num(raw, "left_scale", where), _num(raw, "right_scale", where))

    def to_json(self) -> dict:
        return {"left": self.left.to_json(), "left_scale": self.left_scale, "right": self.right.to_json(),
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class DenseConfig:
    ff: int

    @staticmethod
    def from_dict(raw, where: str) -> "DenseConfig":
        _section(raw, where, ("kind", "ff"))
        if raw["kind"] != DENSE:
            raise ConfigError(f"{where}.kind = {raw['kind']!r}: Fazezen's feed-forward is {DENSE!r}", key=where + ".kind")
        return DenseConfig(_int(raw, "ff", where))

    def to_json(self) -> dict:
        return {"ff": self.ff, "kind": DENSE}


_MIXERS = {LIGHTNING: LightningConfig, PARALLEL: ParallelConfig}


@dataclass(frozen=True)
class FazezenLayer:
    type: str
    mixer: object                    # LightningConfig | ParallelConfig
    mlp: Optional[DenseConfig]

    def __post_init__(self):
        if not isinstance(self.mixer, _MIXERS.get(self.type, ())):
            raise ConfigError(f"a layer of type {self.type!r} needs that type's mixer", known=sorted(_MIXERS))


@dataclass(frozen=True)
class FazezenConfig:
    vocab: int
    width: int
    layers: Tuple[FazezenLayer, ...]
    norm_eps: float = 1e-5
    # not a key of the file (and no part of what makes two configurations equal): what the rotation tables are made for
    max_position: int = field(default=DEFAULT_MAX_POSITION, compare=False)

    def __post_init__(self):
        if self.vocab < 1 or self.width < 1:
            raise ConfigError("vocab and width must be positive", vocab=self.vocab, width=self.width)
        if not self.layers:
            raise ConfigError("a model has at least one layer")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be a positive number", eps=self.norm_eps)

    @staticmethod
    def from_dict(raw: dict) -> "FazezenConfig":
        _section(raw, "config.json", ("architecture", "vocab", "width", "layers", "norm"), ("architectures",))
        if raw["architecture"] != ARCHITECTURE:
            raise ConfigError(f"architecture is {raw['architecture']!r}, this reader takes {ARCHITECTURE!r}")
        norm = _section(raw["norm"], "norm", ("eps",))
        if not isinstance(raw["layers"], list):
            raise ConfigError("layers must be a list", key="layers")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _section(entry, where, ("type", "mixer"), ("mlp",))
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}.type = {entry['type']!r}: Fazezen has {sorted(_MIXERS)}", key=where + ".type")
            mixer = _MIXERS[entry["type"]].from_dict(entry["mixer"], where + ".mixer")
            mlp = None if entry.get("mlp") is None else DenseConfig.from_dict(entry["mlp"], where + ".mlp")
            layers.append(FazezenLayer(entry["type"], mixer, mlp))
        return FazezenConfig(vocab=_int(raw, "vocab", "config.json"), width=_int(raw, "width", "config.json"),
                             layers=tuple(layers), norm_eps=_num(norm, "eps", "norm", True))

    def to_json(self) -> dict:
        return {"architecture": ARCHITECTURE,
                "layers": [{"mixer": L.mixer.to_json(), "mlp": None if L.mlp is None else L.mlp.to_json(), "type": L.type}
                           for L in self.layers],
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}
