"""Typed configuration of Makuzen, read from the design's own config.json keys.

A Makuzen file names its design under ``architecture`` (one string), gives ``vocab``, ``width``,
``embedding.scale``, ``norm.eps``, ``residual_mult`` and a list ``layers``; each entry has a ``type`` (the kind
of its mixer), the mixer's sizes and constants under ``mixer`` and its feed-forward under ``mlp`` (null: none).
Every size and constant is read from there; a layer may differ from its neighbours in all of them.

    mixer  (type "latent_attention"): heads, dim, rot_dim, vdim, q_rank, kv_rank, scale,
           rot {base, dims, scaling {factor, original, fast, slow} | null}, mask {size} | null
    mlp    (kind "moe"): expert {ff}, router {experts, top}, shared {ff} | null

As with the other architectures an unknown key is an error that names the key (a key this reader does not know
would be a mechanism it does not compute); a key whose value is null counts as left out.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..errors import ConfigError

ARCHITECTURE = "Makuzen"
LATENT_ATTENTION = "latent_attention"
MOE = "moe"

# the most positions a request may hold when nothing else bounds it: the file has no such key, the rotation tables
# are made for this many, the engine's own context length is what limits a request
DEFAULT_MAX_POSITION = 1 << 17

# keys that describe provenance, read by nobody
_IGNORED = frozenset({"seed", "name", "description", "comment", "dtype", "torch_dtype"})


def _section(raw, where: str, required, optional=()):
    """``raw`` as a dictionary holding exactly the ``required`` keys and any of the ``optional`` ones."""
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object, found {raw!r}", key=where)
    known = set(required) | set(optional) | _IGNORED
    for k, v in raw.items():
        if k not in known and v is not None:
            raise ConfigError(f"unsupported key {k!r} in {where} (no Makuzen feature declares it)", key=f"{where}.{k}")
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


@dataclass(frozen=True)
class YarnScaling:
    factor: float
    original: float      # the length the frequencies were chosen for
    fast: float          # pairs that turn more often than this over the original length keep their frequency
    slow: float          # pairs that turn less often than this are slowed by ``factor``

    def to_json(self) -> dict:
        return {"factor": self.factor, "fast": self.fast, "original": self.original, "slow": self.slow}


@dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int             # unrotated query/key features of a head
    rot_dim: int         # rotated ones
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    scaling: Optional[YarnScaling]
    window: Optional[int]

    def __post_init__(self):
        if self.rot_dim % 2:
            raise ConfigError("rot_dim must be even: features are rotated in pairs", rot_dim=self.rot_dim)

    @staticmethod
    def from_dict(raw, where: str) -> "LatentAttentionConfig":
        _section(raw, where, ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale"), ("rot", "mask"))
        rot_dim = _int(raw, "rot_dim", where, least=0)
        base, scaling = 10000.0, None
        if raw.get("rot") is not None:
            rot = _section(raw["rot"], where + ".rot", ("base",), ("dims", "scaling"))
            base = _num(rot, "base", where + ".rot", positive=True)
            if rot.get("dims") is not None and _int(rot, "dims", where + ".rot", least=0) != rot_dim:
                raise ConfigError(f"{where}.rot.dims must equal rot_dim: the rotated part of a head is rotated whole",
                                  dims=rot["dims"], rot_dim=rot_dim)
            if rot.get("scaling") is not None:
                s = _section(rot["scaling"], where + ".rot.scaling", ("factor", "original", "fast", "slow"))
                w = where + ".rot.scaling"
                scaling = YarnScaling(_num(s, "factor", w, True), _num(s, "original", w, True), _num(s, "fast", w, True),
                                      _num(s, "slow", w, True))
        elif rot_dim:
            raise ConfigError(f"{where} has rotated features but no 'rot' entry", key=where + ".rot")
        window = None
        if raw.get("mask") is not None:
            window = _int(_section(raw["mask"], where + ".mask", ("size",)), "size", where + ".mask")
        return LatentAttentionConfig(
            heads=_int(raw, "heads", where), dim=_int(raw, "dim", where, least=0), rot_dim=rot_dim,
            vdim=_int(raw, "vdim", where), q_rank=_int(raw, "q_rank", where), kv_rank=_int(raw, "kv_rank", where),
            scale=_num(raw, "scale", where), rot_base=base, scaling=scaling, window=window)

    def to_json(self) -> dict:
        out = {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank,
               "mask": None if self.window is None else {"size": self.window}, "q_rank": self.q_rank,
               "rot": {"base": self.rot_base, "dims": self.rot_dim,
                       "scaling": None if self.scaling is None else self.scaling.to_json()},
               "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}
        return out


@dataclass(frozen=True)
class TableMoEConfig:
    experts: int
    top: int
    ff: int                          # an expert's inner width
    shared_ff: Optional[int]         # the shared expert's (None: no shared expert)

    def __post_init__(self):
        if not 1 <= self.top <= self.experts:
            raise ConfigError("a token uses between one and all of the experts", top=self.top, experts=self.experts)

    @staticmethod
    def from_dict(raw, where: str) -> "TableMoEConfig":
        _section(raw, where, ("kind", "expert", "router"), ("shared",))
        if raw["kind"] != MOE:
            raise ConfigError(f"{where}.kind = {raw['kind']!r}: Makuzen's feed-forward is {MOE!r}", key=where + ".kind")
        ex = _section(raw["expert"], where + ".expert", ("ff",))
        ro = _section(raw["router"], where + ".router", ("experts", "top"))
        shared = None
        if raw.get("shared") is not None:
            shared = _int(_section(raw["shared"], where + ".shared", ("ff",)), "ff", where + ".shared")
        return TableMoEConfig(experts=_int(ro, "experts", where + ".router"), top=_int(ro, "top", where + ".router"),
                              ff=_int(ex, "ff", where + ".expert"), shared_ff=shared)

    def to_json(self) -> dict:
        return {"expert": {"ff": self.ff}, "kind": MOE, "router": {"experts": self.experts, "top": self.top},
                "shared": None if self.shared_ff is None else {"ff": self.shared_ff}}


@dataclass(frozen=True)
class MakuzenLayer:
    mixer: LatentAttentionConfig
    mlp: Optional[TableMoEConfig]
    type: str = LATENT_ATTENTION


@dataclass(frozen=True)
class MakuzenConfig:
    vocab: int
    width: int
    layers: Tuple[MakuzenLayer, ...]
    embedding_scale: float = 1.0
    norm_eps: float = 1e-5
    residual_mult: float = 1.0
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
    def from_dict(raw: dict) -> "MakuzenConfig":
        _section(raw, "config.json", ("architecture", "vocab", "width", "layers", "norm"),
                 ("embedding", "residual_mult", "architectures"))
        if raw["architecture"] != ARCHITECTURE:
            raise ConfigError(f"architecture is {raw['architecture']!r}, this reader takes {ARCHITECTURE!r}")
        norm = _section(raw["norm"], "norm", ("eps",))
        scale = 1.0
        if raw.get("embedding") is not None:
            scale = _num(_section(raw["embedding"], "embedding", ("scale",)), "scale", "embedding")
        if not isinstance(raw["layers"], list):
            raise ConfigError("layers must be a list", key="layers")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _section(entry, where, ("type", "mixer"), ("mlp",))
            if entry["type"] != LATENT_ATTENTION:
                raise ConfigError(f"{where}.type = {entry['type']!r}: Makuzen has {LATENT_ATTENTION!r}", key=where + ".type")
            mlp = None if entry.get("mlp") is None else TableMoEConfig.from_dict(entry["mlp"], where + ".mlp")
            layers.append(MakuzenLayer(LatentAttentionConfig.from_dict(entry["mixer"], where + ".mixer"), mlp))
        return MakuzenConfig(vocab=_int(raw, "vocab", "config.json"), width=_int(raw, "width", "config.json"),
                             layers=tuple(layers), embedding_scale=scale, norm_eps=_num(norm, "eps", "norm", True),
                             residual_mult=1.0 if raw.get("residual_mult") is None else _num(raw, "residual_mult", "config.json"))

    def to_json(self) -> dict:
        return {"architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
                "layers": [{"mixer": L.mixer.to_json(), "mlp": None if L.mlp is None else L.mlp.to_json(), "type": L.type}
                           for L in self.layers],
                "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult, "vocab": self.vocab,
                "width": self.width}
