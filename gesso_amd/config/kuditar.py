"""Typed configuration of Kuditar, read from the design's own config.json keys.

A Kuditar file names its design under ``architecture`` (one string), gives ``vocab``, ``width``, ``embedding.scale``,
``norm.eps`` and a list ``layers``.  Each entry has a ``type`` (the kind of its mixer), the mixer's sizes and constants
under ``mixer`` and its feed-forward under ``mlp`` (null: none).

    mixer (type "attention"):   heads, kv_heads, dim, vdim, scale, softcap?, rot {base, dims, scaling {factor}?}?, v_mix?
    mixer (type "parallel"):    left  {heads, kv_heads, dim, vdim, scale, softcap?, rot {base, dims, scaling?}?,
                                       mask {size, keep_first?}?}
                                right {heads, kv_heads, dim, vdim, conv}
    mixer (type "parallel_2"):  left  {heads, kv_heads, dim, vdim, scale, mask {size}?}
                                right {heads, dim, vdim, tau, rank?}
    mlp (kind "dense"):         ff, limit
    mlp (kind "moe"):           router {experts, top, scale}, expert {ff, limit}

One size has no key of its own in files that other tools write: the width ``rank`` of the bottleneck through which a
``parallel_2`` layer's decays are made is the row count of the stored tensor ``l<i>.mix.right.a1``; :func:`complete`
reads it from there before the keys are parsed.  Files written from here carry it as ``rank``.

As with the other architectures an unknown key is an error that names the key (a key this reader does not know would
be a mechanism it does not compute); a key whose value is null counts as left out.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..errors import ConfigError
from .fazezen import DEFAULT_MAX_POSITION, _int, _num

ARCHITECTURE = "Kuditar"
ATTENTION = "attention"
PARALLEL = "parallel"
PARALLEL_2 = "parallel_2"
DENSE = "dense"
MOE = "moe"

# keys that describe provenance, read by nobody
_IGNORED = frozenset({"seed", "name", "description", "comment", "dtype", "torch_dtype"})


def _section(raw, where: str, required, optional=()):
    """``raw`` as a dictionary holding exactly the ``required`` keys and any of the ``optional`` ones."""
    if not isinstance(raw, dict):
        raise ConfigError(f"{where} must be an object, found {raw!r}", key=where)
    known = set(required) | set(optional) | _IGNORED
    for k, v in raw.items():
        if k not in known and v is not None:
            raise ConfigError(f"unsupported key {k!r} in {where} (no Kuditar feature declares it)", key=f"{where}.{k}")
    for k in required:
        if raw.get(k) is None:
            raise ConfigError(f"{where} lacks the required key {k!r}", key=f"{where}.{k}")
    return raw


@dataclass(frozen=True)
class Turn:
    """Rotary positions over the first ``dims`` features of a head; every frequency is divided by ``factor``."""

    base: float
    dims: int
    factor: float = 1.0

    @staticmethod
    def from_dict(raw, where: str, dim: int) -> Optional["Turn"]:
        if raw is None:
            return None
        _section(raw, where, ("base", "dims"), ("scaling",))
        dims = _int(raw, "dims", where, least=0)
        if dims == 0:
            return None
        if dims % 2 or dims > dim:
            raise ConfigError(f"{where}.dims must be even and at most the head's {dim} features", key=where + ".dims")
        factor = 1.0
        if raw.get("scaling") is not None:
            sc = _section(raw["scaling"], where + ".scaling", (), ("factor",))
            factor = 1.0 if sc.get("factor") is None else _num(sc, "factor", where + ".scaling", positive=True)
        return Turn(_num(raw, "base", where, positive=True), dims, factor)

    def to_json(self) -> dict:
        return {"base": self.base, "dims": self.dims, "scaling": None if self.factor == 1.0 else {"factor": self.factor}}


@dataclass(frozen=True)
class SoftmaxHeads:
    """The sizes and constants that every softmax attention of the design has."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: Optional[float] = None
    rot: Optional[Turn] = None

    def __post_init__(self):
        if self.heads % self.kv_heads:
            raise ConfigError("heads must be a multiple of kv_heads", heads=self.heads, kv_heads=self.kv_heads)

    @staticmethod
    def read(raw, where: str):
        """The common fields of ``raw`` as keyword arguments."""
        dim = _int(raw, "dim", where)
        return dict(heads=_int(raw, "heads", where), kv_heads=_int(raw, "kv_heads", where), dim=dim,
                    vdim=_int(raw, "vdim", where), scale=_num(raw, "scale", where),
                    softcap=None if raw.get("softcap") is None else _num(raw, "softcap", where, positive=True),
                    rot=Turn.from_dict(raw.get("rot"), where + ".rot", dim))

    def common_json(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
                "rot": None if self.rot is None else self.rot.to_json(), "scale": self.scale, "softcap": self.softcap,
                "vdim": self.vdim}


_HEAD_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale")


@dataclass(frozen=True)
class GatedAttentionConfig(SoftmaxHeads):
    v_mix: bool = False

    @staticmethod
    def from_dict(raw, where: str) -> "GatedAttentionConfig":
        _section(raw, where, _HEAD_KEYS, ("softcap", "rot", "v_mix"))
        v_mix = raw.get("v_mix")
        if v_mix is not None and not isinstance(v_mix, bool):
            raise ConfigError(f"{where}.v_mix must be true or false, found {v_mix!r}", key=where + ".v_mix")
        return GatedAttentionConfig(v_mix=bool(v_mix), **SoftmaxHeads.read(raw, where))

    def to_json(self) -> dict:
        return dict(self.common_json(), v_mix=self.v_mix)


@dataclass(frozen=True)
class WindowedAttentionConfig(SoftmaxHeads):
    """Left side of ``parallel``: a window of ``window`` positions (None: all) plus the first ``keep_first``."""

    window: Optional[int] = None
    keep_first: int = 0

    @staticmethod
    def from_dict(raw, where: str) -> "WindowedAttentionConfig":
        _section(raw, where, _HEAD_KEYS, ("softcap", "rot", "mask"))
        window, keep = None, 0
        if raw.get("mask") is not None:
            mask = _section(raw["mask"], where + ".mask", (), ("size", "keep_first"))
            window = None if mask.get("size") is None else _int(mask, "size", where + ".mask")
            keep = 0 if mask.get("keep_first") is None else _int(mask, "keep_first", where + ".mask", least=0)
        return WindowedAttentionConfig(window=window, keep_first=keep, **SoftmaxHeads.read(raw, where))

    def to_json(self) -> dict:
        mask = None if self.window is None else {"keep_first": self.keep_first, "size": self.window}
        return dict(self.common_json(), mask=mask)


@dataclass(frozen=True)
class RunAttentionConfig(SoftmaxHeads):
    """Left side of ``parallel_2``: positions in runs of ``run`` from 0 on (None: one run), no turn, no cap."""

    run: Optional[int] = None

    @staticmethod
    def from_dict(raw, where: str) -> "RunAttentionConfig":
        _section(raw, where, _HEAD_KEYS, ("mask",))
        run = None
        if raw.get("mask") is not None:
            mask = _section(raw["mask"], where + ".mask", (), ("size",))
            run = None if mask.get("size") is None else _int(mask, "size", where + ".mask")
        return RunAttentionConfig(run=run, **SoftmaxHeads.read(raw, where))

    def to_json(self) -> dict:
        out = self.common_json()
        del out["rot"], out["softcap"]
        return dict(out, mask=None if self.run is None else {"size": self.run})


@dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int
    kv_heads: int         # heads of q and k
    dim: int
    vdim: int
    conv: int             # taps of the convolutions over q, k and v

    def __post_init__(self):
        if self.heads % self.kv_heads:
            raise ConfigError("heads must be a multiple of kv_heads", heads=self.heads, kv_heads=self.kv_heads)

    @staticmethod
    def from_dict(raw, where: str) -> "DeltaRuleConfig":
        _section(raw, where, ("heads", "kv_heads", "dim", "vdim", "conv"))
        return DeltaRuleConfig(*(_int(raw, k, where) for k in ("heads", "kv_heads", "dim", "vdim", "conv")))

    def to_json(self) -> dict:
        return {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "vdim": self.vdim}


@dataclass(frozen=True)
class ChannelDecayConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int             # features between the two products that make the decays

    @staticmethod
    def from_dict(raw, where: str) -> "ChannelDecayConfig":
        _section(raw, where, ("heads", "dim", "vdim", "tau"), ("rank",))
        if raw.get("rank") is None:
            raise ConfigError(f"{where}.rank is not given and no stored tensor tells it", key=where + ".rank")
        return ChannelDecayConfig(_int(raw, "heads", where), _int(raw, "dim", where), _int(raw, "vdim", where),
                                  _num(raw, "tau", where, positive=True), _int(raw, "rank", where))

    def to_json(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "rank": self.rank, "tau": self.tau, "vdim": self.vdim}


@dataclass(frozen=True)
class PairConfig:
    left: object
    right: object

    def to_json(self) -> dict:
        return {"left": self.left.to_json(), "right": self.right.to_json()}


def _pair(left_cls, right_cls):
    def read(raw, where: str) -> PairConfig:
        _section(raw, where, ("left", "right"))
        return PairConfig(left_cls.from_dict(raw["left"], where + ".left"), right_cls.from_dict(raw["right"], where + ".right"))
    return read


@dataclass(frozen=True)
class DenseFFConfig:
    ff: int
    limit: float

    def to_json(self) -> dict:
        return {"ff": self.ff, "kind": DENSE, "limit": self.limit}


@dataclass(frozen=True)
class SigmoidMoEConfig:
    experts: int
    top: int
    scale: float          # multiplies the chosen experts' scores
    ff: int
    limit: float

    def __post_init__(self):
        if self.top > self.experts:
            raise ConfigError("top exceeds the number of experts", top=self.top, experts=self.experts)

    def to_json(self) -> dict:
        return {"expert": {"ff": self.ff, "limit": self.limit}, "kind": MOE,
                "router": {"experts": self.experts, "scale": self.scale, "top": self.top}}


def _mlp(raw, where: str):
    if raw is None:
        return None
    if not isinstance(raw, dict) or raw.get("kind") not in (DENSE, MOE):
        raise ConfigError(f"{where}.kind must be {DENSE!r} or {MOE!r}", key=where + ".kind")
    if raw["kind"] == DENSE:
        _section(raw, where, ("kind", "ff", "limit"))
        return DenseFFConfig(_int(raw, "ff", where), _num(raw, "limit", where, positive=True))
    _section(raw, where, ("kind", "router", "expert"))
    r = _section(raw["router"], where + ".router", ("experts", "top"), ("scale",))
    e = _section(raw["expert"], where + ".expert", ("ff", "limit"))
    return SigmoidMoEConfig(_int(r, "experts", where + ".router"), _int(r, "top", where + ".router"),
                            1.0 if r.get("scale") is None else _num(r, "scale", where + ".router"),
                            _int(e, "ff", where + ".expert"), _num(e, "limit", where + ".expert", positive=True))


_MIXERS = {ATTENTION: (GatedAttentionConfig, GatedAttentionConfig.from_dict),
           PARALLEL: (PairConfig, _pair(WindowedAttentionConfig, DeltaRuleConfig)),
           PARALLEL_2: (PairConfig, _pair(RunAttentionConfig, ChannelDecayConfig))}
_SIDES = {PARALLEL: (WindowedAttentionConfig, DeltaRuleConfig), PARALLEL_2: (RunAttentionConfig, ChannelDecayConfig)}


@dataclass(frozen=True)
class KuditarLayer:
    type: str
    mixer: object                    # GatedAttentionConfig | PairConfig
    mlp: Optional[object]            # DenseFFConfig | SigmoidMoEConfig | None

    def __post_init__(self):
        if self.type not in _MIXERS or not isinstance(self.mixer, _MIXERS[self.type][0]):
            raise ConfigError(f"a layer of type {self.type!r} needs that type's mixer", known=sorted(_MIXERS))
        if self.type in _SIDES:
            for side, cls in zip((self.mixer.left, self.mixer.right), _SIDES[self.type]):
                if not isinstance(side, cls):
                    raise ConfigError(f"a {self.type!r} layer pairs {_SIDES[self.type][0].__name__} with "
                                      f"{_SIDES[self.type][1].__name__}")


@dataclass(frozen=True)
class KuditarConfig:
    vocab: int
    width: int
    layers: Tuple[KuditarLayer, ...]
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    # not a key of the file (and no part of what makes two configurations equal): what the rotation tables are made for
    max_position: int = field(default=DEFAULT_MAX_POSITION, compare=False)

    def __post_init__(self):
        if self.vocab < 1 or self.width < 1:
            raise ConfigError("vocab and width must be positive", vocab=self.vocab, width=self.width)
        if not self.layers:
            raise ConfigError("a model has at least one layer")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be a positive number", eps=self.norm_eps)
        shared = {(L.mixer.kv_heads, L.mixer.vdim) for L in self.layers if L.type == ATTENTION and L.mixer.v_mix}
        if len(shared) > 1:
            raise ConfigError("layers that mix their values with the first such layer's need values of its shape",
                              shapes=sorted(shared))

    @staticmethod
    def from_dict(raw: dict) -> "KuditarConfig":
        top = "config.json"
        _section(raw, top, ("architecture", "vocab", "width", "layers", "norm"), ("architectures", "embedding"))
        if raw["architecture"] != ARCHITECTURE:
            raise ConfigError(f"architecture is {raw['architecture']!r}, this reader takes {ARCHITECTURE!r}")
        norm = _section(raw["norm"], "norm", ("eps",))
        scale = 1.0
        if raw.get("embedding") is not None:
            emb = _section(raw["embedding"], "embedding", (), ("scale",))
            scale = 1.0 if emb.get("scale") is None else _num(emb, "scale", "embedding")
        if not isinstance(raw["layers"], list):
            raise ConfigError("layers must be a list", key="layers")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _section(entry, where, ("type", "mixer"), ("mlp",))
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}.type = {entry['type']!r}: Kuditar has {sorted(_MIXERS)}", key=where + ".type")
            mixer = _MIXERS[entry["type"]][1](entry["mixer"], where + ".mixer")
            layers.append(KuditarLayer(entry["type"], mixer, _mlp(entry.get("mlp"), where + ".mlp")))
        return KuditarConfig(vocab=_int(raw, "vocab", top), width=_int(raw, "width", top), layers=tuple(layers),
                             norm_eps=_num(norm, "eps", "norm", True), embedding_scale=scale)

    def to_json(self) -> dict:
        return {"architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
                "layers": [{"mixer": L.mixer.to_json(), "mlp": None if L.mlp is None else L.mlp.to_json(), "type": L.type}
                           for L in self.layers],
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab, "width": self.width}


def complete(raw: dict, shape_of) -> dict:
    """The file's keys with the sizes that only stored tensors tell: a ``parallel_2`` layer's ``right.rank``, the row
    count of ``l<i>.mix.right.a1``, where the file does not give it."""
    layers = raw.get("layers")
    if not isinstance(layers, list):
        return raw
    out = None
    for i, entry in enumerate(layers):
        try:
            right = entry["mixer"]["right"] if entry.get("type") == PARALLEL_2 else None
        except (KeyError, TypeError, AttributeError):
            right = None
        if isinstance(right, dict) and right.get("rank") is None:
            shape = shape_of(f"l{i}.mix.right.a1")
            if shape is not None and len(shape) == 2:
                if out is None:
                    out = copy.deepcopy(raw)
                out["layers"][i]["mixer"]["right"]["rank"] = int(shape[0])
    return raw if out is None else out
