"""Typed configuration of Togalorn, read from the design's own config.json keys.

A Togalorn file names its design under ``architecture`` (one string), gives ``vocab``, ``width``, ``embedding.scale``,
``norm.eps`` and ``norm.groups`` (the stream's norms divide a row in that many equal parts), ``canon.taps`` (the taps
of the convolution over time that every layer lays on its mixer's input; null or absent: no such convolution), a list
``layers`` and, optionally, ``loop`` (``start``, ``stop``, ``times``: the layers ``start .. stop - 1`` run ``times``
times in a row with the same weights, each pass with a cache of its own).  Each entry of ``layers`` has a ``type`` (the
kind of its mixer), the mixer's sizes and constants under ``mixer`` and its feed-forward under ``mlp`` (null: none).

    mixer  (type "latent_attention"): heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot {base, dims}
    mixer  (type "mamba2"):           heads, vdim, state, groups, norm_groups, conv
    mlp    (kind "moe"):              router {experts, top, identity}, expert {ff, limit}, shared {ff, limit} | null

As with the other architectures an unknown key is an error that names the key (a key this reader does not know would
be a mechanism it does not compute); a key whose value is null counts as left out.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple

from ..errors import ConfigError
from .fazezen import DEFAULT_MAX_POSITION, _int, _num

ARCHITECTURE = "Togalorn"
LATENT = "latent_attention"
MAMBA2 = "mamba2"
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
            raise ConfigError(f"unsupported key {k!r} in {where} (no Togalorn feature declares it)", key=f"{where}.{k}")
    for k in required:
        if raw.get(k) is None:
            raise ConfigError(f"{where} lacks the required key {k!r}", key=f"{where}.{k}")
    return raw


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int              # unrotated query/key features of a head
    rot_dim: int          # rotated ones
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float

    @staticmethod
    def from_dict(raw, where: str) -> "LatentMixerConfig":
        _section(raw, where, ("heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale"), ("rot",))
        rot_dim = _int(raw, "rot_dim", where, least=0)
        base = 10000.0
        if rot_dim:
            if raw.get("rot") is None:
                raise ConfigError(f"{where} has rotated features and lacks 'rot'", key=where + ".rot")
            rot = _section(raw["rot"], where + ".rot", ("base", "dims"))
            if _int(rot, "dims", where + ".rot", least=0) != rot_dim:
                raise ConfigError(f"{where}.rot.dims must equal rot_dim ({rot_dim}): the rotated part is rotated whole",
                                  key=where + ".rot.dims")
            base = _num(rot, "base", where + ".rot", positive=True)
        if rot_dim % 2:
            raise ConfigError(f"{where}.rot_dim must be even", key=where + ".rot_dim")
        dim = _int(raw, "dim", where, least=0)
        if dim + rot_dim < 1:
            raise ConfigError(f"{where}: a head needs query/key features", key=where + ".dim")
        return LatentMixerConfig(_int(raw, "heads", where), dim, rot_dim, _int(raw, "vdim", where),
                                 _int(raw, "q_rank", where), _int(raw, "kv_rank", where), _num(raw, "scale", where), base)

    def to_json(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "kv_rank": self.kv_rank, "q_rank": self.q_rank,
                "rot": {"base": self.rot_base, "dims": self.rot_dim} if self.rot_dim else None,
                "rot_dim": self.rot_dim, "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class Mamba2MixerConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int             # taps of the convolution over x, B and C

    def __post_init__(self):
        if self.heads % self.groups:
            raise ConfigError("heads must be a multiple of groups", heads=self.heads, groups=self.groups)
        if (self.heads * self.vdim) % self.norm_groups:
            raise ConfigError("heads * vdim must be a multiple of norm_groups", inner=self.heads * self.vdim,
                              norm_groups=self.norm_groups)

    @staticmethod
    def from_dict(raw, where: str) -> "Mamba2MixerConfig":
        _section(raw, where, ("heads", "vdim", "state", "groups", "norm_groups", "conv"))
        return Mamba2MixerConfig(*(_int(raw, k, where) for k in ("heads", "vdim", "state", "groups", "norm_groups", "conv")))

    def to_json(self) -> dict:
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


@dataclass(frozen=True)
class ExpertConfig:
    ff: int
    limit: float

    @staticmethod
    def from_dict(raw, where: str) -> "ExpertConfig":
        _section(raw, where, ("ff", "limit"))
        return ExpertConfig(_int(raw, "ff", where), _num(raw, "limit", where, positive=True))

    def to_json(self) -> dict:
        return {"ff": self.ff, "limit": self.limit}


@dataclass(frozen=True)
class MoEConfig:
    experts: int          # experts that have weights
    top: int
    identity: int         # further router outputs whose expert gives back its input
    expert: Optional[ExpertConfig]
    shared: Optional[ExpertConfig]

    def __post_init__(self):
        if self.top > self.experts + self.identity:
            raise ConfigError("top exceeds the router's outputs", top=self.top, outputs=self.experts + self.identity)
        if self.experts and self.expert is None:
            raise ConfigError("experts need their sizes under 'expert'")

    @staticmethod
    def from_dict(raw, where: str) -> "MoEConfig":
        _section(raw, where, ("kind", "router"), ("expert", "shared"))
        if raw["kind"] != MOE:
            raise ConfigError(f"{where}.kind = {raw['kind']!r}: Togalorn's feed-forward is {MOE!r}", key=where + ".kind")
        r = _section(raw["router"], where + ".router", ("experts", "top"), ("identity",))
        identity = 0 if r.get("identity") is None else _int(r, "identity", where + ".router", least=0)
        expert = None if raw.get("expert") is None else ExpertConfig.from_dict(raw["expert"], where + ".expert")
        shared = None if raw.get("shared") is None else ExpertConfig.from_dict(raw["shared"], where + ".shared")
        return MoEConfig(_int(r, "experts", where + ".router", least=0), _int(r, "top", where + ".router"), identity,
                         expert, shared)

    def to_json(self) -> dict:
        return {"expert": None if self.expert is None else self.expert.to_json(), "kind": MOE,
                "router": {"experts": self.experts, "identity": self.identity, "top": self.top},
                "shared": None if self.shared is None else self.shared.to_json()}


_MIXERS = {LATENT: LatentMixerConfig, MAMBA2: Mamba2MixerConfig}


@dataclass(frozen=True)
class TogalornLayer:
    type: str
    mixer: object                    # LatentMixerConfig | Mamba2MixerConfig
    mlp: Optional[MoEConfig]

    def __post_init__(self):
        if not isinstance(self.mixer, _MIXERS.get(self.type, ())):
            raise ConfigError(f"a layer of type {self.type!r} needs that type's mixer", known=sorted(_MIXERS))


@dataclass(frozen=True)
class LoopConfig:
    start: int
    stop: int
    times: int

    def to_json(self) -> dict:
        return {"start": self.start, "stop": self.stop, "times": self.times}


@dataclass(frozen=True)
class TogalornConfig:
    vocab: int
    width: int
    layers: Tuple[TogalornLayer, ...]
    norm_eps: float = 1e-6
    norm_groups: int = 1
    embedding_scale: float = 1.0
    canon_taps: Optional[int] = None
    loop: Optional[LoopConfig] = None
    # not a key of the file (and no part of what makes two configurations equal): what the rotation tables are made for
    max_position: int = field(default=DEFAULT_MAX_POSITION, compare=False)

    def __post_init__(self):
        if self.vocab < 1 or self.width < 1:
            raise ConfigError("vocab and width must be positive", vocab=self.vocab, width=self.width)
        if not self.layers:
            raise ConfigError("a model has at least one layer")
        if not self.norm_eps > 0:
            raise ConfigError("norm.eps must be a positive number", eps=self.norm_eps)
        if self.norm_groups < 1 or self.width % self.norm_groups:
            raise ConfigError("width must be a multiple of norm.groups", width=self.width, groups=self.norm_groups)
        if self.loop is not None:
            lp = self.loop
            if not (0 <= lp.start < lp.stop <= len(self.layers)) or lp.times < 1:
                raise ConfigError("loop must name a run of layers and a positive number of passes", start=lp.start,
                                  stop=lp.stop, times=lp.times, layers=len(self.layers))

    @staticmethod
    def from_dict(raw: dict) -> "TogalornConfig":
        top = "config.json"
        _section(raw, top, ("architecture", "vocab", "width", "layers", "norm"),
                 ("architectures", "embedding", "canon", "loop"))
        if raw["architecture"] != ARCHITECTURE:
            raise ConfigError(f"architecture is {raw['architecture']!r}, this reader takes {ARCHITECTURE!r}")
        norm = _section(raw["norm"], "norm", ("eps",), ("groups",))
        scale = 1.0
        if raw.get("embedding") is not None:
            emb = _section(raw["embedding"], "embedding", (), ("scale",))
            scale = 1.0 if emb.get("scale") is None else _num(emb, "scale", "embedding")
        taps = None
        if raw.get("canon") is not None:
            canon = _section(raw["canon"], "canon", (), ("taps",))
            taps = None if canon.get("taps") is None else _int(canon, "taps", "canon")
        loop = None
        if raw.get("loop") is not None:
            lp = _section(raw["loop"], "loop", ("start", "stop", "times"))
            loop = LoopConfig(_int(lp, "start", "loop", least=0), _int(lp, "stop", "loop"), _int(lp, "times", "loop"))
        if not isinstance(raw["layers"], list):
            raise ConfigError("layers must be a list", key="layers")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            _section(entry, where, ("type", "mixer"), ("mlp",))
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}.type = {entry['type']!r}: Togalorn has {sorted(_MIXERS)}", key=where + ".type")
            mixer = _MIXERS[entry["type"]].from_dict(entry["mixer"], where + ".mixer")
            mlp = None if entry.get("mlp") is None else MoEConfig.from_dict(entry["mlp"], where + ".mlp")
            layers.append(TogalornLayer(entry["type"], mixer, mlp))
        return TogalornConfig(vocab=_int(raw, "vocab", top), width=_int(raw, "width", top), layers=tuple(layers),
                              norm_eps=_num(norm, "eps", "norm", True),
                              norm_groups=1 if norm.get("groups") is None else _int(norm, "groups", "norm"),
                              embedding_scale=scale, canon_taps=taps, loop=loop)

    def to_json(self) -> dict:
        return {"architecture": ARCHITECTURE,
                "canon": None if self.canon_taps is None else {"taps": self.canon_taps},
                "embedding": {"scale": self.embedding_scale},
                "layers": [{"mixer": L.mixer.to_json(), "mlp": None if L.mlp is None else L.mlp.to_json(), "type": L.type}
                           for L in self.layers],
                "loop": None if self.loop is None else self.loop.to_json(),
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "vocab": self.vocab, "width": self.width}
