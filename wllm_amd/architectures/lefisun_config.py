"""Typed configuration of Lefisun, read from its config.json.

The file is nested: `architecture`, `vocab`, `width`, `embedding.scale`, `norm.eps` and `layers`, a list
whose entries carry `type` (which mixer: `parallel` or `retention`), the mixer's sizes and constants
under `mixer`, and the feed-forward under `mlp` (`kind` = `moe` with `expert.ff` and `router`), or null
for a layer without one.  A `parallel` mixer is two mixers side by side, `left` (attention inside
chunks: `heads`, `kv_heads`, `dim`, `vdim`, `scale`, `mask.size`, `rot`) and `right` (a matrix memory
with exponential gates: `heads`, `dim`, `vdim`, `gate_cap`), with `left_scale` and `right_scale`; a
`retention` mixer has `heads`, `dim`, `vdim`, `rot` and one `decay` a head.  `rot` is `dims`, `base`
and optionally `scaling.factor`.  Every layer carries its own sizes, so two layers of one model may
differ in all of them, and the order of the mixers is the file's.  A key the design needs and the
file lacks is an error; a key this code does not read is named in a warning (`UnknownConfigKey`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from wllm_amd.architectures.tasosun_config import _number, _positive_int, _section
from wllm_amd.config.registry import ConfigError

MIXER_TYPES = ("parallel", "retention")


@dataclass(frozen=True)
class LefisunRotation:
    dims: int                       # the first `dims` elements of a head turn
    base: float
    scaling_factor: float = 1.0     # linear scaling: frequencies divided by it

    @classmethod
    def from_dict(cls, where: str, raw, head_dim: int) -> "LefisunRotation":
        raw = _section(where, raw, ("dims", "base"), ("scaling",))
        dims = _positive_int(f"{where}.dims", raw["dims"])
        if dims % 2 or dims > head_dim:
            raise ConfigError(f"{where}.dims ({dims}) must be even and at most the head's size ({head_dim})")
        factor = 1.0
        if raw.get("scaling") is not None:
            factor = _number(f"{where}.scaling.factor",
                             _section(f"{where}.scaling", raw["scaling"], ("factor",))["factor"])
        return cls(dims, _number(f"{where}.base", raw["base"]), factor)

    def to_dict(self) -> dict:
        out = {"dims": self.dims, "base": self.base}
        if self.scaling_factor != 1.0:
            out["scaling"] = {"factor": self.scaling_factor}
        return out


@dataclass(frozen=True)
class LefisunAttention:
    heads: int
    kv_heads: int
    dim: int                        # query/key size of a head
    vdim: int                       # value size of a head
    scale: float
    chunk: Optional[int]            # mask.size; None: every earlier position is seen
    rotation: Optional[LefisunRotation]

    @classmethod
    def from_dict(cls, where: str, raw) -> "LefisunAttention":
        raw = _section(where, raw, ("heads", "kv_heads", "dim", "vdim", "scale"), ("mask", "rot"))
        heads, kv_heads = _positive_int(f"{where}.heads", raw["heads"]), _positive_int(f"{where}.kv_heads", raw["kv_heads"])
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        dim = _positive_int(f"{where}.dim", raw["dim"])
        chunk = None
        if raw.get("mask") is not None:
            chunk = _positive_int(f"{where}.mask.size", _section(f"{where}.mask", raw["mask"], ("size",))["size"])
        rotation = None
        if raw.get("rot") is not None:
            rotation = LefisunRotation.from_dict(f"{where}.rot", raw["rot"], dim)
        return cls(heads, kv_heads, dim, _positive_int(f"{where}.vdim", raw["vdim"]),
                   _number(f"{where}.scale", raw["scale"]), chunk, rotation)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.chunk is not None:
            out["mask"] = {"size": self.chunk}
        if self.rotation is not None:
            out["rot"] = self.rotation.to_dict()
        return out


@dataclass(frozen=True)
class LefisunMemory:
    heads: int
    dim: int
    vdim: int
    gate_cap: float

    @classmethod
    def from_dict(cls, where: str, raw) -> "LefisunMemory":
        raw = _section(where, raw, ("heads", "dim", "vdim", "gate_cap"))
        return cls(*[_positive_int(f"{where}.{k}", raw[k]) for k in ("heads", "dim", "vdim")],
                   _number(f"{where}.gate_cap", raw["gate_cap"]))

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}


@dataclass(frozen=True)
class LefisunParallel:
    left: LefisunAttention
    right: LefisunMemory
    left_scale: float
    right_scale: float

    @classmethod
    def from_dict(cls, where: str, raw) -> "LefisunParallel":
        raw = _section(where, raw, ("left", "right", "left_scale", "right_scale"))
        scales = []
        for k in ("left_scale", "right_scale"):
            v = raw[k]
            if isinstance(v, bool) or not isinstance(v, (int, float)):
                raise ConfigError(f"{where}.{k} must be a number, got {v!r}")
            scales.append(float(v))
        return cls(LefisunAttention.from_dict(f"{where}.left", raw["left"]),
                   LefisunMemory.from_dict(f"{where}.right", raw["right"]), *scales)

    def to_dict(self) -> dict:
        return {"left": self.left.to_dict(), "right": self.right.to_dict(), "left_scale": self.left_scale,
                "right_scale": self.right_scale}


@dataclass(frozen=True)
class LefisunRetention:
    heads: int
    dim: int
    vdim: int
    decay: tuple                    # one a head
    rotation: Optional[LefisunRotation]

    @classmethod
    def from_dict(cls, where: str, raw) -> "LefisunRetention":
        raw = _section(where, raw, ("heads", "dim", "vdim", "decay"), ("rot",))
        heads, dim = _positive_int(f"{where}.heads", raw["heads"]), _positive_int(f"{where}.dim", raw["dim"])
        decay = raw["decay"]
        if not isinstance(decay, list) or len(decay) != heads:
            raise ConfigError(f"{where}.decay must be a list of one number a head ({heads}), got {decay!r}")
        decay = tuple(_number(f"{where}.decay[{i}]", d, positive=False) for i, d in enumerate(decay))
        rotation = None
        if raw.get("rot") is not None:
            rotation = LefisunRotation.from_dict(f"{where}.rot", raw["rot"], dim)
        return cls(heads, dim, _positive_int(f"{where}.vdim", raw["vdim"]), decay, rotation)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay)}
        if self.rotation is not None:
            out["rot"] = self.rotation.to_dict()
        return out


@dataclass(frozen=True)
class LefisunExperts:
    ff: int
    experts: int
    top: int
    groups: int
    keep: int

    @classmethod
    def from_dict(cls, where: str, raw) -> "LefisunExperts":
        raw = _section(where, raw, ("kind", "expert", "router"))
        if raw["kind"] != "moe":
            raise ConfigError(f"{where}.kind {raw['kind']!r}: this design's feed-forwards are: moe")
        ff = _positive_int(f"{where}.expert.ff", _section(f"{where}.expert", raw["expert"], ("ff",))["ff"])
        router = _section(f"{where}.router", raw["router"], ("experts", "top"), ("groups",))
        experts, top = _positive_int(f"{where}.router.experts", router["experts"]), _positive_int(f"{where}.router.top", router["top"])
        groups = keep = 1
        if router.get("groups") is not None:
            g = _section(f"{where}.router.groups", router["groups"], ("count", "keep"))
            groups, keep = _positive_int(f"{where}.router.groups.count", g["count"]), _positive_int(f"{where}.router.groups.keep", g["keep"])
        if experts % groups or keep > groups:
            raise ConfigError(f"{where}.router: groups.count ({groups}) must divide experts ({experts}) and groups.keep "
                              f"({keep}) be at most groups.count")
        if top > keep * (experts // groups):
            raise ConfigError(f"{where}.router.top ({top}) is more than the experts of the kept groups "
                              f"({keep * (experts // groups)})")
        return cls(ff, experts, top, groups, keep)

    def to_dict(self) -> dict:
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.keep}}}


_MIXERS = {"parallel": LefisunParallel, "retention": LefisunRetention}


@dataclass(frozen=True)
class LefisunLayer:
    type: str
    mixer: object
    mlp: Optional[LefisunExperts]


@dataclass(frozen=True)
class LefisunConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: tuple
    raw: Optional[dict] = None

    @classmethod
    def from_dict(cls, raw: dict) -> "LefisunConfig":
        raw = _section("config.json", raw, ("vocab", "width", "norm", "layers", "embedding"), ("architecture", "architectures"))
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config.json: layers must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            entry = _section(where, entry, ("type", "mixer"), ("mlp",))
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}.type {entry['type']!r}: this design's mixers are: {', '.join(MIXER_TYPES)}")
            mixer = _MIXERS[entry["type"]].from_dict(f"{where}.mixer", entry["mixer"])
            mlp = LefisunExperts.from_dict(f"{where}.mlp", entry["mlp"]) if entry.get("mlp") is not None else None
            layers.append(LefisunLayer(entry["type"], mixer, mlp))
        scale = _section("embedding", raw["embedding"], ("scale",))["scale"]
        if isinstance(scale, bool) or not isinstance(scale, (int, float)):
            raise ConfigError(f"embedding.scale must be a number, got {scale!r}")
        return cls(vocab=_positive_int("vocab", raw["vocab"]), width=_positive_int("width", raw["width"]),
                   embedding_scale=float(scale),
                   norm_eps=_number("norm.eps", _section("norm", raw["norm"], ("eps",))["eps"], positive=False),
                   layers=tuple(layers), raw=raw)

    def to_dict(self) -> dict:
        """The config.json of this configuration."""
        if self.raw is not None:
            return dict(self.raw)
        return {"architecture": "Lefisun", "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                "layers": [{"type": layer.type, "mixer": layer.mixer.to_dict(),
                            "mlp": None if layer.mlp is None else layer.mlp.to_dict()} for layer in self.layers]}
