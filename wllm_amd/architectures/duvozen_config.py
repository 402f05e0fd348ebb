"""Typed configuration of Duvozen, read from its config.json.

The file is nested: `architecture`, `vocab`, `width`, `embedding.scale`, `norm.eps`, `canon.taps`, `logit_scale`
and `layers`, a list whose entries carry `type` (which mixer: `hgrn2`, `latent_attention` or `attention`), the
mixer's sizes and constants under `mixer`, and the feed-forward under `mlp` (`kind` = `dense` with `ff`, or
`moe` with `expert.ff`, `router.experts`, `router.top` and optionally `shared.ff`), or null for a layer without
one.  `rot` is `dims`, `base` and optionally `scaling` (`factor`, `original`, `fast`, `slow`).  Every layer
carries its own sizes, so two layers of one model may differ in all of them, and the order of the mixers is the
file's.  A key the design needs and the file lacks is an error; a key this code does not read is named in a
warning (`UnknownConfigKey`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from wllm_amd.architectures.tasosun_config import _number, _positive_int, _section
from wllm_amd.config.registry import ConfigError

MIXER_TYPES = ("hgrn2", "latent_attention", "attention")


def _any_number(where: str, v) -> float:
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{where} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class DuvozenRotation:
    dims: int                       # the first `dims` elements of what turns
    base: float
    scaling: Optional[tuple] = None     # (factor, original, fast, slow): frequencies interpolated pair by pair

    @classmethod
    def from_dict(cls, where: str, raw, most: int) -> "DuvozenRotation":
        raw = _section(where, raw, ("dims", "base"), ("scaling",))
        dims = _positive_int(f"{where}.dims", raw["dims"])
        if dims % 2 or dims > most:
            raise ConfigError(f"{where}.dims ({dims}) must be even and at most {most}")
        scaling = None
        if raw.get("scaling") is not None:
            sc = _section(f"{where}.scaling", raw["scaling"], ("factor", "original", "fast", "slow"))
            scaling = tuple(_number(f"{where}.scaling.{k}", sc[k]) for k in ("factor", "original", "fast", "slow"))
        base = _number(f"{where}.base", raw["base"])
        if scaling is not None and not base > 1.0:
            raise ConfigError(f"{where}.base must be above 1 where the frequencies are interpolated, got {base}")
        return cls(dims, base, scaling)

    def to_dict(self) -> dict:
        out = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.scaling))
        return out


@dataclass(frozen=True)
class DuvozenRecurrence:
    heads: int
    dim: int                        # channels of the forget gate and of the query a head
    vdim: int

    @classmethod
    def from_dict(cls, where: str, raw) -> "DuvozenRecurrence":
        raw = _section(where, raw, ("heads", "dim", "vdim"))
        return cls(*[_positive_int(f"{where}.{k}", raw[k]) for k in ("heads", "dim", "vdim")])

    def to_dict(self) -> dict:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim}


@dataclass(frozen=True)
class DuvozenLatentAttention:
    heads: int
    dim: int                        # elements of a query/key head that do not turn
    rot_dim: int                    # elements that turn; the keys' are one part shared by the heads
    vdim: int
    kv_rank: int
    scale: float
    rotation: Optional[DuvozenRotation]

    @classmethod
    def from_dict(cls, where: str, raw) -> "DuvozenLatentAttention":
        raw = _section(where, raw, ("heads", "dim", "vdim", "kv_rank", "scale"), ("rot_dim", "rot"))
        rot_dim = 0 if raw.get("rot_dim") in (None, 0) else _positive_int(f"{where}.rot_dim", raw["rot_dim"])
        rotation = None
        if rot_dim:
            if raw.get("rot") is None:
                raise ConfigError(f"{where}: rot_dim without rot")
            rotation = DuvozenRotation.from_dict(f"{where}.rot", raw["rot"], rot_dim)
            if rotation.dims != rot_dim:
                raise ConfigError(f"{where}: rot.dims ({rotation.dims}) must equal rot_dim ({rot_dim})")
        return cls(_positive_int(f"{where}.heads", raw["heads"]), _positive_int(f"{where}.dim", raw["dim"]), rot_dim,
                   _positive_int(f"{where}.vdim", raw["vdim"]), _positive_int(f"{where}.kv_rank", raw["kv_rank"]),
                   _number(f"{where}.scale", raw["scale"]), rotation)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "kv_rank": self.kv_rank, "scale": self.scale}
        if self.rot_dim:
            out["rot_dim"] = self.rot_dim
            out["rot"] = self.rotation.to_dict()
        return out


@dataclass(frozen=True)
class DuvozenAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rotation: Optional[DuvozenRotation]

    @classmethod
    def from_dict(cls, where: str, raw) -> "DuvozenAttention":
        raw = _section(where, raw, ("heads", "kv_heads", "dim", "vdim", "scale"), ("rot",))
        heads, kv_heads = _positive_int(f"{where}.heads", raw["heads"]), _positive_int(f"{where}.kv_heads", raw["kv_heads"])
        if heads % kv_heads:
            raise ConfigError(f"{where}: heads ({heads}) must be a multiple of kv_heads ({kv_heads})")
        dim = _positive_int(f"{where}.dim", raw["dim"])
        rotation = DuvozenRotation.from_dict(f"{where}.rot", raw["rot"], dim) if raw.get("rot") is not None else None
        return cls(heads, kv_heads, dim, _positive_int(f"{where}.vdim", raw["vdim"]), _number(f"{where}.scale", raw["scale"]),
                   rotation)

    def to_dict(self) -> dict:
        out = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rotation is not None:
            out["rot"] = self.rotation.to_dict()
        return out


@dataclass(frozen=True)
class DuvozenFeedForward:
    kind: str                       # "dense" or "moe"
    ff: int                         # of the dense layer, or of one expert
    experts: int = 0
    top: int = 0
    shared_ff: Optional[int] = None

    @classmethod
    def from_dict(cls, where: str, raw) -> "DuvozenFeedForward":
        if not isinstance(raw, dict) or "kind" not in raw:
            raise ConfigError(f"{where} must be an object with a kind, got {raw!r}")
        if raw["kind"] == "dense":
            raw = _section(where, raw, ("kind", "ff"))
            return cls("dense", _positive_int(f"{where}.ff", raw["ff"]))
        if raw["kind"] != "moe":
            raise ConfigError(f"{where}.kind {raw['kind']!r}: this design's feed-forwards are: dense, moe")
        raw = _section(where, raw, ("kind", "expert", "router"), ("shared",))
        ff = _positive_int(f"{where}.expert.ff", _section(f"{where}.expert", raw["expert"], ("ff",))["ff"])
        router = _section(f"{where}.router", raw["router"], ("experts", "top"))
        experts, top = _positive_int(f"{where}.router.experts", router["experts"]), _positive_int(f"{where}.router.top", router["top"])
        if top > experts:
            raise ConfigError(f"{where}.router.top ({top}) is more than the experts ({experts})")
        shared = None
        if raw.get("shared") is not None:
            shared = _positive_int(f"{where}.shared.ff", _section(f"{where}.shared", raw["shared"], ("ff",))["ff"])
        return cls("moe", ff, experts, top, shared)

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        out = {"kind": "moe", "expert": {"ff": self.ff}, "router": {"experts": self.experts, "top": self.top}}
        if self.shared_ff is not None:
            out["shared"] = {"ff": self.shared_ff}
        return out


_MIXERS = {"hgrn2": DuvozenRecurrence, "latent_attention": DuvozenLatentAttention, "attention": DuvozenAttention}


@dataclass(frozen=True)
class DuvozenLayer:
    type: str
    mixer: object
    mlp: Optional[DuvozenFeedForward]


@dataclass(frozen=True)
class DuvozenConfig:
    vocab: int
    width: int
    embedding_scale: float
    logit_scale: float
    norm_eps: float
    taps: int
    layers: tuple
    raw: Optional[dict] = None

    @classmethod
    def from_dict(cls, raw: dict) -> "DuvozenConfig":
        raw = _section("config.json", raw, ("vocab", "width", "norm", "layers", "canon"),
                       ("architecture", "architectures", "embedding", "logit_scale"))
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config.json: layers must be a list with at least one layer")
        layers = []
        for i, entry in enumerate(raw["layers"]):
            where = f"layers[{i}]"
            entry = _section(where, entry, ("type", "mixer"), ("mlp",))
            if entry["type"] not in _MIXERS:
                raise ConfigError(f"{where}.type {entry['type']!r}: this design's mixers are: {', '.join(MIXER_TYPES)}")
            mixer = _MIXERS[entry["type"]].from_dict(f"{where}.mixer", entry["mixer"])
            mlp = DuvozenFeedForward.from_dict(f"{where}.mlp", entry["mlp"]) if entry.get("mlp") is not None else None
            layers.append(DuvozenLayer(entry["type"], mixer, mlp))
        scale = 1.0
        if raw.get("embedding") is not None:
            scale = _any_number("embedding.scale", _section("embedding", raw["embedding"], ("scale",))["scale"])
        taps = _positive_int("canon.taps", _section("canon", raw["canon"], ("taps",))["taps"])
        if taps > 64:
            raise ConfigError(f"canon.taps ({taps}): at most 64")
        return cls(vocab=_positive_int("vocab", raw["vocab"]), width=_positive_int("width", raw["width"]),
                   embedding_scale=scale,
                   logit_scale=_any_number("logit_scale", raw["logit_scale"]) if raw.get("logit_scale") is not None else 1.0,
                   norm_eps=_number("norm.eps", _section("norm", raw["norm"], ("eps",))["eps"], positive=False),
                   taps=taps, layers=tuple(layers), raw=raw)

    def to_dict(self) -> dict:
        """The config.json of this configuration."""
        if self.raw is not None:
            return dict(self.raw)
        return {"architecture": "Duvozen", "vocab": self.vocab, "width": self.width,
                "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
                "norm": {"eps": self.norm_eps}, "canon": {"taps": self.taps},
                "layers": [{"type": layer.type, "mixer": layer.mixer.to_dict(),
                            "mlp": None if layer.mlp is None else layer.mlp.to_dict()} for layer in self.layers]}
