"""Typed configuration of a Zuvasun decoder, read from a model folder's ``config.json``.

The file names the design under ``architecture`` and gives ``vocab``, ``width``, the norms' ``eps``
(``norm.eps``) and ``layers``: per layer its ``type`` (``latent_attention``: attention whose keys and
values are made from a low-rank vector, with a rotated key part all heads share, over a sliding
window; ``attention``: grouped-query attention without rotation whose values are its keys), the
mixer's sizes (``mixer``) and its feed-forward (``mlp``: a mixture of experts, or null). Every size
and every constant that may differ between two models of the design is read here. Absent
options mean "not there": no ``kv_heads`` a key head per query head, no ``mask`` every earlier key
in sight, no ``rot.scaling`` plain frequencies, no ``q_temp`` queries as they are, no ``kv_from`` a
latent of the layer's own, no ``router.scale`` weights as normalised.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .deginex import _positive, _unknown
from .model import ConfigError
from .zisedra import _number


@dataclass(frozen=True)
class StretchedFrequencies:
    """YaRN's change of a rotation's frequencies: pairs that turn more often than ``fast`` times
    over ``original`` positions keep theirs, pairs that turn less often than ``slow`` times have
    theirs divided by ``factor``, a linear ramp over the pairs in between; cosines and sines are
    multiplied by ``0.1 ln(factor) + 1``."""

    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "StretchedFrequencies":
        _unknown(where + " rot.scaling", raw, {"factor", "original", "fast", "slow"})
        return cls(*(_number(where + " rot.scaling", key, raw) for key in ("factor", "original", "fast", "slow")))

    def to_dict(self) -> dict[str, Any]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class PairRotation:
    """The first ``dims`` elements of the rotated vector turn, element ``2i`` against element
    ``2i + 1``, with frequencies ``base^(-2i/dims)``, stretched by ``scaling`` if there is one."""

    dims: int
    base: float
    scaling: StretchedFrequencies | None = None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "PairRotation":
        dims = raw.get("dims")
        if isinstance(dims, bool) or not isinstance(dims, int) or dims < 0 or dims % 2:
            raise ConfigError(f"{where}: rot.dims must be an even number of elements, got {dims!r}")
        _unknown(where + " rot", raw, {"dims", "base", "scaling"})
        scaling = raw.get("scaling")
        return cls(dims, _number(where + " rot", "base", raw),
                   None if scaling is None else StretchedFrequencies.from_dict(scaling, where))

    def to_dict(self) -> dict[str, Any]:
        raw: dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.scaling is not None:
            raw["scaling"] = self.scaling.to_dict()
        return raw


def _window(raw: Mapping[str, Any], where: str) -> int | None:
    mask = raw.get("mask")
    if mask is None:
        return None
    _unknown(where + " mask", mask, {"size"})
    return None if mask.get("size") is None else _positive(where, "mask.size", mask["size"])


@dataclass(frozen=True)
class SharedLatentSizes:
    """``heads`` heads whose queries and keys have ``dim`` elements that do not turn and ``rot_dim``
    that do, values of ``vdim``; keys and values come from a vector of ``kv_rank`` elements. A query
    sees itself and the ``window - 1`` tokens before it (None: all). ``kv_from``: the layer whose
    cached latent and rotated key part this one reads instead of making its own."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    rot: PairRotation
    window: int | None = None
    kv_from: int | None = None

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "SharedLatentSizes":
        for key in ("heads", "dim", "rot_dim", "kv_rank", "scale", "rot"):
            if key not in raw:
                raise ConfigError(f"{where}: the mixer lacks {key!r}")
        dim = _positive(where, "dim", raw["dim"])
        rot_dim = _positive(where, "rot_dim", raw["rot_dim"])
        rot = PairRotation.from_dict(raw["rot"], where)
        if rot.dims > rot_dim:
            raise ConfigError(f"{where}: {rot.dims} rotated elements in a part of {rot_dim}")
        kv_from = raw.get("kv_from")
        if kv_from is not None and (isinstance(kv_from, bool) or not isinstance(kv_from, int) or kv_from < 0):
            raise ConfigError(f"{where}: kv_from names an earlier layer, got {kv_from!r}")
        _unknown(where + " mixer", raw, {"heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot", "mask", "kv_from"})
        return cls(_positive(where, "heads", raw["heads"]), dim, rot_dim, _positive(where, "vdim", raw.get("vdim", dim)),
                   _positive(where, "kv_rank", raw["kv_rank"]), _number(where, "scale", raw), rot, _window(raw, where), kv_from)

    def to_dict(self) -> dict[str, Any]:
        raw: dict[str, Any] = {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim,
                               "kv_rank": self.kv_rank, "scale": self.scale, "rot": self.rot.to_dict()}
        if self.window is not None:
            raw["mask"] = {"size": self.window}
        if self.kv_from is not None:
            raw["kv_from"] = self.kv_from
        return raw


@dataclass(frozen=True)
class KeyValueSizes:
    """``heads`` query heads on ``kv_heads`` key heads of ``dim`` elements whose values are the keys as
    projected; scores times ``scale``; queries at position ``p`` times
    ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)`` (``temp_coef`` None: as they are)."""

    heads: int
    kv_heads: int
    dim: int
    scale: float
    temp_coef: float | None = None
    temp_every: int = 1

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "KeyValueSizes":
        for key in ("heads", "dim", "scale"):
            if key not in raw:
                raise ConfigError(f"{where}: the mixer lacks {key!r}")
        heads = _positive(where, "heads", raw["heads"])
        kv_heads = _positive(where, "kv_heads", raw.get("kv_heads", heads))
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} query heads do not divide into {kv_heads} key/value heads")
        dim = _positive(where, "dim", raw["dim"])
        if raw.get("vdim", dim) != dim:
            raise ConfigError(f"{where}: the values are the keys, of {dim} elements; vdim is {raw['vdim']!r}")
        coef, every = None, 1
        temp = raw.get("q_temp")
        if temp is not None:
            _unknown(where + " q_temp", temp, {"coef", "every"})
            coef = _number(where + " q_temp", "coef", temp, positive=False)
            every = _positive(where, "q_temp.every", temp.get("every"))
        _unknown(where + " mixer", raw, {"heads", "kv_heads", "dim", "vdim", "scale", "q_temp"})
        return cls(heads, kv_heads, dim, _number(where, "scale", raw), coef, every)

    def to_dict(self) -> dict[str, Any]:
        raw: dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.dim,
                               "scale": self.scale}
        if self.temp_coef is not None:
            raw["q_temp"] = {"coef": self.temp_coef, "every": self.temp_every}
        return raw


@dataclass(frozen=True)
class MixtureSizes:
    """``experts`` experts of inner width ``ff``, ``top`` a token, their weights times ``scale``."""

    ff: int
    experts: int
    top: int
    scale: float = 1.0

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "MixtureSizes":
        if raw.get("kind") != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {raw.get('kind')!r} (moe)")
        router, expert = raw.get("router") or {}, raw.get("expert") or {}
        experts = _positive(where, "mlp.router.experts", router.get("experts"))
        top = _positive(where, "mlp.router.top", router.get("top"))
        if top > experts:
            raise ConfigError(f"{where}: {top} of {experts} experts")
        _unknown(where + " mlp", raw, {"kind", "router", "expert"})
        _unknown(where + " mlp.router", router, {"experts", "top", "scale"})
        _unknown(where + " mlp.expert", expert, {"ff"})
        scale = _number(where + " mlp.router", "scale", router, positive=False) if "scale" in router else 1.0
        return cls(_positive(where, "mlp.expert.ff", expert.get("ff")), experts, top, scale)

    def to_dict(self) -> dict[str, Any]:
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "scale": self.scale}}


MIXERS = {"latent_attention": SharedLatentSizes, "attention": KeyValueSizes}


@dataclass(frozen=True)
class ZuvasunLayer:
    kind: str  # a key of MIXERS
    mixer: Any
    feed_forward: MixtureSizes | None


@dataclass(frozen=True)
class ZuvasunConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple[ZuvasunLayer, ...]
    max_positions: int = 1 << 20
    eos_token_id: int | None = None

    architecture = "Zuvasun"

    def __post_init__(self) -> None:
        _positive("config", "vocab", self.vocab)
        _positive("config", "width", self.width)
        if not self.eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps!r}")
        if not self.layers:
            raise ConfigError("the model has no layers")
        for i, layer in enumerate(self.layers):
            src = getattr(layer.mixer, "kv_from", None)
            if src is None:
                continue
            if not 0 <= src < i or self.layers[src].kind != "latent_attention" or self.layers[src].mixer.kv_from is not None:
                raise ConfigError(f"layer {i}: kv_from {src} is no earlier latent layer with a latent of its own")
            own, other = layer.mixer, self.layers[src].mixer
            if (own.kv_rank, own.rot_dim, own.rot) != (other.kv_rank, other.rot_dim, other.rot):
                raise ConfigError(f"layer {i}: latent, rotated part and rotation must equal those of layer {src}, whose cache it reads")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "ZuvasunConfig":
        if raw.get("architecture") != cls.architecture and cls.architecture not in (raw.get("architectures") or []):
            raise ConfigError(f"unsupported architecture: {raw.get('architecture')!r}")
        for key in ("vocab", "width", "layers", "norm"):
            if key not in raw:
                raise ConfigError(f"config.json lacks {key!r}")
        layers = []
        for i, spec in enumerate(raw["layers"]):
            where = f"layer {i}"
            kind = spec.get("type")
            if kind not in MIXERS:
                raise ConfigError(f"{where}: unknown mixer type {kind!r} ({', '.join(MIXERS)})")
            mlp = spec.get("mlp")
            _unknown(where, spec, {"type", "mixer", "mlp"})
            layers.append(ZuvasunLayer(kind, MIXERS[kind].from_dict(spec.get("mixer") or {}, where),
                                       None if mlp is None else MixtureSizes.from_dict(mlp, where)))
        eos = raw.get("eos_token_id")
        _unknown("config", raw, {"architecture", "architectures", "vocab", "width", "layers", "norm", "max_positions",
                                 "eos_token_id"})
        return cls(vocab=raw["vocab"], width=raw["width"], eps=float((raw["norm"] or {}).get("eps", 0.0)),
                   layers=tuple(layers), max_positions=int(raw.get("max_positions", 1 << 20)),
                   eos_token_id=None if eos is None else int(eos))

    def to_dict(self) -> dict[str, Any]:
        """The config.json a model folder of this configuration carries."""
        raw: dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
            "layers": [{"type": layer.kind, "mixer": layer.mixer.to_dict(),
                        "mlp": None if layer.feed_forward is None else layer.feed_forward.to_dict()} for layer in self.layers]}
        if self.max_positions != 1 << 20:
            raw["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            raw["eos_token_id"] = self.eos_token_id
        return raw
