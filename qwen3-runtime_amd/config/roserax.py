"""Typed configuration of a Roserax decoder, read from a model folder's ``config.json``.

The file names the design under ``architecture`` and gives ``vocab``, ``width``, the norms' ``eps``
(``norm.eps``), what the embedding is multiplied by (``embedding.scale``) and the logits
(``logit_scale``), and ``layers``: per layer its ``type`` (``attention``: softmax attention over a
window that keeps the sequence's first tokens in sight, with a sink in the softmax;
``latent_attention``: attention whose queries and keys/values pass through low-rank vectors;
``retention``: linear attention with a fixed decay per head), the mixer's sizes (``mixer``) and its
feed-forward (``mlp``: ``dense``, ``moe``, or null). Every size and every constant that may differ
between two models of the design is read here. Absent options mean "not there": no ``kv_heads`` a
key head per query head, no ``vdim`` values as wide as keys, no ``keep_first`` none kept, no
``groups`` one group.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping

from .deginex import _positive, _unknown
from .model import ConfigError
from .zisedra import _number


@dataclass(frozen=True)
class HalfRotation:
    """The first ``dims`` elements of the rotated vector turn, element ``i`` against element
    ``i + dims/2``, with frequencies ``base^(-2i/dims)``."""

    dims: int
    base: float

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "HalfRotation":
        dims = raw.get("dims")
        if isinstance(dims, bool) or not isinstance(dims, int) or dims < 0 or dims % 2:
            raise ConfigError(f"{where}: rot.dims must be an even number of elements, got {dims!r}")
        _unknown(where + " rot", raw, {"dims", "base"})
        return cls(dims, _number(where + " rot", "base", raw))

    def to_dict(self) -> dict[str, Any]:
        return {"dims": self.dims, "base": self.base}


def _heads(raw: Mapping[str, Any], where: str, need=("heads", "dim")) -> None:
    for key in need:
        if key not in raw:
            raise ConfigError(f"{where}: the mixer lacks {key!r}")


@dataclass(frozen=True)
class WindowSinkSizes:
    """``heads`` query heads on ``kv_heads`` key/value heads, keys of ``dim`` and values of ``vdim``
    elements, scores times ``scale``; a query sees itself, the ``window - 1`` tokens before it and
    the sequence's first ``keep_first``."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "WindowSinkSizes":
        _heads(raw, where, ("heads", "dim", "scale", "mask"))
        heads = _positive(where, "heads", raw["heads"])
        kv_heads = _positive(where, "kv_heads", raw.get("kv_heads", heads))
        if heads % kv_heads:
            raise ConfigError(f"{where}: {heads} query heads do not divide into {kv_heads} key/value heads")
        dim = _positive(where, "dim", raw["dim"])
        mask = raw["mask"]
        keep = mask.get("keep_first", 0)
        if isinstance(keep, bool) or not isinstance(keep, int) or keep < 0:
            raise ConfigError(f"{where}: mask.keep_first must be a number of tokens, got {keep!r}")
        _unknown(where + " mask", mask, {"size", "keep_first"})
        _unknown(where + " mixer", raw, {"heads", "kv_heads", "dim", "vdim", "scale", "mask"})
        return cls(heads, kv_heads, dim, _positive(where, "vdim", raw.get("vdim", dim)), _number(where, "scale", raw),
                   _positive(where, "mask.size", mask.get("size")), keep)

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale,
                "mask": {"size": self.window, "keep_first": self.keep_first}}


@dataclass(frozen=True)
class LatentSizes:
    """``heads`` heads whose queries and keys have ``dim`` elements that do not turn and ``rot_dim``
    that do, values of ``vdim``; queries come from a vector of ``q_rank`` elements, keys and values
    from one of ``kv_rank``."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot: HalfRotation

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "LatentSizes":
        _heads(raw, where, ("heads", "dim", "rot_dim", "q_rank", "kv_rank", "scale", "rot"))
        dim = _positive(where, "dim", raw["dim"])
        rot_dim = _positive(where, "rot_dim", raw["rot_dim"])
        rot = HalfRotation.from_dict(raw["rot"], where)
        if rot.dims > rot_dim:
            raise ConfigError(f"{where}: {rot.dims} rotated elements in a part of {rot_dim}")
        _unknown(where + " mixer", raw, {"heads", "dim", "rot_dim", "vdim", "q_rank", "kv_rank", "scale", "rot"})
        return cls(_positive(where, "heads", raw["heads"]), dim, rot_dim, _positive(where, "vdim", raw.get("vdim", dim)),
                   _positive(where, "q_rank", raw["q_rank"]), _positive(where, "kv_rank", raw["kv_rank"]),
                   _number(where, "scale", raw), rot)

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class RetentionSizes:
    """``heads`` heads with keys of ``dim`` and values of ``vdim`` elements and one ``decay`` each."""

    heads: int
    dim: int
    vdim: int
    decay: tuple[float, ...]
    rot: HalfRotation

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "RetentionSizes":
        _heads(raw, where, ("heads", "dim", "decay", "rot"))
        heads = _positive(where, "heads", raw["heads"])
        dim = _positive(where, "dim", raw["dim"])
        decay = raw["decay"]
        if not isinstance(decay, (list, tuple)) or len(decay) != heads or \
                any(isinstance(x, bool) or not isinstance(x, (int, float)) for x in decay):
            raise ConfigError(f"{where}: decay lists one number per head ({heads}), got {decay!r}")
        rot = HalfRotation.from_dict(raw["rot"], where)
        if rot.dims > dim:
            raise ConfigError(f"{where}: {rot.dims} rotated elements in heads of {dim}")
        _unknown(where + " mixer", raw, {"heads", "dim", "vdim", "decay", "rot"})
        return cls(heads, dim, _positive(where, "vdim", raw.get("vdim", dim)), tuple(float(x) for x in decay), rot)

    def to_dict(self) -> dict[str, Any]:
        return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "decay": list(self.decay), "rot": self.rot.to_dict()}


@dataclass(frozen=True)
class FeedForwardSizes:
    """``kind`` "dense": inner width ``ff``. ``kind`` "moe": ``experts`` experts of inner width ``ff``,
    ``top`` a token, from the ``keep`` best of ``groups`` groups."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0
    groups: int = 1
    keep: int = 1

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any], where: str) -> "FeedForwardSizes":
        kind = raw.get("kind")
        if kind == "dense":
            _unknown(where + " mlp", raw, {"kind", "ff"})
            return cls("dense", _positive(where, "mlp.ff", raw.get("ff")))
        if kind != "moe":
            raise ConfigError(f"{where}: unknown feed-forward kind {kind!r} (dense, moe)")
        router, expert = raw.get("router") or {}, raw.get("expert") or {}
        experts = _positive(where, "mlp.router.experts", router.get("experts"))
        top = _positive(where, "mlp.router.top", router.get("top"))
        groups, keep = 1, 1
        if router.get("groups") is not None:
            groups = _positive(where, "mlp.router.groups.count", router["groups"].get("count"))
            keep = _positive(where, "mlp.router.groups.keep", router["groups"].get("keep"))
        if experts % groups or keep > groups or keep * (experts // groups) < top or groups > 64:
            raise ConfigError(f"{where}: {experts} experts in {groups} groups (64 at most) of which {keep} stay, {top} chosen")
        _unknown(where + " mlp", raw, {"kind", "router", "expert"})
        _unknown(where + " mlp.router", router, {"experts", "top", "groups"})
        _unknown(where + " mlp.expert", expert, {"ff"})
        return cls("moe", _positive(where, "mlp.expert.ff", expert.get("ff")), experts, top, groups, keep)

    def to_dict(self) -> dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.keep}}}


MIXERS = {"attention": WindowSinkSizes, "latent_attention": LatentSizes, "retention": RetentionSizes}


@dataclass(frozen=True)
class RoseraxLayer:
    kind: str  # a key of MIXERS
    mixer: Any
    feed_forward: FeedForwardSizes | None


@dataclass(frozen=True)
class RoseraxConfig:
    vocab: int
    width: int
    eps: float
    layers: tuple[RoseraxLayer, ...]
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    max_positions: int = 1 << 20
    eos_token_id: int | None = None

    architecture = "Roserax"

    def __post_init__(self) -> None:
        _positive("config", "vocab", self.vocab)
        _positive("config", "width", self.width)
        if not self.eps > 0.0:
            raise ConfigError(f"norm.eps must be positive, got {self.eps!r}")
        if not self.layers:
            raise ConfigError("the model has no layers")

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "RoseraxConfig":
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
            layers.append(RoseraxLayer(kind, MIXERS[kind].from_dict(spec.get("mixer") or {}, where),
                                       None if mlp is None else FeedForwardSizes.from_dict(mlp, where)))
        eos = raw.get("eos_token_id")
        embedding = raw.get("embedding") or {}
        _unknown("config embedding", embedding, {"scale"})
        _unknown("config", raw, {"architecture", "architectures", "vocab", "width", "layers", "norm", "embedding",
                                 "logit_scale", "max_positions", "eos_token_id"})
        return cls(vocab=raw["vocab"], width=raw["width"], eps=float((raw["norm"] or {}).get("eps", 0.0)),
                   layers=tuple(layers), embedding_scale=float(embedding.get("scale", 1.0)),
                   logit_scale=float(raw.get("logit_scale", 1.0)),
                   max_positions=int(raw.get("max_positions", 1 << 20)), eos_token_id=None if eos is None else int(eos))

    def to_dict(self) -> dict[str, Any]:
        """The config.json a model folder of this configuration carries."""
        raw: dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.eps},
            "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale,
            "layers": [{"type": layer.kind, "mixer": layer.mixer.to_dict(),
                        "mlp": None if layer.feed_forward is None else layer.feed_forward.to_dict()} for layer in self.layers]}
        if self.max_positions != 1 << 20:
            raw["max_positions"] = self.max_positions
        if self.eos_token_id is not None:
            raw["eos_token_id"] = self.eos_token_id
        return raw
