"""The Roserax decoder as a plan of parts.

One residual stream that starts as the embedding times a constant; every sub-layer has an RMS
norm in front of it and one behind it (``x += norm_b(f(norm(x)))``). A layer's mixer is softmax
attention over a window that keeps the sequence's first tokens in sight and has a sink in its
softmax, attention through a latent, or retention; its feed-forward is dense with a squared relu,
a routed mixture of silu-gated experts chosen by softmax scores from the best groups, or nothing.
The head is the embedding table and the logits are multiplied by a constant. Tensor names are
those of the model file: ``embed``, ``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.mix.*``,
``l<i>.mlp.up|down`` or ``l<i>.mlp.router`` and ``l<i>.mlp.e<j>.gate|up|down``, ``final.norm``.
"""

from __future__ import annotations

from ..config.roserax import (FeedForwardSizes, HalfRotation, LatentSizes, RetentionSizes, RoseraxConfig, RoseraxLayer,
                              WindowSinkSizes)
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, RunStep
from ..registry import part_class, register_architecture, register_preset


def _norm(cfg: RoseraxConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, {"weight": name})


def _mixer(cfg: RoseraxConfig, layer: RoseraxLayer, p: str) -> PartSpec:
    s = layer.mixer
    if layer.kind == "attention":
        tensors = {n: f"{p}.{n}" for n in ("q", "k", "v", "o")}
        tensors.update(q_norm=f"{p}.q.norm", k_norm=f"{p}.k.norm")
        return PartSpec("gqa_attention", {"hidden_size": cfg.width, "num_heads": s.heads, "num_kv_heads": s.kv_heads,
                                          "head_dim": s.dim, "value_dim": s.vdim, "scale": s.scale, "window": s.window,
                                          "keep_first": s.keep_first, "sink": True, "qk_norm_eps": cfg.eps}, tensors)
    if layer.kind == "latent_attention":
        tensors = {n: f"{p}.{n}" for n in ("dq", "uq", "dkv", "uk", "uv", "g", "o")}
        tensors.update(dq_norm=f"{p}.dq.norm", dkv_norm=f"{p}.dkv.norm")
        return PartSpec("latent_attention", {"hidden_size": cfg.width, "num_heads": s.heads, "head_dim": s.dim,
                                             "rot_dim": s.rot_dim, "value_dim": s.vdim, "q_rank": s.q_rank,
                                             "kv_rank": s.kv_rank, "scale": s.scale, "norm_eps": cfg.eps,
                                             "rot_dims": s.rot.dims, "rot_base": s.rot.base}, tensors)
    return PartSpec("retention", {"hidden_size": cfg.width, "num_heads": s.heads, "head_dim": s.dim, "value_dim": s.vdim,
                                  "decay": tuple(s.decay), "norm_eps": cfg.eps, "rot_dims": s.rot.dims,
                                  "rot_base": s.rot.base}, {n: f"{p}.{n}" for n in ("q", "k", "v", "g", "o")})


def _feed_forward(cfg: RoseraxConfig, s: FeedForwardSizes | None, p: str) -> PartSpec | None:
    if s is None:
        return None
    if s.kind == "dense":
        return PartSpec("act_mlp", {"hidden_size": cfg.width, "intermediate_size": s.ff, "activation": "relu2"},
                        {"up": f"{p}.mlp.up", "down": f"{p}.mlp.down"})
    tensors = {n: f"{p}.mlp.e{{e}}.{n}" for n in ("gate", "up", "down")}
    tensors["router"] = f"{p}.mlp.router"
    return PartSpec("routed_experts", {"hidden_size": cfg.width, "intermediate_size": s.ff, "num_experts": s.experts,
                                       "top": s.top, "router_bias": False, "scoring": "softmax_all", "groups": s.groups,
                                       "keep": s.keep, "group_score": "max"}, tensors)


def plan_roserax(cfg: RoseraxConfig) -> ModelPlan:
    layers, caches, order, unread = [], [], [], []
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ff = _feed_forward(cfg, layer.feed_forward, p)
        norms = {"input": _norm(cfg, f"{p}.norm1"), "after_mixer": _norm(cfg, f"{p}.norm1b")}
        if ff is not None:
            norms.update(post_mixer=_norm(cfg, f"{p}.norm2"), after_ff=_norm(cfg, f"{p}.norm2b"))
        else:  # a file may carry the norms of a feed-forward that is not there
            unread += [f"{p}.norm2", f"{p}.norm2b"]
        mixer = _mixer(cfg, layer, f"{p}.mix")
        layers.append(LayerSpec(PartSpec("sandwich_norm"), mixer, ff, norms))
        specs = part_class("mixer", mixer.kind)(**mixer.args, tensors=mixer.tensors).cache_specs()
        ids = tuple(range(len(caches), len(caches) + len(specs)))
        caches.extend(specs)
        order.append(RunStep(layer=i, cache=ids[0] if len(ids) == 1 else (ids or None)))
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width}
    return ModelPlan(
        hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("token_embedding", {**sizes, "scale": cfg.embedding_scale}, {"weight": "embed"}),
        layers=layers, caches=caches, order=order, final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear_head", {**sizes, "scale": cfg.logit_scale}, {"weight": "embed"}),
        ignorable=tuple(unread), eos_token_id=cfg.eos_token_id,
    )


# Small configurations for tests and examples; they differ in every size and option.
_ROT = HalfRotation
PRESETS: dict[str, RoseraxConfig] = {
    "roserax_tiny_a": RoseraxConfig(
        vocab=210, width=80, eps=1e-5, embedding_scale=3.0, logit_scale=0.5,
        layers=(
            RoseraxLayer("retention", RetentionSizes(3, 32, 16, (0.9, 0.97, 0.995), _ROT(16, 5000.0)),
                         FeedForwardSizes("moe", 24, experts=12, top=3, groups=4, keep=2)),
            RoseraxLayer("attention", WindowSinkSizes(6, 2, 32, 16, 0.2, 21, 3), FeedForwardSizes("dense", 112)),
            RoseraxLayer("latent_attention", LatentSizes(5, 16, 8, 24, 40, 24, 0.3, _ROT(8, 100.0)), None),
            RoseraxLayer("attention", WindowSinkSizes(4, 4, 16, 16, 0.25, 9, 0),
                         FeedForwardSizes("moe", 40, experts=6, top=2, groups=1, keep=1)),
        ),
    ),
    "roserax_tiny_b": RoseraxConfig(
        vocab=150, width=64, eps=1e-6, embedding_scale=1.0, logit_scale=1.0,
        layers=(
            RoseraxLayer("latent_attention", LatentSizes(2, 32, 16, 16, 24, 48, 0.15, _ROT(12, 1e4)),
                         FeedForwardSizes("moe", 32, experts=8, top=1, groups=2, keep=1)),
            RoseraxLayer("attention", WindowSinkSizes(2, 1, 48, 48, 0.1, 40, 17), None),
            RoseraxLayer("retention", RetentionSizes(2, 24, 40, (0.5, 1.0), _ROT(24, 1e6)), FeedForwardSizes("dense", 96)),
        ),
    ),
}
PRESET_PAGE_SIZE = {"roserax_tiny_a": 16, "roserax_tiny_b": 8}


def sized(width: int, layers: int, heads: int, kv_heads: int, dim: int, vocab: int, *, ff: int, expert_ff: int,
          experts: int = 16, top: int = 2, window: int = 2048, keep_first: int = 4, kv_rank: int = 384, q_rank: int = 768,
          rot_dim: int = 64) -> RoseraxConfig:
    """A configuration of the sizes of a real model, for measurements: latent attention, retention
    and two windowed layers in turn, dense feed-forwards and mixtures alternating."""
    att = WindowSinkSizes(heads, kv_heads, dim, dim, dim ** -0.5, window, keep_first)
    lat = LatentSizes(heads, dim, rot_dim, dim, q_rank, kv_rank, (dim + rot_dim) ** -0.5, _ROT(rot_dim, 1e6))
    ret = RetentionSizes(heads, dim, dim, tuple(1.0 - 0.06 / (1 + j) for j in range(heads)),
                         _ROT(dim, 1e6))
    dense, moe = FeedForwardSizes("dense", ff), FeedForwardSizes("moe", expert_ff, experts=experts, top=top, groups=4, keep=2)
    kinds = (("latent_attention", lat), ("retention", ret), ("attention", att), ("attention", att))
    return RoseraxConfig(vocab=vocab, width=width, eps=1e-5, embedding_scale=1.0, logit_scale=1.0, layers=tuple(
        RoseraxLayer(*kinds[i % 4], dense if i % 2 == 0 else moe) for i in range(layers)))


register_architecture(RoseraxConfig.architecture, RoseraxConfig.from_dict, plan_roserax)
for _name, _cfg in PRESETS.items():
    register_preset(_name, _cfg.to_dict(), PRESET_PAGE_SIZE.get(_name, 16))
# layers of the sizes of the 4B and 8B dense presets, and of a smaller width, with a mixture like
# `deginex_4b_moe`'s in every second layer, for measurements beside it
register_preset("roserax_4b", sized(2560, 36, 32, 8, 128, 151936, ff=9728, expert_ff=1536).to_dict(), 16)
register_preset("roserax_8b", sized(4096, 36, 32, 8, 128, 151936, ff=12288, expert_ff=2048, kv_rank=448, q_rank=1536).to_dict(), 16)
register_preset("roserax_2b", sized(2048, 28, 16, 4, 128, 151936, ff=6144, expert_ff=1024, kv_rank=256, q_rank=512).to_dict(), 16)
