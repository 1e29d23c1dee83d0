"""The Zuvasun decoder as a plan of parts.

One residual stream. A layer has one RMS norm that both of its sub-layers read; their outputs,
each times a vector, join the stream in one sum (``x += s1 * mixer(n) + s2 * ff(n)``, ``n = norm(x)``).
A layer's mixer is attention through a latent (full-rank queries, pairs of neighbours rotated with
stretched frequencies, a sliding window; a layer may read the latent that an earlier layer
cached instead of making one) or grouped-query attention without rotation whose values are its
keys, with biases, a norm over each whole projection and a query temperature. Its feed-forward is
a mixture of squared-relu experts chosen by softmax scores plus a correction, the chosen scores
renormalised and scaled, or nothing. The head has a matrix of its own. Tensor names are those of
the model file: ``embed``, ``l<i>.norm1``, ``l<i>.ls1|ls2``, ``l<i>.mix.*``, ``l<i>.mlp.router|correction``,
``l<i>.mlp.e<j>.up|down``, ``final.norm``, ``head``.
"""

from __future__ import annotations

from ..config.zuvasun import (KeyValueSizes, MixtureSizes, PairRotation, SharedLatentSizes, StretchedFrequencies,
                              ZuvasunConfig, ZuvasunLayer)
from ..parts.plan import LayerSpec, ModelPlan, PartSpec, RunStep
from ..registry import part_class, register_architecture, register_preset


def _norm(cfg: ZuvasunConfig, name: str) -> PartSpec:
    return PartSpec("rmsnorm", {"size": cfg.width, "eps": cfg.eps}, {"weight": name})


def _cache_windows(cfg: ZuvasunConfig) -> dict[int, int | None]:
    """Per layer that owns a latent cache: how many tokens it keeps, the widest window among the
    layer itself and the layers that read its cache (None: all tokens)."""
    keep: dict[int, int | None] = {}
    for i, layer in enumerate(cfg.layers):
        if layer.kind != "latent_attention":
            continue
        owner = i if layer.mixer.kv_from is None else layer.mixer.kv_from
        window = layer.mixer.window
        if owner not in keep:
            keep[owner] = window
        elif keep[owner] is not None:
            keep[owner] = None if window is None else max(keep[owner], window)
    return keep


def _mixer(cfg: ZuvasunConfig, layer: ZuvasunLayer, p: str, cache_window) -> PartSpec:
    s = layer.mixer
    if layer.kind == "latent_attention":
        own = s.kv_from is None
        tensors = {n: f"{p}.{n}" for n in ("q", "uk", "uv", "o")}
        if own:
            tensors.update(dkv=f"{p}.dkv", dkv_norm=f"{p}.dkv.norm")
        sc = s.rot.scaling
        return PartSpec("latent_attention", {
            "hidden_size": cfg.width, "num_heads": s.heads, "head_dim": s.dim, "rot_dim": s.rot_dim, "value_dim": s.vdim,
            "q_rank": None, "kv_rank": s.kv_rank, "scale": s.scale, "norm_eps": cfg.eps, "rot_dims": s.rot.dims,
            "rot_base": s.rot.base, "output_gate": False, "window": s.window, "cache_window": cache_window,
            "rotation": "pairs", "rot_scaling": None if sc is None else (sc.factor, sc.original, sc.fast, sc.slow),
            "own_latent": own}, tensors)
    tensors = {"q": f"{p}.q", "k": f"{p}.k", "o": f"{p}.o", "q_bias": f"{p}.q.b", "k_bias": f"{p}.k.b",
               "q_norm": f"{p}.q.norm", "k_norm": f"{p}.k.norm"}
    return PartSpec("gqa_attention", {
        "hidden_size": cfg.width, "num_heads": s.heads, "num_kv_heads": s.kv_heads, "head_dim": s.dim, "scale": s.scale,
        "qk_norm_eps": cfg.eps, "qk_norm_scope": "projection", "values_are_keys": True, "bias": True,
        "q_temp": None if s.temp_coef is None else (s.temp_coef, s.temp_every)}, tensors)


def _feed_forward(cfg: ZuvasunConfig, s: MixtureSizes | None, p: str) -> PartSpec | None:
    if s is None:
        return None
    tensors = {n: f"{p}.mlp.e{{e}}.{n}" for n in ("up", "down")}
    tensors.update(router=f"{p}.mlp.router", correction=f"{p}.mlp.correction")
    return PartSpec("routed_experts", {"hidden_size": cfg.width, "intermediate_size": s.ff, "num_experts": s.experts,
                                       "top": s.top, "router_bias": False, "scoring": "softmax_all", "activation": "relu2",
                                       "correction": True, "renormalise": True, "weight_scale": s.scale}, tensors)


def plan_zuvasun(cfg: ZuvasunConfig) -> ModelPlan:
    layers, caches, order, unread = [], [], [], []
    keep = _cache_windows(cfg)
    cache_of: dict[int, int] = {}  # latent layer with a cache of its own -> its cache
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}"
        ff = _feed_forward(cfg, layer.feed_forward, p)
        src = getattr(layer.mixer, "kv_from", None)
        mixer = _mixer(cfg, layer, f"{p}.mix", keep.get(i if src is None else src))
        scales = {"scale1": f"{p}.ls1"}
        if ff is not None:
            scales["scale2"] = f"{p}.ls2"
        else:  # a file may carry the vector of a feed-forward that is not there
            unread.append(f"{p}.ls2")
        layers.append(LayerSpec(PartSpec("parallel_scaled", {"hidden_size": cfg.width}, scales), mixer, ff,
                                {"input": _norm(cfg, f"{p}.norm1")}))
        if src is not None:
            # the layer reads what layer `src` stored earlier in the same pass
            order.append(RunStep(layer=i, cache=cache_of[src], writes_cache=False))
            continue
        (spec,) = part_class("mixer", mixer.kind)(**mixer.args, tensors=mixer.tensors).cache_specs()
        cache_of[i] = len(caches)
        caches.append(spec)
        order.append(RunStep(layer=i, cache=cache_of[i]))
    sizes = {"vocab_size": cfg.vocab, "hidden_size": cfg.width}
    return ModelPlan(
        hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=PartSpec("token_embedding", sizes, {"weight": "embed"}),
        layers=layers, caches=caches, order=order, final_norm=_norm(cfg, "final.norm"),
        head=PartSpec("linear_head", sizes, {"weight": "head"}),
        ignorable=tuple(unread), eos_token_id=cfg.eos_token_id,
    )


# Small configurations for tests and examples; they differ in every size and option.
_STRETCH = StretchedFrequencies
PRESETS: dict[str, ZuvasunConfig] = {
    "zuvasun_tiny_a": ZuvasunConfig(
        vocab=230, width=96, eps=1e-5,
        layers=(
            ZuvasunLayer("attention", KeyValueSizes(6, 2, 16, 0.2, 0.3, 5), MixtureSizes(40, 6, 2, 1.5)),
            ZuvasunLayer("latent_attention", SharedLatentSizes(3, 16, 16, 24, 32, 0.2, PairRotation(16, 1000.0, _STRETCH(8.0, 64, 4.0, 1.0)), 13),
                         MixtureSizes(24, 10, 3, 2.0)),
            ZuvasunLayer("attention", KeyValueSizes(4, 4, 32, 0.1), None),
            ZuvasunLayer("latent_attention", SharedLatentSizes(5, 8, 16, 16, 32, 0.3, PairRotation(16, 1000.0, _STRETCH(8.0, 64, 4.0, 1.0)), 22, kv_from=1),
                         MixtureSizes(24, 10, 3, 2.0)),
        ),
    ),
    "zuvasun_tiny_b": ZuvasunConfig(
        vocab=170, width=64, eps=1e-6,
        layers=(
            ZuvasunLayer("latent_attention", SharedLatentSizes(2, 32, 8, 16, 24, 0.15, PairRotation(6, 1e4), None), None),
            ZuvasunLayer("latent_attention", SharedLatentSizes(4, 16, 8, 32, 24, 0.25, PairRotation(6, 1e4), 9, kv_from=0),
                         MixtureSizes(32, 5, 1, 1.0)),
            ZuvasunLayer("attention", KeyValueSizes(2, 1, 48, 0.12, 1.0, 1), MixtureSizes(48, 4, 4, 0.5)),
        ),
    ),
}
PRESET_PAGE_SIZE = {"zuvasun_tiny_a": 16, "zuvasun_tiny_b": 8}


def sized(width: int, layers: int, heads: int, kv_heads: int, dim: int, vocab: int, *, expert_ff: int, experts: int = 16,
          top: int = 2, window: int = 2048, kv_rank: int = 384, rot_dim: int = 64) -> ZuvasunConfig:
    """A configuration of the sizes of a real model, for measurements: a latent layer, a latent layer
    that reads the first one's cache, and two layers whose values are their keys, in turn; a
    mixture in every layer."""
    rot = PairRotation(rot_dim, 1e6, _STRETCH(8.0, 4096, 16.0, 1.0))
    own = SharedLatentSizes(heads, dim, rot_dim, dim, kv_rank, (dim + rot_dim) ** -0.5, rot, window)
    att = KeyValueSizes(heads, kv_heads, dim, dim ** -0.5, 0.1, 1024)
    ff = MixtureSizes(expert_ff, experts, top, 1.0)
    out = []
    for i in range(layers):
        if i % 4 == 1:
            out.append(ZuvasunLayer("latent_attention", SharedLatentSizes(heads, dim, rot_dim, dim, kv_rank, own.scale, rot, window,
                                                                          kv_from=i - 1), ff))
        else:
            out.append(ZuvasunLayer("latent_attention" if i % 4 == 0 else "attention", own if i % 4 == 0 else att, ff))
    return ZuvasunConfig(vocab=vocab, width=width, eps=1e-5, layers=tuple(out))


register_architecture(ZuvasunConfig.architecture, ZuvasunConfig.from_dict, plan_zuvasun)
for _name, _cfg in PRESETS.items():
    register_preset(_name, _cfg.to_dict(), PRESET_PAGE_SIZE.get(_name, 16))
# layers of the sizes of the 4B and 8B dense presets, and of a smaller width, with a mixture like
# `roserax_4b`'s in every layer, for measurements beside it
register_preset("zuvasun_4b", sized(2560, 36, 32, 8, 128, 151936, expert_ff=1536).to_dict(), 16)
register_preset("zuvasun_8b", sized(4096, 36, 32, 8, 128, 151936, expert_ff=2048, kv_rank=448).to_dict(), 16)
register_preset("zuvasun_2b", sized(2048, 28, 16, 4, 128, 151936, expert_ff=1024, kv_rank=256).to_dict(), 16)
