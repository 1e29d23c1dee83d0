"""Plain, slow Zuvasun decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the engine: it reads config.json and the safetensors file itself and
works on one whole sequence at a time in ``dtype`` (float64 unless asked otherwise).

The design in short. One residual stream. A layer has one RMS norm whose output both of its
sub-layers read; their outputs, each times a vector of its own, join the stream in one sum:
``x <- x + s1 * mixer(n) + s2 * ff(n)`` with ``n = norm(x)``. Two mixers: attention through a
latent (full-rank queries; keys and values made from a low-rank vector, one rotated key part
shared by all heads; rotation of neighbouring pairs with frequencies stretched as YaRN does;
a sliding window; a layer may read another layer's latent instead of making its own) and
grouped-query attention without rotation whose values are its keys as projected, with
biases, one RMS norm over all heads of the queries and one over all heads of the keys, and
queries that grow with the logarithm of the position. The feed-forward is a mixture of
squared-relu experts: softmax scores over all experts, the choice made on scores plus a
correction, the chosen scores renormalised and scaled.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last dimension."""
    y = x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def yarn_frequencies(dims, base, scaling, dtype=torch.float64):
    """(frequencies [dims/2], factor of cos and sin). Without ``scaling``: base^(-2i/dims) and 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f.to(dtype), 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_to_dim(turns):  # the (fractional) pair whose wave makes ``turns`` turns over the original length
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_to_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_to_dim(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f.to(dtype), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, dims, base, scaling):
    """x [T, heads, D]: of the first ``dims`` elements of every head, element 2i turns against
    element 2i+1 by position * f_i; the rest passes. cos and sin carry YaRN's factor."""
    if dims == 0:
        return x
    f, mag = yarn_frequencies(dims, base, scaling, x.dtype)
    ang = torch.as_tensor(positions, dtype=x.dtype)[:, None] * f[None, :]
    cos, sin = ang.cos()[:, None, :] * mag, ang.sin()[:, None, :] * mag
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).flatten(-2)
    return torch.cat([turned, x[..., dims:]], dim=-1)


def visible(t, window):
    """[T, T] bool: query i sees key j iff 0 <= i - j (< window, if there is one)."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    m = j <= i
    return m if window is None else m & (i - j < window)


def latent_keys(h, w, sizes, eps):
    """What a latent layer makes for itself and for layers that read it: the normed latent
    c [T, kv_rank] and the rotated key part [T, rot_dim]."""
    rank, rot = sizes["kv_rank"], sizes["rot"]
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :rank], w["dkv.norm"], eps)
    k_rot = rotate_pairs(down[:, None, rank:], range(h.shape[0]), rot["dims"], rot["base"], rot.get("scaling"))[:, 0]
    return c, k_rot


def latent_attention(h, w, sizes, eps, shared=None):
    """The mixer 'latent_attention'. ``shared``: (c, k_rot) of the layer named by ``kv_from``."""
    t = h.shape[0]
    n, d, r, dv = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"]
    rot = sizes["rot"]
    c, k_rot = latent_keys(h, w, sizes, eps) if shared is None else shared
    q = (h @ w["q"].T).view(t, n, d + r)
    q_plain = q[..., :d]
    q_rot = rotate_pairs(q[..., d:], range(t), rot["dims"], rot["base"], rot.get("scaling"))
    k_plain = (c @ w["uk"].T).view(t, n, d)
    v = (c @ w["uv"].T).view(t, n, dv)
    scores = (torch.einsum("qhd,khd->hqk", q_plain, k_plain) + torch.einsum("qhr,kr->hqk", q_rot, k_rot)) * sizes["scale"]
    mask = visible(t, (sizes.get("mask") or {}).get("size"))
    p = torch.softmax(scores.masked_fill(~mask[None], float("-inf")), dim=-1)
    out = torch.einsum("hqk,khd->qhd", p, v).reshape(t, n * dv)
    return out @ w["o"].T, (c, k_rot)


def query_temperature(t, coef, every, dtype):
    """[T]: 1 + coef * ln(floor((p + 1) / every) + 1)."""
    p = torch.arange(t, dtype=torch.float64)
    return (1.0 + coef * torch.log(torch.floor((p + 1.0) / every) + 1.0)).to(dtype)


def key_value_attention(h, w, sizes, eps):
    """The mixer 'attention': the values are the keys as projected."""
    t = h.shape[0]
    nq, d = sizes["heads"], sizes["dim"]
    nkv = sizes.get("kv_heads", nq)
    q = h @ w["q"].T + w["q.b"]
    k = h @ w["k"].T + w["k.b"]
    v = k.view(t, nkv, d)
    q = rms_norm(q, w["q.norm"], eps)  # one norm over all heads' rows
    k = rms_norm(k, w["k.norm"], eps).view(t, nkv, d)
    temp = sizes.get("q_temp")
    if temp:
        q = q * query_temperature(t, temp["coef"], temp["every"], q.dtype)[:, None]
    q = q.view(t, nq, d)
    g = nq // nkv
    k, v = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * sizes["scale"]
    p = torch.softmax(scores.masked_fill(~visible(t, None)[None], float("-inf")), dim=-1)
    return torch.einsum("hqk,khd->qhd", p, v).reshape(t, nq * d) @ w["o"].T


def route(h, router, correction, top, scale):
    """(index [T, top], weight [T, top]): softmax over all experts; the ``top`` largest of score +
    correction are chosen; their scores, divided by their sum, times ``scale``."""
    s = torch.softmax(h @ router.T, dim=-1)
    index = torch.topk(s + correction, top, dim=-1).indices
    chosen = torch.gather(s, 1, index)
    return index, chosen / (chosen.sum(dim=-1, keepdim=True) + 1e-20) * scale


def mixture(h, w, mlp):
    """Sum over the chosen experts of weight * down(relu(up h)^2)."""
    router = mlp["router"]
    index, weight = route(h, w["router"], w["correction"], router["top"], router.get("scale", 1.0))
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for j in range(index.shape[1]):
            e = int(index[i, j])
            out[i] += weight[i, j] * (w[f"e{e}.down"] @ torch.relu(w[f"e{e}.up"] @ h[i]).pow(2))
    return out


def read_safetensors(path, dtype=torch.float64):
    raw = Path(path).read_bytes()
    n = int.from_bytes(raw[:8], "little")
    header = json.loads(raw[8: 8 + n])
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32}
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        a, b = meta["data_offsets"]
        t = torch.frombuffer(bytearray(raw[8 + n + a: 8 + n + b]), dtype=kinds[meta["dtype"]]).view(meta["shape"])
        out[name] = t if meta["dtype"] == "I32" else t.to(dtype)
    return out


def sub(weights, prefix):
    return {n[len(prefix):]: x for n, x in weights.items() if n.startswith(prefix)}


def forward(cfg, weights, ids, return_layers=False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer)."""
    eps = cfg["norm"]["eps"]
    x = weights["embed"][torch.as_tensor(ids, dtype=torch.long)]
    after, latents = [], {}
    for i, layer in enumerate(cfg["layers"]):
        w = sub(weights, f"l{i}.")
        n = rms_norm(x, w["norm1"], eps)
        if layer["type"] == "latent_attention":
            src = layer["mixer"].get("kv_from")
            y, latents[i] = latent_attention(n, sub(w, "mix."), layer["mixer"], eps, None if src is None else latents[src])
        elif layer["type"] == "attention":
            y = key_value_attention(n, sub(w, "mix."), layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        y = y * w["ls1"]
        if layer.get("mlp"):
            if layer["mlp"]["kind"] != "moe":
                raise ValueError(layer["mlp"]["kind"])
            y = y + mixture(n, sub(w, "mlp."), layer["mlp"]) * w["ls2"]
        x = x + y
        after.append(x)
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["head"].T
    return (logits, torch.stack(after)) if return_layers else logits


def load(folder, dtype=torch.float64):
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    return cfg, read_safetensors(folder / "model.safetensors", dtype)
