"""Plain, slow Roserax decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the engine: it reads config.json and the safetensors file itself and
works on one whole sequence at a time in ``dtype`` (float64 unless asked otherwise).

The design in short. One residual stream that starts as the embedding times a constant. Every
sub-layer is normed on both sides: ``x <- x + norm_after(f(norm_before(x)))``, RMS norms with plain
weights. Three mixers: softmax attention over a sliding window that also keeps the first few
tokens of the sequence in sight, with normed queries and keys, no rotation, and a softmax whose
denominator carries one more term of one (a sink without a value); attention through a latent
(queries and keys/values each squeezed through a low-rank vector, part of every head rotated, the
rotated key part shared by all heads, an output gate); and retention (linear attention with a fixed
decay per head, rotated queries and keys, the read-out normed per head and gated). Feed-forwards are
dense with a squared relu, or a routed mixture of silu-gated experts chosen from the best groups
by softmax scores that are not renormalised. The head is the embedding table, the logits times a
constant.
"""

from __future__ import annotations

import json
import math
from pathlib import Path

import torch


def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last dimension (no weight: None)."""
    y = x / torch.sqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotate_half(x, positions, dims, base):
    """x [T, heads, D]: the first ``dims`` elements of every head turn, element i against element
    i + dims/2, by the angle position * base^(-2i/dims); the rest passes."""
    if dims == 0:
        return x
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = base ** (-2.0 * i / dims)
    ang = torch.as_tensor(positions, dtype=x.dtype)[:, None] * freq[None, :]
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def window_mask(t, size, keep_first):
    """[T, T] bool: query i sees key j iff j <= i and (i - j < size or j < keep_first)."""
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def softmax_with_sink(scores, mask):
    """p_j = exp(s_j) / (1 + sum_visible exp(s_j)): one more term in the denominator, of score 0."""
    s = scores.masked_fill(~mask, float("-inf"))
    m = torch.clamp(s.amax(dim=-1, keepdim=True), min=0.0)  # the sink's score takes part in the maximum
    e = torch.exp(s - m)
    return e / (torch.exp(-m) + e.sum(dim=-1, keepdim=True))


def window_attention(h, w, sizes, eps):
    """The mixer 'attention'. h [T, width]."""
    t = h.shape[0]
    nq, d = sizes["heads"], sizes["dim"]
    nkv, dv = sizes.get("kv_heads", nq), sizes.get("vdim", d)
    q = rms_norm((h @ w["q"].T).view(t, nq, d), w["q.norm"], eps)
    k = rms_norm((h @ w["k"].T).view(t, nkv, d), w["k.norm"], eps)
    v = (h @ w["v"].T).view(t, nkv, dv)
    g = nq // nkv
    k, v = k.repeat_interleave(g, dim=1), v.repeat_interleave(g, dim=1)
    scores = torch.einsum("qhd,khd->hqk", q, k) * sizes["scale"]
    mask = window_mask(t, sizes["mask"]["size"], sizes["mask"].get("keep_first", 0))
    p = softmax_with_sink(scores, mask[None])
    out = torch.einsum("hqk,khd->qhd", p, v).reshape(t, nq * dv)
    return out @ w["o"].T


def latent_attention(h, w, sizes, eps):
    """The mixer 'latent_attention'."""
    t = h.shape[0]
    nq, d, r, dv, rank = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    rot = sizes["rot"]
    pos = list(range(t))
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).view(t, nq, d + r)
    q_plain, q_rot = q[..., :d], rotate_half(q[..., d:], pos, rot["dims"], rot["base"])
    down = h @ w["dkv"].T
    c = rms_norm(down[:, :rank], w["dkv.norm"], eps)
    k_rot = rotate_half(down[:, None, rank:], pos, rot["dims"], rot["base"])[:, 0]  # one part for all heads
    k_plain = (c @ w["uk"].T).view(t, nq, d)
    v = (c @ w["uv"].T).view(t, nq, dv)
    scores = (torch.einsum("qhd,khd->hqk", q_plain, k_plain) + torch.einsum("qhr,kr->hqk", q_rot, k_rot)) * sizes["scale"]
    causal = torch.arange(t)[None, :] <= torch.arange(t)[:, None]
    p = torch.softmax(scores.masked_fill(~causal[None], float("-inf")), dim=-1)
    out = torch.einsum("hqk,khd->qhd", p, v).reshape(t, nq * dv)
    out = out * torch.sigmoid(h @ w["g"].T)
    return out @ w["o"].T


def retention_head(q, k, v, decay):
    """One head, token by token: S <- decay S + k v^T; o = S^T q. q, k [T, D]; v [T, Dv]."""
    s = q.new_zeros(k.shape[1], v.shape[1])
    out = []
    for i in range(q.shape[0]):
        s = decay * s + torch.outer(k[i], v[i])
        out.append(s.T @ q[i])
    return torch.stack(out)


def retention(h, w, sizes, eps):
    """The mixer 'retention'."""
    t = h.shape[0]
    n, d = sizes["heads"], sizes["dim"]
    dv = sizes.get("vdim", d)
    rot = sizes["rot"]
    pos = list(range(t))
    q = rotate_half((h @ w["q"].T).view(t, n, d), pos, rot["dims"], rot["base"])
    k = rotate_half((h @ w["k"].T).view(t, n, d), pos, rot["dims"], rot["base"]) * d ** -0.5
    v = (h @ w["v"].T).view(t, n, dv)
    o = torch.stack([retention_head(q[:, j], k[:, j], v[:, j], sizes["decay"][j]) for j in range(n)], dim=1)
    o = rms_norm(o, None, eps).reshape(t, n * dv)
    z = h @ w["g"].T
    return (o * z * torch.sigmoid(z)) @ w["o"].T


def dense_ff(h, w):
    """down(relu(up h)^2)."""
    return torch.relu(h @ w["up"].T).pow(2) @ w["down"].T


def route(h, router, top, groups, keep):
    """(index [T, top], weight [T, top]): softmax over all experts; a group's score is its largest
    score; the ``top`` largest scores among the experts of the ``keep`` best groups, as they are."""
    s = torch.softmax(h @ router.T, dim=-1)
    t, e = s.shape
    pick = s
    if groups > 1 and keep < groups:
        per = e // groups
        best = s.view(t, groups, per).amax(dim=-1)
        stay = torch.zeros(t, groups, dtype=torch.bool)
        stay.scatter_(1, torch.topk(best, keep, dim=-1).indices, True)
        pick = s.masked_fill(~stay.repeat_interleave(per, dim=1), float("-inf"))
    index = torch.topk(pick, top, dim=-1).indices
    return index, torch.gather(s, 1, index)


def mixture(h, w, mlp):
    """Sum over the chosen experts of score * down(silu(gate h) * (up h))."""
    router = mlp["router"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    index, weight = route(h, w["router"], router["top"], groups["count"], groups["keep"])
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for j in range(index.shape[1]):
            e = int(index[i, j])
            z = w[f"e{e}.gate"] @ h[i]
            out[i] += weight[i, j] * (w[f"e{e}.down"] @ (z * torch.sigmoid(z) * (w[f"e{e}.up"] @ h[i])))
    return out


def feed_forward(h, w, mlp):
    if mlp["kind"] == "dense":
        return dense_ff(h, w)
    if mlp["kind"] == "moe":
        return mixture(h, w, mlp)
    raise ValueError(mlp["kind"])


MIXERS = {"attention": window_attention, "latent_attention": latent_attention, "retention": retention}


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
    x = weights["embed"][torch.as_tensor(ids, dtype=torch.long)] * cfg.get("embedding", {}).get("scale", 1.0)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        w = sub(weights, f"l{i}.")
        y = MIXERS[layer["type"]](rms_norm(x, w["norm1"], eps), sub(w, "mix."), layer["mixer"], eps)
        x = x + rms_norm(y, w["norm1b"], eps)
        if layer.get("mlp"):
            y = feed_forward(rms_norm(x, w["norm2"], eps), sub(w, "mlp."), layer["mlp"])
            x = x + rms_norm(y, w["norm2b"], eps)
        after.append(x)
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["embed"].T * cfg.get("logit_scale", 1.0)
    return (logits, torch.stack(after)) if return_layers else logits


def load(folder, dtype=torch.float64):
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    return cfg, read_safetensors(folder / "model.safetensors", dtype)
