"""Plain torch version of every device op, one function per kernel.

Two uses: the GPU tests compare each HIP kernel alone with its function here,
and ``TorchOps`` lets the host-side tests drive the engine (cache manager,
step function, scheduler) on the CPU, where no kernel can run. The engine
itself never imports this file: its only ops are the HIP ones.

Arithmetic inside each op is float32 (or ``compute``), results are cast to the
output type, as the kernels do. The cache layout is the engine's: keys
``[page, head, offset, D]``, values ``[page, head, D, offset]``.
"""

from __future__ import annotations

import math

import torch


def embed(ids, table, scale=1.0):
    x = table[ids.long()].to(torch.float32)
    return x if scale == 1.0 else x * scale


def add_rmsnorm(residual, delta, weight, eps, out_dtype, rows=None, compute=torch.float32, delta_scale=1.0,
                delta_norm=None):
    if delta is not None and delta.dim() == 3:
        delta = delta.to(residual.dtype).sum(0)
    if delta_norm is not None:  # the pending output is normed on its way into the stream
        after_w, after_eps = delta_norm
        d = delta.to(torch.float32)
        delta = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + after_eps) * after_w
    if delta is not None and delta_scale != 1.0:
        delta = delta.to(residual.dtype) * delta_scale
    if delta is not None:
        if rows is None:
            residual += delta.to(residual.dtype)
            x = residual
        else:
            x = residual[rows.long()] + delta[rows.long()].to(residual.dtype)
    else:
        x = residual if rows is None else residual[rows.long()]
    x = x.to(compute)
    var = x.pow(2).mean(dim=-1, keepdim=True)
    return (x * torch.rsqrt(var + eps) * weight.to(compute)).to(out_dtype)


def linear(x, w, out_f32=False, compute=torch.float32):
    y = x.to(compute) @ w.to(compute).T
    return y.to(torch.float32 if out_f32 else x.dtype)


def head_rmsnorm(x, weight, eps, compute=torch.float32):
    x = x.to(compute)
    if weight is None:
        return x
    return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight.to(compute)


def rope_rotate(x, positions, inv_freq, compute=torch.float32):
    """x [T, heads, D] (compute dtype); angles = float32(pos) * inv_freq in float32."""
    d = x.shape[-1]
    ang = (positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]).to(compute)
    cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)


def qk_norm_split(qkv, nq, nkv, d, q_w, k_w, eps, compute=torch.float32):
    t = qkv.shape[0]
    q = qkv[:, : nq * d].reshape(t, nq, d)
    k = qkv[:, nq * d: (nq + nkv) * d].reshape(t, nkv, d)
    v = qkv[:, (nq + nkv) * d:].reshape(t, nkv, d)
    q = head_rmsnorm(q, q_w, eps, compute).to(qkv.dtype)
    k = head_rmsnorm(k, k_w, eps, compute).to(qkv.dtype)
    return q, k, v.contiguous()


def kv_store(k, v, k_cache, v_cache, slots, page_size):
    """k, v: [T, heads, D]; slot = page * page_size + offset."""
    pages = (slots // page_size).long()
    offs = (slots % page_size).long()
    k_cache[pages, :, offs, :] = k.to(k_cache.dtype)
    v_cache[pages, :, :, offs] = v.to(v_cache.dtype)


def qk_norm_rope_store(qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions,
                       k_cache=None, v_cache=None, slots=None, page_size=None, compute=torch.float32,
                       value_dim=None):
    t = qkv.shape[0]
    dv = d if value_dim is None else value_dim
    q = qkv[:, : nq * d].reshape(t, nq, d)
    k = qkv[:, nq * d: (nq + nkv) * d].reshape(t, nkv, d)
    v = qkv[:, (nq + nkv) * d: (nq + nkv) * d + nkv * dv].reshape(t, nkv, dv)
    q = head_rmsnorm(q, q_w, eps, compute)
    k = head_rmsnorm(k, k_w, eps, compute)
    if inv_freq is not None:
        q = rope_rotate(q, positions, inv_freq, compute)
        k = rope_rotate(k, positions, inv_freq, compute)
    if k_cache is not None:
        kv_store(k, v, k_cache, v_cache, slots, page_size)
    return q.to(qkv.dtype).reshape(t, nq * d)


def gather_kv(k_cache, v_cache, table_row, lo, hi, page_size):
    """Keys and values of positions lo..hi-1 of one sequence: [hi-lo, heads, D] each."""
    pos = torch.arange(lo, hi, device=k_cache.device)
    pages = table_row.long()[pos // page_size]
    offs = pos % page_size
    if (pages < 0).any():
        raise AssertionError("attention reads a position whose page was given back")
    k = k_cache[pages, :, offs, :]
    v = v_cache[pages, :, :, offs]
    return k, v


def paged_attention(q, k_cache, v_cache, cu_q, kv_lens, block_table, page_size, nq, nkv, d,
                    scale, window=None, compute=torch.float32, round_probs=False, chunk=None, softcap=None,
                    value_dim=None, gate=None, keep_first=0, sink=False):
    """q [T, nq*D] -> [T, nq*Dv]. ``keep_first``: beside a window the sequence's first tokens stay
    visible; ``sink``: one more term of score 0 in the softmax's denominator.
    Query row i of a sequence sits at position
    kv_len - q_len + i and sees keys j <= its position (and > position - window, or, with
    ``chunk``, in its own chunk of positions). ``softcap``: scores become cap * tanh(score / cap).
    ``gate`` [T, nq*Dv]: the output is multiplied by its sigmoid."""
    dv = d if value_dim is None else value_dim
    out = torch.zeros((q.shape[0], nq * dv), dtype=q.dtype, device=q.device)
    g = nq // nkv
    cu = [int(x) for x in cu_q]
    for s in range(len(cu) - 1):
        a, b = cu[s], cu[s + 1]
        q_len, kv_len = b - a, int(kv_lens[s])
        if q_len == 0 or kv_len == 0:
            continue
        first_pos = kv_len - q_len
        lo = 0 if window is None or keep_first else max(0, first_pos - window + 1)
        if chunk is not None:
            lo = first_pos - first_pos % chunk
        qpos = torch.arange(first_pos, kv_len, device=q.device)[:, None]
        kpos = torch.arange(lo, kv_len, device=q.device)[None, :]
        ok = kpos <= qpos
        if window is not None:
            ok = ok & ((kpos > qpos - window) | (kpos < keep_first))
        if chunk is not None:
            ok = ok & (kpos // chunk == qpos // chunk)
        if keep_first and window is not None:
            # the pages between the kept tokens and the window may be gone: read only what some row sees
            idx = ok.any(dim=0).nonzero()[:, 0]
            pos_seen = kpos[0, idx]
            pages = block_table[s].long()[pos_seen // page_size]
            if (pages < 0).any():
                raise AssertionError("attention reads a position whose page was given back")
            k = torch.zeros((kv_len - lo, nkv, d), dtype=k_cache.dtype, device=q.device)
            v = torch.zeros((kv_len - lo, nkv, dv), dtype=v_cache.dtype, device=q.device)
            k[idx] = k_cache[pages, :, pos_seen % page_size, :]
            v[idx] = v_cache[pages, :, :, pos_seen % page_size]
        else:
            k, v = gather_kv(k_cache, v_cache, block_table[s], lo, kv_len, page_size)
        k = k.to(compute).repeat_interleave(g, dim=1)
        v = v.to(compute).repeat_interleave(g, dim=1)
        qs = q[a:b].reshape(q_len, nq, d).to(compute)
        scores = torch.einsum("qhd,khd->hqk", qs, k) * scale
        if softcap is not None:
            scores = softcap * torch.tanh(scores / softcap)
        scores = scores.masked_fill(~ok, float("-inf"))
        if sink:
            m = torch.clamp(scores.amax(dim=-1, keepdim=True), min=0.0)
            e = torch.exp(scores - m)
            probs = e / (torch.exp(-m) + e.sum(dim=-1, keepdim=True))
        else:
            probs = torch.softmax(scores, dim=-1)
        if round_probs:
            probs = probs.to(q.dtype).to(compute)
        ctx = torch.einsum("hqk,khd->qhd", probs, v).reshape(q_len, nq * dv)
        if gate is not None:
            ctx = ctx * torch.sigmoid(gate[a:b].to(compute))
        out[a:b] = ctx.to(q.dtype)
    return out


def mix_norm(streams, update, read, weight, bias, eps, out_dtype, rows=None, compute=torch.float32):
    """Residual streams [T, S, H] (or one stream [T, H]) float32. ``update``: None, a plain delta
    (one stream only), or an object with ``y`` [T, H] (or planes [P, T, H]), ``mix`` [S, S]
    (indexed [from, to]) and ``out`` [S]: new[:, t] = sum_s mix[s, t] old[:, s] + out[t] y,
    written back unless ``rows`` is given. Returns the norm (layer norm with ``bias``, RMS norm
    without) of sum_t read[t] new[:, t] at the rows asked for."""
    one = streams.dim() == 2
    x = streams[:, None, :] if one else streams
    new = x
    if update is not None:
        if hasattr(update, "y"):
            y, mix, out = update.y, update.mix, update.out
        else:
            y, mix, out = update, None, None
        if y.dim() == 3:
            y = y.to(torch.float32).sum(0)
        y = y.to(torch.float32)
        new = x if mix is None else torch.einsum("sr,tsh->trh", mix.to(torch.float32), x)
        new = new + (y[:, None, :] if out is None else out.to(torch.float32)[None, :, None] * y[:, None, :])
        if rows is None:
            x.copy_(new)
    u = new[:, 0] if read is None else torch.einsum("s,tsh->th", read.to(torch.float32), new)
    if rows is not None:
        u = u[rows.long()]
    u = u.to(compute)
    if bias is None:
        y = u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * weight.to(compute)
    else:
        mu = u.mean(-1, keepdim=True)
        var = (u - mu).pow(2).mean(-1, keepdim=True)
        y = (u - mu) * torch.rsqrt(var + eps) * weight.to(compute) + bias.to(compute)
    return y.to(out_dtype)


def route_top(x, router, router_bias, top, scoring="softmax_top", groups=1, keep=None, group_score="top2",
              correction=None, renormalise=False, weight_scale=1.0):
    """float32 logits x W^T + b; the ``top`` largest per token (ties: the lower index first) and
    the softmax over those alone. Returns (int32 [T, top], float32 [T, top]). With sigmoid scoring
    the scores are the weights; with groups only the best ``keep`` groups' experts can be chosen.
    ``correction`` [E] is added to the scores for the choice alone; ``renormalise`` divides the chosen
    scores by their sum (+ 1e-20); ``weight_scale`` multiplies the weights at the end."""
    logits = x.to(torch.float32) @ router.to(torch.float32).T
    if router_bias is not None:
        logits = logits + router_bias.to(torch.float32)
    values = torch.sigmoid(logits) if scoring == "sigmoid" else \
        torch.softmax(logits, dim=-1) if scoring == "softmax_all" else logits
    pick = values if correction is None else values + correction.to(torch.float32)
    if groups > 1 and keep is not None and keep < groups:
        if correction is not None:
            raise NotImplementedError("groups of experts beside a correction of the choice")
        t, e = values.shape
        per = e // groups
        g = values.view(t, groups, per)
        gscore = g.amax(dim=-1) if group_score == "max" else torch.topk(g, min(2, per), dim=-1).values.sum(-1)
        stay = torch.zeros(t, groups, dtype=torch.bool, device=x.device)
        stay.scatter_(1, torch.topk(gscore, keep, dim=-1).indices, True)
        pick = torch.where(stay[:, :, None].expand(t, groups, per).reshape(t, e), values,
                           torch.full_like(values, float("-inf")))
    best, index = torch.topk(pick, top, dim=-1)
    if scoring == "softmax_top":
        return index.to(torch.int32), torch.softmax(best, dim=-1)
    weight = torch.gather(values, 1, index)
    if renormalise:
        weight = weight / (weight.sum(-1, keepdim=True) + 1e-20)
    return index.to(torch.int32), weight * weight_scale if weight_scale != 1.0 else weight


def gated(g, u, activation="swiglu", limit=0.0):
    if activation == "clamped":
        g = torch.clamp(g, max=limit)
        u = torch.clamp(u, min=-limit, max=limit)
        return g * torch.sigmoid(1.702 * g) * (u + 1)
    return g * torch.sigmoid(g) * u


def moe_swiglu(x, gate_up, down, index, weight, compute=torch.float32, activation="swiglu", limit=0.0):
    """x [T, H]; gate_up [E, 2I, H]; down [E, H, I]; index/weight [T, top] -> [T, H] (float32)."""
    t, h = x.shape
    inter = gate_up.shape[1] // 2
    out = torch.zeros((t, h), dtype=torch.float32, device=x.device)
    xc = x.to(compute)
    for j in range(index.shape[1]):
        for e in index[:, j].unique().tolist():
            sel = (index[:, j] == e).nonzero()[:, 0]
            gu = (xc[sel] @ gate_up[e].to(compute).T).to(x.dtype).to(compute)
            if activation == "relu2":  # no gate: the tensor holds the up rows alone
                act = torch.relu(gu).pow(2).to(x.dtype).to(compute)
            else:
                act = gated(gu[:, :inter], gu[:, inter:], activation, limit).to(x.dtype).to(compute)
            out[sel] += weight[sel, j, None] * (act @ down[e].to(compute).T).to(torch.float32)
    return out


def swiglu(gate_up, compute=torch.float32):
    i = gate_up.shape[-1] // 2
    g, u = gate_up[..., :i].to(compute), gate_up[..., i:].to(compute)
    return (g * torch.sigmoid(g) * u).to(gate_up.dtype)


def planes_sum(y):
    return y.to(torch.float32).sum(0) if y.dim() == 3 else y.to(torch.float32)


def norm_mean(ya, wa, yb, wb, eps):
    def normed(y, w):
        y = planes_sum(y)
        return y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps) * w
    return 0.5 * (normed(ya, wa) + normed(yb, wb))


def bias_rotate_pairs(x, bias, positions, freq, rot_heads, head_dim):
    t, w = x.shape
    y = x.to(torch.float32)
    if bias is not None:
        y = y + bias
    if freq is not None and freq.numel():
        n = freq.numel()
        heads = y[:, : rot_heads * head_dim].reshape(t, rot_heads, head_dim).clone()
        ang = positions.to(torch.float32)[:, None] * freq[None, :]
        cos, sin = ang.cos()[:, None, :], ang.sin()[:, None, :]
        a, b = heads[..., 0: 2 * n: 2].clone(), heads[..., 1: 2 * n: 2].clone()
        heads[..., 0: 2 * n: 2] = a * cos - b * sin
        heads[..., 1: 2 * n: 2] = b * cos + a * sin
        y = torch.cat([heads.reshape(t, -1), y[:, rot_heads * head_dim:]], dim=1)
    x.copy_(y.to(x.dtype))
    return x


def delta_conv(y, channels, taps, tail, cu_q, slots, segments, unit_eps):
    """Causal convolution + silu + unit vectors per head, span by span; ``tail`` updated in place."""
    k = taps.shape[1]
    out = torch.empty((y.shape[0], channels), dtype=torch.float32, device=y.device)
    for s in range(len(cu_q) - 1):
        a, b = int(cu_q[s]), int(cu_q[s + 1])
        slot = int(slots[s])
        x = y[a:b, :channels].to(torch.float32)
        full = torch.cat([tail[slot, :, : k - 1].T, x], dim=0) if k > 1 else x
        acc = torch.zeros_like(x)
        for j in range(k):
            acc = acc + full[j: j + (b - a)] * taps[:, j]
        out[a:b] = acc * torch.sigmoid(acc)
        if k > 1:
            tail[slot, :, : k - 1] = full[full.shape[0] - (k - 1):].T
    first = 0
    for heads, width, mode in segments:
        if mode:
            seg = out[:, first: first + heads * width].view(-1, heads, width)
            seg = seg / torch.sqrt(seg.pow(2).sum(-1, keepdim=True) + unit_eps)
            if mode == 2:
                seg = seg * width ** -0.5
            out[:, first: first + heads * width] = seg.reshape(-1, heads * width)
        first += heads * width
    return out


def delta_rule(qkv, beta, a_logits, a_log, dt_bias, state, cu_q, slots, heads, kv_heads, dim, vdim, per_channel):
    t = qkv.shape[0]
    q = qkv[:, : kv_heads * dim].view(t, kv_heads, dim)
    k = qkv[:, kv_heads * dim: 2 * kv_heads * dim].view(t, kv_heads, dim)
    v = qkv[:, 2 * kv_heads * dim:].view(t, heads, vdim)
    b = torch.sigmoid(beta.to(torch.float32))
    sp = torch.nn.functional.softplus(a_logits.to(torch.float32) + dt_bias)
    rate = torch.exp(a_log)
    g = torch.exp(-rate[None, :, None] * sp.view(t, heads, dim)) if per_channel else torch.exp(-rate[None, :] * sp)
    out = torch.empty((t, heads, vdim), dtype=torch.float32, device=qkv.device)
    group = heads // kv_heads
    for s in range(len(cu_q) - 1):
        slot = int(slots[s])
        for h in range(heads):
            st = state[slot, h].T.clone()  # [dim, vdim]
            for i in range(int(cu_q[s]), int(cu_q[s + 1])):
                st = st * (g[i, h][:, None] if per_channel else g[i, h])
                u = b[i, h] * (v[i, h] - st.T @ k[i, h // group])
                st = st + torch.outer(k[i, h // group], u)
                out[i, h] = st.T @ q[i, h // group]
            state[slot, h] = st.T
    return out


def delta_out(o, weight, gate, eps, gate_kind, out_dtype):
    t, heads, vdim = o.shape
    z = gate.to(torch.float32).reshape(t, heads, vdim)
    act = z * torch.sigmoid(z) if gate_kind == "silu" else torch.sigmoid(z)
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * weight * act
    return y.reshape(t, heads * vdim).to(out_dtype)


def argmax(logits):
    return torch.argmax(logits, dim=-1).to(torch.int32)


def rotate_half_copy(x, in_stride, in_offset, out, out_stride, out_offset, heads, width, positions, freq,
                     neighbours=False, magnitude=1.0):
    """For every token and head copy ``width`` elements from ``x[t, h * in_stride + in_offset ...]`` to
    ``out[t, h * out_stride + out_offset ...]``, the first ``2 len(freq)`` of them turned: element i
    against element i + len(freq) (``neighbours``: element 2i against element 2i + 1), by
    ``position * freq[i]`` (float32 angles), cosines and sines times ``magnitude``."""
    t = x.shape[0]
    src = x[:, : heads * in_stride].reshape(t, heads, in_stride)[:, :, in_offset: in_offset + width].to(torch.float32)
    n = 0 if freq is None else freq.numel()
    if n:
        ang = positions.to(torch.float32)[:, None] * freq.to(torch.float32)[None, :]
        cos, sin = ang.cos()[:, None, :] * magnitude, ang.sin()[:, None, :] * magnitude
        if neighbours:
            u, v = src[..., 0: 2 * n: 2], src[..., 1: 2 * n: 2]
            turned = torch.stack([u * cos - v * sin, v * cos + u * sin], dim=-1).flatten(-2)
            src = torch.cat([turned, src[..., 2 * n:]], dim=-1)
        else:
            u, v = src[..., :n], src[..., n: 2 * n]
            src = torch.cat([u * cos - v * sin, v * cos + u * sin, src[..., 2 * n:]], dim=-1)
    out[:, : heads * out_stride].view(t, heads, out_stride)[:, :, out_offset: out_offset + width] = src.to(out.dtype)
    return out


def rmsnorm_columns(y, first, width, weight, eps):
    x = y[:, first: first + width].to(torch.float32)
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * weight).to(y.dtype)


def latent_store(y, first, rank, rot_dim, weight, eps, positions, freq, k_cache, v_cache, slots, page_size,
                 neighbours=False, magnitude=1.0):
    """Columns ``first .. first + rank`` of ``y`` RMS-normed (the latent) and the ``rot_dim`` behind them
    rotated: the key row ``[c | k_rot]`` and the value row ``[c | 0]`` of one key/value head."""
    t = y.shape[0]
    c = rmsnorm_columns(y, first, rank, weight, eps).to(torch.float32)
    rot = torch.empty((t, rot_dim), dtype=torch.float32, device=y.device)
    rotate_half_copy(y[:, first + rank: first + rank + rot_dim].contiguous(), rot_dim, 0, rot, rot_dim, 0, 1, rot_dim,
                     positions, freq, neighbours, magnitude)
    k = torch.cat([c, rot], dim=1)[:, None, :]
    v = torch.cat([c, torch.zeros_like(rot)], dim=1)[:, None, :]
    kv_store(k, v, k_cache, v_cache, slots, page_size)


def heads_linear(x, in_stride, in_offset, w, out, out_stride, out_offset, compute=torch.float32):
    """Per head h: out[t, h * out_stride + out_offset + n] = sum_k w[h, n, k] x[t, h * in_stride + in_offset + k]."""
    t = x.shape[0]
    heads, n, k = w.shape
    src = x[:, : heads * in_stride].reshape(t, heads, in_stride)[:, :, in_offset: in_offset + k].to(compute)
    res = torch.einsum("thk,hnk->thn", src, w.to(compute))
    out[:, : heads * out_stride].view(t, heads, out_stride)[:, :, out_offset: out_offset + n] = res.to(out.dtype)
    return out


def retention_prepare(y, heads, dim, vdim, positions, freq, k_scale):
    """float32 [T, 2 heads dim + heads vdim]: queries and keys rotated (keys then scaled), values as they are."""
    t = y.shape[0]
    out = torch.empty((t, 2 * heads * dim + heads * vdim), dtype=torch.float32, device=y.device)
    src = y[:, : 2 * heads * dim].contiguous()
    rotate_half_copy(src, dim, 0, out[:, : 2 * heads * dim], dim, 0, 2 * heads, dim, positions, freq)
    out[:, heads * dim: 2 * heads * dim] *= k_scale
    out[:, 2 * heads * dim:] = y[:, 2 * heads * dim: 2 * heads * dim + heads * vdim].to(torch.float32)
    return out


def retention_rule(qkv, decay, state, cu_q, slots, heads, dim, vdim):
    """S <- decay S + k v^T; o = S^T q, per sequence and head from the slot's state [slots, heads, vdim, dim]."""
    t = qkv.shape[0]
    q = qkv[:, : heads * dim].view(t, heads, dim)
    k = qkv[:, heads * dim: 2 * heads * dim].view(t, heads, dim)
    v = qkv[:, 2 * heads * dim:].view(t, heads, vdim)
    out = torch.empty((t, heads, vdim), dtype=torch.float32, device=qkv.device)
    for s in range(len(cu_q) - 1):
        slot = int(slots[s])
        st = state[slot].clone()  # [heads, vdim, dim]
        for i in range(int(cu_q[s]), int(cu_q[s + 1])):
            st = st * decay[:, None, None] + v[i][:, :, None] * k[i][:, None, :]
            out[i] = torch.einsum("hvd,hd->hv", st, q[i])
        state[slot] = st
    return out


def unary_act(x, kind):
    if kind != "relu2":
        raise ValueError(kind)
    return torch.relu(x.to(torch.float32)).pow(2).to(x.dtype)


def scaled_add_rmsnorm(residual, parts, weight, eps, out_dtype, rows=None, compute=torch.float32):
    """``residual += sum_i scale_i * y_i`` in place (each ``y_i`` a matrix or planes), then the rows' RMS
    norm; with ``rows`` only those, and ``residual`` is left alone."""
    total = None
    for y, scale in parts:
        term = planes_sum(y) * scale.to(torch.float32)
        total = term if total is None else total + term
    return add_rmsnorm(residual, total, weight, eps, out_dtype, rows, compute)


def qk_joint_norm_store(qk, nq, nkv, d, bias, q_w, k_w, eps, positions, q_temp, values_are_keys,
                        k_cache=None, v_cache=None, slots=None, page_size=None):
    """Columns q | k (| v) of a product: biases added in float32; the values are the keys as they
    then are (or the v columns); all query elements of a token are divided by their one root
    mean square and multiplied by ``q_w`` [nq d], likewise the keys with ``k_w`` [nkv d]; queries at
    position p times ``1 + coef ln(floor((p + 1) / every) + 1)``; keys and values go to the cache."""
    t = qk.shape[0]
    y = qk.to(torch.float32)
    if bias is not None:
        y = y + bias
    q, k = y[:, : nq * d], y[:, nq * d: (nq + nkv) * d]
    v = k if values_are_keys else y[:, (nq + nkv) * d: (nq + 2 * nkv) * d]
    v = v.to(qk.dtype)
    q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * q_w
    k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * k_w
    if q_temp is not None:
        coef, every = q_temp
        p = positions.to(torch.float32)
        q = q * (1.0 + coef * torch.log(torch.floor((p + 1.0) / every) + 1.0))[:, None]
    if k_cache is not None:
        kv_store(k.view(t, nkv, d), v.view(t, nkv, d), k_cache, v_cache, slots, page_size)
    return q.to(qk.dtype)


class TorchOps:
    """The engine's op interface over the functions above (tests only)."""

    def __init__(self, compute=torch.float32):
        self.compute = compute

    def embed(self, ids, table, scale=1.0):
        return embed(ids, table, scale)

    def add_rmsnorm(self, residual, delta, weight, eps, out_dtype, rows=None, delta_scale=1.0, delta_norm=None):
        return add_rmsnorm(residual, delta, weight, eps, out_dtype, rows, self.compute, delta_scale, delta_norm)

    def scale(self, x, factor):
        return x.mul_(factor)

    def new_rows(self, t, width, dtype, device):
        return torch.empty((t, width), dtype=dtype, device=device)

    def rmsnorm_columns(self, y, first, width, weight, eps):
        return rmsnorm_columns(y, first, width, weight, eps)

    def latent_store(self, y, first, rank, rot_dim, weight, eps, positions, freq, cache, neighbours=False, magnitude=1.0):
        if cache is not None:
            latent_store(y, first, rank, rot_dim, weight, eps, positions, freq, cache.k, cache.v, cache.group.slots,
                         cache.group.page_size, neighbours, magnitude)

    def scaled_add_rmsnorm(self, residual, parts, weight, eps, out_dtype, rows=None):
        return scaled_add_rmsnorm(residual, parts, weight, eps, out_dtype, rows, self.compute)

    def qk_joint_norm_store(self, qk, nq, nkv, d, bias, q_w, k_w, eps, positions, q_temp, values_are_keys, cache):
        if cache is None:
            return qk_joint_norm_store(qk, nq, nkv, d, bias, q_w, k_w, eps, positions, q_temp, values_are_keys)
        return qk_joint_norm_store(qk, nq, nkv, d, bias, q_w, k_w, eps, positions, q_temp, values_are_keys,
                                   cache.k, cache.v, cache.group.slots, cache.group.page_size)

    def heads_linear(self, x, in_stride, in_offset, w, out, out_stride, out_offset):
        return heads_linear(x, in_stride, in_offset, w, out, out_stride, out_offset, self.compute)

    def rotate_half(self, x, in_stride, in_offset, out, out_stride, out_offset, heads, width, positions, freq,
                    neighbours=False, magnitude=1.0):
        return rotate_half_copy(x, in_stride, in_offset, out, out_stride, out_offset, heads, width, positions, freq,
                                neighbours, magnitude)

    def sigmoid_gate(self, out, gate):
        out.copy_((out.to(torch.float32) * torch.sigmoid(gate.to(torch.float32))).to(out.dtype))
        return out

    def retention_prepare(self, y, heads, dim, vdim, positions, freq, k_scale):
        return retention_prepare(y, heads, dim, vdim, positions, freq, k_scale)

    def retention_rule(self, ctx, qkv, decay, state, heads, dim, vdim):
        return retention_rule(qkv, decay, state, ctx.cu_q, ctx.state_slots, heads, dim, vdim)

    def unary_act(self, x, kind):
        return unary_act(x, kind)

    def norm_mean(self, ya, wa, yb, wb, eps):
        return norm_mean(ya, wa, yb, wb, eps)

    def add_concat(self, residual, delta, delta_scale, origin, out_dtype):
        x = residual if delta is None else residual + delta_scale * planes_sum(delta)
        return torch.cat([x, origin], dim=1).to(out_dtype)

    def linear_planes_with_spare(self, x, w):
        return None  # no planes here: the sum is taken by ``accumulate``

    def accumulate(self, acc, y):
        acc += planes_sum(y)
        return acc

    def gated_act(self, gate_up, activation="swiglu", limit=0.0):
        i = gate_up.shape[-1] // 2
        return gated(gate_up[..., :i].to(self.compute), gate_up[..., i:].to(self.compute), activation, limit).to(gate_up.dtype)

    def bias_rotate_pairs(self, x, bias, positions, freq, rot_heads, head_dim):
        return bias_rotate_pairs(x, bias, positions, freq, rot_heads, head_dim)

    def delta_conv(self, ctx, y, channels, taps, tail, segments, unit_eps):
        return delta_conv(y, channels, taps, tail, ctx.cu_q, ctx.state_slots, segments, unit_eps)

    def delta_rule(self, ctx, qkv, beta, a_logits, a_log, dt_bias, state, heads, kv_heads, dim, vdim, per_channel):
        return delta_rule(qkv, beta, a_logits, a_log, dt_bias, state, ctx.cu_q, ctx.state_slots, heads, kv_heads,
                          dim, vdim, per_channel)

    def delta_out(self, o, weight, gate, eps, gate_kind, out_dtype):
        return delta_out(o, weight, gate, eps, gate_kind, out_dtype)

    def linear(self, x, w, out_f32=False):
        return linear(x, w, out_f32, self.compute)

    def linear_for_residual(self, x, w):
        return linear(x, w, False, self.compute)

    def qk_norm_rope_store(self, qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions, cache, ctx=None,
                           angles_key=None, value_dim=None, extra=0):
        if cache is None:
            return qk_norm_rope_store(qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions,
                                      compute=self.compute, value_dim=value_dim)
        return qk_norm_rope_store(qkv, nq, nkv, d, q_w, k_w, eps, inv_freq, positions,
                                  cache.k, cache.v, cache.group.slots, cache.group.page_size, self.compute,
                                  value_dim=value_dim)

    def mix_norm(self, streams, update, read, weight, bias, eps, out_dtype, rows=None):
        return mix_norm(streams, update, read, weight, bias, eps, out_dtype, rows, self.compute)

    def route_top(self, x, router, router_bias, top, scoring="softmax_top", groups=1, keep=None, group_score="top2",
                  correction=None, renormalise=False, weight_scale=1.0):
        return route_top(x, router, router_bias, top, scoring, groups, keep, group_score, correction, renormalise,
                         weight_scale)

    def moe_swiglu(self, x, gate_up, down, index, weight, activation="swiglu", limit=0.0):
        return moe_swiglu(x, gate_up, down, index, weight, self.compute, activation, limit)

    def fuses_decode_attention(self, ctx, qkv, nq, nkv, d, cache, **more):
        return False  # no one-kernel form of a decode step's attention here: the steps above, in order

    def qk_norm_split(self, qkv, nq, nkv, d, q_w, k_w, eps):
        return qk_norm_split(qkv, nq, nkv, d, q_w, k_w, eps, self.compute)

    def rope_neox(self, q, k, positions, inv_freq):
        return (rope_rotate(q.to(self.compute), positions, inv_freq, self.compute).to(q.dtype),
                rope_rotate(k.to(self.compute), positions, inv_freq, self.compute).to(k.dtype))

    def kv_store(self, k, v, cache):
        kv_store(k, v, cache.k, cache.v, cache.group.slots, cache.group.page_size)

    def paged_attention(self, q, cache, ctx, nq, nkv, d, scale, window, chunk=None, softcap=None, value_dim=None,
                        gate=None, keep_first=0, sink=False):
        return paged_attention(q, cache.k, cache.v, ctx.cu_q, ctx.kv_lens, cache.group.block_table,
                               cache.group.page_size, nq, nkv, d, scale, window, self.compute, chunk=chunk,
                               softcap=softcap, value_dim=value_dim, gate=gate, keep_first=keep_first, sink=sink)

    def swiglu(self, gate_up):
        return swiglu(gate_up, self.compute)

    def gated_linear(self, x, w_gate_up, activation="swiglu", limit=0.0):
        return self.gated_act(linear(x, w_gate_up, False, self.compute), activation, limit)

    def argmax(self, logits):
        return argmax(logits)
