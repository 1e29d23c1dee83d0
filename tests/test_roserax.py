"""Roserax: every mechanism alone against its plain function, and whole models under every cutting.

Each test runs with the plain torch ops on the CPU (which pins the host side: plan, packing,
pages, windows with kept first tokens, state slots, the loop) and with the HIP ops on the GPU
(marked ``gpu``; float32 and bfloat16). The oracle is ``plain/roserax_plain.py``: whole sequences,
no cache, no state carried, float64. Configurations are made here and differ from each other in
every size and option, also in values that a model may happen to make equal or 1. Where random
weights would hide a fault (a key far back, the sink, the edge of a window, the first tokens a
window keeps), one token's key or value is made to stand out.
"""

from __future__ import annotations

import math
from types import SimpleNamespace

import pytest
import torch

import traces
from plain import roserax_plain as P
from plain.ops_ref import TorchOps

from drivers import BACKENDS, DT, GPU, DictFetch, MixerDriver, f64, in_steps, make_ops, rnd, rounded, tol  # noqa: F401


# ------------------------------------------------------------------ windowed attention with a sink
def window_weights(width, heads, kv_heads, d, dv, seed=0):
    return {"q": rnd(heads * d, width, seed=seed + 1, scale=0.3), "k": rnd(kv_heads * d, width, seed=seed + 2, scale=0.3),
            "v": rnd(kv_heads * dv, width, seed=seed + 3, scale=0.3), "o": rnd(width, heads * dv, seed=seed + 4, scale=0.3),
            "q.norm": 1 + rnd(d, seed=seed + 5, scale=0.2), "k.norm": 1 + rnd(d, seed=seed + 6, scale=0.2)}


def window_mixer(width, sizes, eps, w, device, dt):
    from qwen3_runtime_amd.parts.attention import GroupedQueryAttention

    names = {n: n for n in ("q", "k", "v", "o")} | {"q_norm": "q.norm", "k_norm": "k.norm"}
    mixer = GroupedQueryAttention(width, sizes["heads"], sizes["kv_heads"], sizes["dim"], qk_norm_eps=eps, value_dim=sizes["vdim"],
                                  scale=sizes["scale"], window=sizes["mask"]["size"], keep_first=sizes["mask"]["keep_first"],
                                  sink=True, tensors=names)
    mixer.load(DictFetch(w, device, dt))
    return mixer


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,kv_heads,d,dv,window,keep,page", [
    (4, 2, 32, 32, 40, 5, 16),     # kept tokens inside the first page
    (6, 2, 16, 24, 21, 19, 8),     # values wider than keys; kept tokens over three pages, the last one partly
    (2, 2, 64, 64, 70, 16, 16),    # kept tokens end where a page ends; a key head per query head
    (3, 1, 48, 20, 9, 1, 8),       # one kept token
    (2, 1, 128, 128, 130, 0, 16),  # none kept
    (5, 5, 8, 8, 1, 3, 8),         # a window of the query itself
    (8, 2, 96, 96, 33, 7, 32),
    (4, 2, 32, 32, 40, 70, 16),    # kept tokens over three blocks of 32 keys
    (2, 1, 64, 64, 24, 64, 16),    # ... exactly two
    (4, 4, 128, 128, 50, 33, 16),
])
def test_window_keeps_first_tokens_and_has_a_sink(backend, heads, kv_heads, d, dv, window, keep, page):
    """The attention mixer (normed queries and keys, no rotation, window, kept first tokens, sink) over
    a paged cache whose pages between the kept tokens and the window go back to the pool: against
    the plain mixer on the whole sequence. Two tokens' inputs are scaled so that their values stand
    out wherever they are seen: the last token that is kept (its neighbour, the first one that is
    not, is marked with the opposite sign) and one in the middle, whose window's edge the queries
    pass one by one and in a portion."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, eps = 40, 1e-5
    t = keep + 3 * window + 50
    sizes = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": dv, "scale": 1.3 / math.sqrt(d),
             "mask": {"size": window, "keep_first": keep}}
    w = rounded(window_weights(width, heads, kv_heads, d, dv), dt)
    h = rnd(t, width, seed=8)
    marked = t - window - 25
    # queries and keys are normed, so a scaled input leaves its score alone and scales its value
    h[marked] *= 40.0
    if keep:
        h[keep - 1] *= 30.0
    h[keep] *= -30.0
    h = h.to(dt).float()
    want = P.window_attention(h.double(), f64(w), sizes, eps)
    edge = marked + window  # the first query that no longer sees the marked token
    pages = -(-(keep + page) // page) + -(-(window + 64) // page) + 2
    for cuts in (in_steps(edge - 3, (64, 5)) + [(p, 1) for p in range(edge - 3, edge + 4)] + [(edge + 4, t - edge - 4)],
                 in_steps(edge - 10, (7, 2, 30)) + [(edge - 10, 20)] + in_steps(t, (1,), edge + 10)):
        driver = MixerDriver(window_mixer(width, sizes, eps, w, device, dt), device, dt, ops, page, pages)
        got = driver.run("a", h, cuts)
        assert driver.cache.groups[0].pool.num_free == pages
        # bfloat16: probabilities and values rounded to 8 bits move a row by about a hundredth of its largest element
        row_bound = 2e-4 + 2e-4 * want.abs().amax(1) if dtype == "float32" else 0.02 + 0.02 * want.abs().amax(1)
        assert (want[edge - 1] - want[edge]).abs().max() > max(0.5, 5 * float(row_bound[edge - 1]))  # the window's edge shows
        worst = (got.double() - want).abs().amax(1) / row_bound
        assert float(worst.max()) <= 1.0, (int(worst.argmax()), float(worst.max()))
    if keep and window > 1:
        # the kept tokens show far beyond the window: without them the last rows would differ
        no_keep = P.window_attention(h.double(), f64(w), {**sizes, "mask": {"size": window, "keep_first": keep - 1}}, eps)
        assert (no_keep[-1] - want[-1]).abs().max() > max(0.3, 5 * float(row_bound[-1]))
        one_more = P.window_attention(h.double(), f64(w), {**sizes, "mask": {"size": window, "keep_first": keep + 1}}, eps)
        assert (one_more[-1] - want[-1]).abs().max() > max(0.3, 5 * float(row_bound[-1]))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("nq,nkv,d,dv,page", [(4, 2, 32, 32, 16), (2, 1, 80, 48, 8), (3, 3, 16, 16, 16), (8, 1, 176, 176, 16)])
def test_the_sink_takes_the_weight_when_every_score_is_low(backend, nq, nkv, d, dv, page):
    """The attention op on keys written to pages directly. Queries against all keys (scores far below
    zero: the outputs shrink towards nothing, where an ordinary softmax would return an average
    of the values), queries along them (the sink's share vanishes), and, among three hundred keys,
    one far back that the query points at."""
    from qwen3_runtime_amd.parts.base import CacheView, GroupView, StepContext
    from qwen3_runtime_amd.parts.plan import CacheSpec

    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    t = 300
    unit = lambda x: x / x.norm(dim=-1, keepdim=True)  # noqa: E731
    common, own = unit(rnd(nkv, d, seed=5)), rnd(nkv, d, seed=6)
    own = unit(own - (own * common).sum(-1, keepdim=True) * common)   # the far key's direction, which nobody else shares
    k = rnd(t, nkv, d, seed=1, scale=d ** -0.5) + 1.2 * common          # every key has a share of one direction
    k = unit(k - (k * own).sum(-1, keepdim=True) * own)
    k[7] = own
    k = k.to(dt)
    v = (1.0 + rnd(t, nkv, dv, seed=2, scale=0.1)).to(dt)
    v[7] += 4.0
    pages = -(-t // page)
    kc = torch.full((pages + 1, nkv, page, d), float("nan"), dtype=dt, device=device)
    vc = torch.full((pages + 1, nkv, dv, page), float("inf"), dtype=dt, device=device)
    order = torch.randperm(pages + 1, generator=torch.Generator().manual_seed(3))[:pages].to(torch.int32)
    table = order[None].to(device)
    slots = torch.tensor([int(order[p // page]) * page + p % page for p in range(t)], dtype=torch.int32, device=device)
    spec = CacheSpec("paged_kv", heads=nkv, head_dim=d, value_dim=None if dv == d else dv)
    view = CacheView(spec, group=GroupView(page, None, table, slots), k=kc, v=vc)
    for p in range(t):  # keys [page, head, offset, D], values transposed within a page [page, head, Dv, offset]
        kc[int(order[p // page]), :, p % page, :] = k[p].to(device)
        vc[int(order[p // page]), :, :, p % page] = v[p].to(device)
    g = nq // nkv
    queries = {"against": -40.0 * (common + own), "along": 30.0 * k[-1].float(), "far": 30.0 * own}
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)  # noqa: E731
    for name, qk in queries.items():
        q = qk.repeat_interleave(g, dim=0).reshape(1, nq * d).to(dt)
        ctx = StepContext(ops=ops, dtype=dt, device=torch.device(device), num_tokens=1, num_seqs=1, positions=i32([t - 1]),
                          cu_q=i32([0, 1]), kv_lens=i32([t]), seq_of_token=i32([0]), state_slots=i32([0]), first_span=i32([0]),
                          q_lens_host=[1], kv_lens_host=[t], max_q_len=1, max_kv_len=t)
        ctx.groups = [view.group]
        more = {} if dv == d else {"value_dim": dv}
        got = ops.paged_attention(q.to(device), view, ctx, nq, nkv, d, 1.0, None, sink=True, **more).float().cpu().view(nq, dv)
        s = torch.einsum("hd,khd->hk", q.float().view(nq, d).double(), k.double().repeat_interleave(g, dim=1))
        p = P.softmax_with_sink(s, torch.ones_like(s, dtype=torch.bool))
        want = torch.einsum("hk,khd->hd", p, v.double().repeat_interleave(g, dim=1))
        torch.testing.assert_close(got.double(), want, **(dict(atol=2e-5, rtol=2e-4) if dtype == "float32" else dict(atol=3e-2, rtol=3e-2)))
        if name == "against":
            assert want.abs().max() < 0.6 and p.sum(-1).max() < 0.6   # an ordinary softmax would give about 1
        elif name == "along":
            assert p.sum(-1).min() > 0.99
        else:
            assert want.max() > 3.0  # the far key's value, not the others' average


# ------------------------------------------------------------------ attention through a latent
def latent_weights(width, n, d, r, dv, q_rank, kv_rank, seed=0):
    s = 0.3
    return {"dq": rnd(q_rank, width, seed=seed + 1, scale=s), "dq.norm": 1 + rnd(q_rank, seed=seed + 2, scale=0.2),
            "uq": rnd(n * (d + r), q_rank, seed=seed + 3, scale=s), "dkv": rnd(kv_rank + r, width, seed=seed + 4, scale=s),
            "dkv.norm": 1 + rnd(kv_rank, seed=seed + 5, scale=0.2), "uk": rnd(n * d, kv_rank, seed=seed + 6, scale=s),
            "uv": rnd(n * dv, kv_rank, seed=seed + 7, scale=s), "g": rnd(n * dv, width, seed=seed + 8, scale=s),
            "o": rnd(width, n * dv, seed=seed + 9, scale=s)}


def latent_mixer(width, sizes, eps, w, device, dt):
    from qwen3_runtime_amd.parts.latent import LatentAttention

    names = {n: n for n in ("dq", "uq", "dkv", "uk", "uv", "g", "o")} | {"dq_norm": "dq.norm", "dkv_norm": "dkv.norm"}
    mixer = LatentAttention(width, sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["q_rank"], sizes["kv_rank"],
                            sizes["scale"], eps, sizes["rot"]["dims"], sizes["rot"]["base"], tensors=names)
    mixer.load(DictFetch(w, device, dt))
    return mixer


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("n,d,r,dv,q_rank,kv_rank,base,page", [
    (4, 32, 16, 32, 48, 64, 100.0, 16),
    (3, 16, 8, 24, 20, 40, 1e4, 8),      # values wider than the plain key part, three heads
    (1, 64, 64, 16, 96, 32, 50.0, 16),   # one head, as many turning elements as plain ones
    (5, 24, 2, 8, 12, 24, 7.0, 8),       # one pair turns
    (2, 128, 64, 128, 160, 192, 1e6, 16),
])
def test_attention_through_a_latent(backend, n, d, r, dv, q_rank, kv_rank, base, page):
    """The latent mixer over pages that hold only the latent and the shared turning key part, in
    portions down to two tokens and token by token, two requests side by side in other steps: against the plain
    mixer, which builds every head's keys and values. Positions enter through the rotation only:
    the same inputs shifted by a few positions give other outputs."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, eps, t = 56, 1e-5, 150
    sizes = {"heads": n, "dim": d, "rot_dim": r, "vdim": dv, "q_rank": q_rank, "kv_rank": kv_rank,
             "scale": 0.5 / math.sqrt(d + r), "rot": {"dims": r, "base": base}}
    w = rounded(latent_weights(width, n, d, r, dv, q_rank, kv_rank), dt)
    h = [rnd(t, width, seed=8).to(dt).float(), rnd(90, width, seed=9).to(dt).float()]
    want = [P.latent_attention(x.double(), f64(w), sizes, eps) for x in h]
    mixer = latent_mixer(width, sizes, eps, w, device, dt)
    spec = mixer.cache_specs()[0]
    assert spec.heads * spec.head_dim == kv_rank + r   # nothing per head is kept
    pages = -(-t // page) + -(-90 // page)
    driver = MixerDriver(mixer, device, dt, ops, page, pages)
    top = max(1.0, float(want[0].abs().max()))
    bound = dict(atol=1e-4 * top, rtol=2e-4) if dtype == "float32" else dict(atol=0.03 * top, rtol=0.05)
    got = driver.run("a", h[0], in_steps(100, (33, 2, 1, 17)) + in_steps(t, (1,), 100))
    torch.testing.assert_close(got.double(), want[0], **bound)
    # two requests in the same steps, unequal portions; pages of the first run are used again
    driver.admit("a"), driver.admit("b")
    outs = {"a": [], "b": []}
    plan = {"a": in_steps(t, (40, 1, 9)), "b": in_steps(90, (2, 31, 1))}
    for i in range(max(len(p) for p in plan.values())):
        live = [r for r in ("a", "b") if i < len(plan[r])]
        res = driver.step([(r, h["ab".index(r)][plan[r][i][0]: plan[r][i][0] + plan[r][i][1]]) for r in live])
        for r, o in zip(live, res):
            outs[r].append(o)
    for j, rid in enumerate("ab"):
        torch.testing.assert_close(torch.cat(outs[rid]).double(), want[j], **bound)
    still = P.latent_attention(h[0].double(), f64(w), {**sizes, "rot": {"dims": 0, "base": base}}, eps)
    assert (still - want[0]).abs().max() > 10 * bound["atol"]   # the rotation matters to these outputs


# ------------------------------------------------------------------ rotation
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,width,dims,in_stride,in_off,out_stride,out_off,base", [
    (4, 32, 32, 48, 16, 40, 8, 1e4), (3, 24, 8, 24, 0, 24, 0, 100.0), (1, 64, 0, 64, 0, 70, 3, 1e4), (6, 16, 2, 20, 4, 16, 0, 3.0),
    (2, 128, 128, 128, 0, 128, 0, 1e6)])
def test_half_rotation_of_a_part_of_each_head(backend, heads, width, dims, in_stride, in_off, out_stride, out_off, base):
    """Element i against element i + dims/2, the rest of the head passes, at positions up to tens of
    thousands (float32 angles), from columns of one matrix into columns of another."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    t = 11
    pos = torch.tensor([0, 1, 2, 3, 17, 255, 256, 1000, 4097, 30000, 65535], dtype=torch.int32)
    x = rnd(t, heads * in_stride + 5, seed=1).to(dt)
    out = torch.full((t, heads * out_stride + 2), 7.0, dtype=dt, device=device)
    freq = (base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / max(dims, 1))).float() if dims else None
    ops.rotate_half(x.to(device)[:, : heads * in_stride + 5], in_stride, in_off, out, out_stride, out_off, heads, width,
                    pos.to(device), None if freq is None else freq.to(device))
    src = x[:, : heads * in_stride].view(t, heads, in_stride)[:, :, in_off: in_off + width].double()
    want = P.rotate_half(src, pos.tolist(), dims, base)
    got = out.cpu()[:, : heads * out_stride].view(t, heads, out_stride)
    # float32 angles at position 65,535 are good to 65535 * 2^-24 radians
    torch.testing.assert_close(got[:, :, out_off: out_off + width].double(), want,
                               **(dict(atol=2e-2, rtol=0) if dtype == "float32" else dict(atol=5e-2, rtol=2e-2)))
    torch.testing.assert_close(got[:4, :, out_off: out_off + width].double(), want[:4], **tol(dtype))
    rest = torch.ones(heads, out_stride, dtype=torch.bool)
    rest[:, out_off: out_off + width] = False
    assert (got[:, rest] == 7.0).all() and (out.cpu()[:, heads * out_stride:] == 7.0).all()  # nothing else is written


# ------------------------------------------------------------------ retention
def retention_weights(width, n, d, dv, seed=0):
    return {"q": rnd(n * d, width, seed=seed + 1, scale=0.3), "k": rnd(n * d, width, seed=seed + 2, scale=0.3),
            "v": rnd(n * dv, width, seed=seed + 3, scale=0.3), "g": rnd(n * dv, width, seed=seed + 4, scale=0.3),
            "o": rnd(width, n * dv, seed=seed + 5, scale=0.3)}


def retention_mixer(width, sizes, eps, w, device, dt):
    from qwen3_runtime_amd.parts.retention import Retention

    mixer = Retention(width, sizes["heads"], sizes["dim"], sizes["vdim"], sizes["decay"], eps, sizes["rot"]["dims"],
                      sizes["rot"]["base"], tensors={n: n for n in ("q", "k", "v", "g", "o")})
    mixer.load(DictFetch(w, device, dt))
    return mixer


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("n,d,dv,decay,dims,base", [
    (3, 32, 16, (0.9, 0.97, 0.995), 16, 5000.0),
    (2, 24, 40, (0.5, 1.0), 24, 1e6),          # a head that forgets nothing, one that forgets fast
    (1, 64, 64, (0.99,), 64, 1e4),
    (4, 16, 8, (0.8, 0.8, 0.95, 0.0), 0, 1.0),  # no rotation; a head that remembers only the token itself
    (5, 8, 72, (0.9, 0.91, 0.92, 0.93, 0.94), 2, 10.0),
    (2, 128, 128, (0.94, 0.998), 128, 1e6),
    (2, 40, 1, (0.9, 0.99), 20, 100.0),        # one value channel: the read-out's norm leaves its sign
])
def test_retention_against_the_recurrence_written_out(backend, n, d, dv, decay, dims, base):
    """The retention mixer with its state in a slot, a whole prompt at once, portions down to one
    token, and two requests in the same steps whose slots are then taken again by others."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, eps = 48, 1e-5
    t = 60 if device == "cpu" else 200
    sizes = {"heads": n, "dim": d, "vdim": dv, "decay": list(decay), "rot": {"dims": dims, "base": base}}
    w = rounded(retention_weights(width, n, d, dv), dt)
    h = [rnd(t, width, seed=8).to(dt).float(), rnd(t // 2, width, seed=9).to(dt).float()]
    want = [P.retention(x.double(), f64(w), sizes, eps) for x in h]
    driver = MixerDriver(retention_mixer(width, sizes, eps, w, device, dt), device, dt, ops, 16, 1, max_requests=3)
    bound = dict(atol=3e-4, rtol=3e-4) if dtype == "float32" else dict(atol=0.03 * float(want[0].abs().max()), rtol=0.05)
    for state in driver.cache._state_of_cache.values():
        state.fill_(float("nan"))  # a slot is zeroed when it is taken
    driver.admit("other")  # slot 0 is somebody else's
    torch.testing.assert_close(driver.run("a", h[0], [(0, t)]).double(), want[0], **bound)
    torch.testing.assert_close(driver.run("a", h[0], in_steps(t, (17, 1, 2, 1, 1, 30, 3))).double(), want[0], **bound)
    driver.admit("a"), driver.admit("b")
    outs = {"a": [], "b": []}
    plan = {"a": in_steps(t, (25, 1, 64)), "b": in_steps(t // 2, (1, 2, 40))}
    for i in range(max(len(p) for p in plan.values())):
        live = [r for r in ("b", "a") if i < len(plan[r])]
        res = driver.step([(r, h["ab".index(r)][plan[r][i][0]: plan[r][i][0] + plan[r][i][1]]) for r in live])
        for r, o in zip(live, res):
            outs[r].append(o)
    for j, r in enumerate("ab"):
        torch.testing.assert_close(torch.cat(outs[r]).double(), want[j], **bound)
    driver.release("a"), driver.release("b")
    torch.testing.assert_close(driver.run("c", h[1], in_steps(t // 2, (5, 1))).double(), want[1], **bound)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,d,dv", [(2, 32, 16), (1, 64, 64), (3, 8, 40), (2, 128, 128), (2, 256, 8), (1, 100, 3)])
def test_retention_reads_a_write_from_far_back_and_a_slot_taken_again_is_empty(backend, heads, d, dv):
    """The recurrence alone, float32. One head forgets nothing: a marker written under a key of its
    own 400 tokens back, across many portions and beside a second sequence, is read whole; the
    other heads' decays have left nothing of theirs. The rule has no denominator: values add up.
    After the slot is zeroed the same query reads nothing."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    t = 420
    decay = torch.tensor([1.0] + [0.9] * (heads - 1))
    unit = lambda x: x / x.norm(dim=-1, keepdim=True)  # noqa: E731
    q, k, v = torch.zeros(t, heads, d), unit(rnd(t, heads, d, seed=1)), rnd(t, heads, dv, seed=2)
    direction = unit(rnd(d, seed=77))
    k = k - (k @ direction)[..., None] * direction     # nobody else writes under the marker's key
    k[5], v[5] = direction, 9.0
    k[300, 0], v[300, 0] = direction, 2.0               # a second write under it adds to the first
    q[-1] = direction
    want = torch.stack([P.retention_head(q[:, j].double(), k[:, j].double(), v[:, j].double(), float(decay[j])) for j in range(heads)], 1)
    assert (want[-1, 0] - 11.0).abs().max() < 1e-4 and (heads == 1 or want[-1, 1:].abs().max() < 1e-4)
    state = torch.full((3, heads, dv, d), float("nan"), device=device)
    state[1:] = 0.0
    qkv = torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], 1)
    qkv2 = torch.cat([x.reshape(t, -1) for x in (rnd(t, heads, d, seed=5), unit(rnd(t, heads, d, seed=6)), rnd(t, heads, dv, seed=7))], 1)
    got = torch.zeros(t, heads, dv)
    for p, n in in_steps(t, (64, 3, 1, 100, 2)):
        ctx = SimpleNamespace(num_tokens=2 * n, num_seqs=2, cu_q=torch.tensor([0, n, 2 * n], dtype=torch.int32, device=device),
                              state_slots=torch.tensor([2, 1], dtype=torch.int32, device=device))
        rows = torch.cat([qkv2[p: p + n], qkv[p: p + n]]).contiguous().to(device)
        got[p: p + n] = ops.retention_rule(ctx, rows, decay.to(device), state, heads, d, dv).cpu()[n:]
    torch.testing.assert_close(got.double(), want, atol=1e-4, rtol=1e-4)
    assert torch.isnan(state[0]).all()
    state[1].zero_()
    ctx = SimpleNamespace(num_tokens=1, num_seqs=1, cu_q=torch.tensor([0, 1], dtype=torch.int32, device=device),
                          state_slots=torch.tensor([1], dtype=torch.int32, device=device))
    again = ops.retention_rule(ctx, qkv[-1:].contiguous().to(device), decay.to(device), state, heads, d, dv).cpu()
    assert again.abs().max() < 1e-6


# ------------------------------------------------------------------ norms on both sides, feed-forwards
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,tokens,planes", [(96, 5, 0), (352, 3, 4), (2560, 2, 1), (50, 7, 2), (1, 4, 0)])
def test_a_sub_layer_output_joins_the_stream_through_its_norm(backend, width, tokens, planes):
    """``x += rmsnorm(y) * w_after`` and the next norm of the sum in one call; ``y`` a matrix or float32
    planes whose sum it is; all rows or chosen ones."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    x = rnd(tokens, width, seed=1)
    y = rnd(planes, tokens, width, seed=2, scale=3.0) if planes else rnd(tokens, width, seed=2, scale=3.0).to(dt)
    w_after, w_next = 1 + rnd(width, seed=3, scale=0.2), 1 + rnd(width, seed=4, scale=0.2)
    total = (y.sum(0) if planes else y).double()
    new_x = x.double() + P.rms_norm(total, w_after.double(), 1e-5)
    want = P.rms_norm(new_x, w_next.double(), 1e-6)
    res = x.clone().to(device)
    got = ops.add_rmsnorm(res, y.to(device), w_next.to(device), 1e-6, dt, delta_norm=(w_after.to(device), 1e-5))
    torch.testing.assert_close(res.cpu().double(), new_x, atol=1e-5, rtol=1e-5)   # the stream itself stays float32
    torch.testing.assert_close(got.cpu().double(), want, **tol(dtype))
    rows = torch.tensor([tokens - 1, 0], dtype=torch.int32)
    res = x.clone().to(device)
    got = ops.add_rmsnorm(res, y.to(device), w_next.to(device), 1e-6, dt, rows=rows.to(device), delta_norm=(w_after.to(device), 1e-5))
    torch.testing.assert_close(got.cpu().double(), want[rows.long()], **tol(dtype))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,inner,tokens", [(64, 112, 9), (256, 96, 1), (40, 7, 70), (128, 512, 300)])
def test_dense_feed_forward_with_a_squared_relu(backend, width, inner, tokens):
    from qwen3_runtime_amd.parts.mlp import ActMLP

    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    w = rounded({"up": rnd(inner, width, seed=1, scale=0.2), "down": rnd(width, inner, seed=2, scale=0.2)}, dt)
    part = ActMLP(width, inner, "relu2", tensors={"up": "up", "down": "down"})
    part.load(DictFetch(w, device, dt))
    x = rnd(tokens, width, seed=3).to(dt)
    got = part.forward(SimpleNamespace(ops=ops, dtype=dt), x.to(device))
    got = (got.sum(0) if got.dim() == 3 else got).double().cpu()
    want = P.dense_ff(x.double(), f64(w))
    assert (x.double() @ w["up"].double().T < 0).any()
    torch.testing.assert_close(got, want, **(tol(dtype) if dtype == "float32" else dict(atol=0.02 * float(want.abs().max()), rtol=0.05)))


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,groups,keep,width", [(18, 2, 3, 1, 200), (12, 3, 3, 2, 96), (6, 2, 1, 1, 64), (8, 4, 8, 4, 50),
                                                           (64, 6, 8, 3, 128), (4, 4, 2, 2, 31), (16, 4, 2, 1, 256), (5, 1, 5, 1, 40)])
def test_router_softmax_over_all_experts_and_groups_by_their_best(backend, experts, top, groups, keep, width):
    """Scores are the softmax over all experts; the chosen ones' scores weigh as they are (they sum
    to less than one)."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    x, router = rnd(40, width, seed=1).to(dt), rnd(experts, width, seed=2, scale=0.2)
    index, weight = ops.route_top(x.to(device), router.to(device), None, top, scoring="softmax_all", groups=groups, keep=keep,
                                  group_score="max")
    want_i, want_w = P.route(x.double(), router.double(), top, groups, keep)
    assert torch.equal(index.cpu().long().sort(1).values, want_i.sort(1).values)
    torch.testing.assert_close(weight.cpu().double().sort(1).values, want_w.sort(1).values, atol=1e-6, rtol=1e-5)
    if top < experts:
        assert weight.sum(1).max() < 1.0


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_group_is_judged_by_its_best_expert(backend):
    """Group 0 holds the best expert and two weak ones, group 1 three middling ones whose two best
    together outweigh group 0's: with one group kept, the choice is group 0's experts, the
    second of them a weak one, although every expert of group 1 scores higher than it."""
    device, dtype = backend
    ops = make_ops(device)
    router = torch.zeros(6, 4)
    router[:, 0] = torch.tensor([5.0, -3.0, -4.0, 4.6, 4.6, 4.4])
    x = torch.tensor([[1.0, 0, 0, 0]]).to(DT[dtype])
    index, weight = ops.route_top(x.to(device), router.to(device), None, 2, scoring="softmax_all", groups=2, keep=1, group_score="max")
    want_i, want_w = P.route(x.double(), router.double(), 2, 2, 1)
    assert sorted(index[0].tolist()) == sorted(want_i[0].tolist()) == [0, 1]
    torch.testing.assert_close(weight.cpu().double().sort(1).values, want_w.sort(1).values, atol=1e-6, rtol=1e-5)
    other, _ = ops.route_top(x.to(device), router.to(device), None, 2, scoring="softmax_all", groups=2, keep=1)  # by the two best
    assert sorted(other[0].tolist()) == [3, 4]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,inner,experts,top,groups,keep", [(128, 64, 8, 2, 2, 1), (384, 64, 16, 4, 4, 2), (96, 48, 12, 12, 3, 3),
                                                                 (256, 128, 4, 1, 1, 1), (80, 24, 6, 3, 2, 1)])
def test_mixture_of_silu_gated_experts_at_every_step_size(backend, width, inner, experts, top, groups, keep):
    """The feed-forward part over steps of 1 to 300 tokens: every form of the experts' products."""
    from qwen3_runtime_amd.parts.moe import RoutedSwiGLU

    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    names = {"router": "router", "gate": "e{e}.gate", "up": "e{e}.up", "down": "e{e}.down"}
    w = {"router": rnd(experts, width, seed=1, scale=0.3)}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (rnd(inner, width, seed=10 + e, scale=0.15), rnd(inner, width, seed=40 + e, scale=0.15),
                                                            rnd(width, inner, seed=70 + e, scale=0.15))
    w = rounded(w, dt)
    part = RoutedSwiGLU(width, inner, experts, top, router_bias=False, scoring="softmax_all", groups=groups, keep=keep,
                        group_score="max", tensors=names)
    part.load(DictFetch(w, device, dt))
    mlp = {"kind": "moe", "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    for tokens in (1, 8, 17, 70, 100, 300):
        x = rnd(tokens, width, seed=tokens).to(dt)
        got = part.forward(SimpleNamespace(ops=ops, dtype=dt), x.to(device))
        got = (got.sum(0) if got.dim() == 3 else got).double().cpu()
        want = P.mixture(x.double(), f64(w), mlp)
        if dtype == "float32":
            torch.testing.assert_close(got, want, atol=1e-4, rtol=1e-4)
        else:  # a token whose choice falls the other way in bfloat16 is another token; all others are close
            close = ((got - want).abs() <= 6e-2 + 6e-2 * want.abs()).all(dim=1)
            assert int((~close).sum()) <= max(1, tokens // 10), (tokens, int((~close).sum()))


# ------------------------------------------------------------------ whole models
def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, experts, top, groups=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def attention(heads, kv_heads, dim, vdim, scale, size, keep):
    raw = {"heads": heads, "dim": dim, "scale": scale, "mask": {"size": size}}
    if kv_heads != heads:
        raw["kv_heads"] = kv_heads
    if vdim != dim:
        raw["vdim"] = vdim
    if keep:
        raw["mask"]["keep_first"] = keep
    return raw


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
            "rot": {"dims": rot_dim, "base": base}}


def retention(heads, dim, vdim, decay, dims, base):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": {"dims": dims, "base": base}}


def model(vocab, width, layers, eps=1e-5, embedding=None, logit_scale=None):
    raw = {"architecture": "Roserax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if embedding is not None:
        raw["embedding"] = {"scale": embedding}
    if logit_scale is not None:
        raw["logit_scale"] = logit_scale
    return raw


def config_a():
    """All three mixers and both feed-forwards, unequal sizes everywhere; the window keeps five tokens
    of the first page; embedding and logits scaled."""
    return model(300, 96, [
        {"type": "retention", "mixer": retention(3, 32, 16, (0.9, 0.97, 0.995), 16, 5000.0), "mlp": moe(24, 12, 3, (4, 2))},
        {"type": "attention", "mixer": attention(6, 2, 16, 24, 0.2, 21, 5), "mlp": dense(112)},
        {"type": "latent_attention", "mixer": latent(3, 16, 8, 24, 20, 40, 0.3, 100.0), "mlp": None},
        {"type": "attention", "mixer": attention(4, 4, 32, 32, 0.15, 40, 19), "mlp": moe(40, 6, 2)}],
        embedding=7.0, logit_scale=0.5), 8


def config_b():
    """Begins with a latent layer; a window that keeps more tokens than it is long, over several pages;
    a head that forgets nothing; one expert a token from one of two groups; no scales in the file."""
    return model(150, 64, [
        {"type": "latent_attention", "mixer": latent(2, 32, 16, 16, 24, 48, 0.15, 1e4), "mlp": moe(32, 8, 1, (2, 1))},
        {"type": "attention", "mixer": attention(2, 1, 48, 48, 0.1, 9, 17), "mlp": None},
        {"type": "retention", "mixer": retention(2, 24, 40, (0.5, 1.0), 24, 1e6), "mlp": dense(96)}], eps=1e-6), 8


def config_c():
    """Retention only: a model without a single page of cache."""
    return model(90, 48, [
        {"type": "retention", "mixer": retention(1, 16, 16, (0.98,), 8, 10.0), "mlp": dense(40)},
        {"type": "retention", "mixer": retention(4, 8, 24, (0.7, 0.8, 0.9, 0.99), 0, 1.0), "mlp": moe(16, 4, 2, (2, 2))}],
        embedding=2.0, logit_scale=3.0), 16


def config_d():
    """Sizes that are multiples of nothing: width 90, keys of 10, 6 and 14, values of 7, 5 and 3, a
    window of 13 that keeps none and one of 1 that keeps two, experts of 9, groups of one expert; the
    last layer has no feed-forward, so the final norm takes the mixer's output through its norm."""
    return model(77, 90, [
        {"type": "attention", "mixer": attention(3, 1, 10, 7, 0.3, 13, 0), "mlp": moe(9, 5, 2, (5, 3))},
        {"type": "latent_attention", "mixer": latent(5, 6, 2, 5, 7, 11, 0.4, 7.0), "mlp": dense(33)},
        {"type": "retention", "mixer": retention(2, 14, 3, (0.9, 0.95), 6, 50.0), "mlp": dense(20)},
        {"type": "attention", "mixer": attention(2, 2, 6, 6, 0.5, 1, 2), "mlp": None}], embedding=0.5), 8


def config_e():
    """Two windowed layers of equal sizes (one pool of pages for both) and two of another window; the
    latent layer's pages in a pool of their own."""
    att = attention(4, 2, 32, 32, 0.18, 24, 6)
    return model(200, 80, [
        {"type": "attention", "mixer": att, "mlp": dense(64)},
        {"type": "latent_attention", "mixer": latent(4, 16, 16, 16, 32, 32, 0.2, 1e6), "mlp": moe(24, 16, 4, (2, 1))},
        {"type": "attention", "mixer": att, "mlp": moe(24, 16, 4, (2, 1))},
        {"type": "attention", "mixer": attention(4, 2, 32, 32, 0.18, 50, 6), "mlp": None},
        {"type": "retention", "mixer": retention(4, 32, 32, (0.97, 0.99, 0.997, 0.999), 32, 1e6), "mlp": dense(64)}],
        embedding=9.0, logit_scale=2.0), 16


def config_g():
    """Layers of a real model's proportions (heads of 128, a window of 256 that keeps 40 tokens, a latent of 256 with 64
    turning elements, experts of 512): the kernel forms that small sizes never reach."""
    return model(500, 1024, [
        {"type": "latent_attention", "mixer": latent(8, 128, 64, 128, 384, 256, 0.07, 1e4), "mlp": dense(2048)},
        {"type": "retention", "mixer": retention(8, 128, 128, tuple(1 - 0.08 / (1 + j) for j in range(8)), 128, 1e4),
         "mlp": moe(512, 8, 2, (4, 2))},
        {"type": "attention", "mixer": attention(8, 2, 128, 128, 0.09, 256, 40), "mlp": moe(512, 8, 2, (4, 2))}],
        embedding=4.0), 16


def every_expert(make):
    """The same model with a router that has no choice to make (every expert of every group is taken,
    weighted by its score): for runs in bfloat16, where a choice between two experts whose scores
    lie within rounding of each other may fall the other way, which moves that position's logits by
    a large part of their spread, and later positions' through the recurrent state. The choice
    itself is held to the plain one in float32 here, and in both types in the router's own test."""
    def made():
        raw, page = make()
        for layer in raw["layers"]:
            if layer["mlp"] and layer["mlp"]["kind"] == "moe":
                router = layer["mlp"]["router"]
                router["top"] = router["experts"]
                if "groups" in router:
                    router["groups"]["keep"] = router["groups"]["count"]
        return raw, page
    return made


CONFIGS = {"a": config_a, "b": config_b, "c": config_c, "d": config_d, "e": config_e, "g": config_g}
CONFIGS.update({name + "_every": every_expert(make) for name, make in list(CONFIGS.items())})
# bfloat16: the bound on the largest error of a position's logits, in units of their deviation
NOISE = {"a": 0.4, "b": 0.4, "c": 0.4, "d": 0.4, "e": 0.4, "g": 0.3}
LENGTHS = {"a": [1, 7, 45, 130], "b": [3, 17, 50, 64, 101], "c": [2, 16, 17, 120], "d": [1, 5, 40, 83], "e": [1, 9, 40, 150]}
_folders: dict = {}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    from qwen3_runtime_amd.weights import write_model_folder

    def get(name, dtype="float32"):
        if dtype == "bfloat16":
            name += "_every"
        if name not in _folders:
            raw, _ = CONFIGS[name]()
            _folders[name] = write_model_folder(tmp_path_factory.mktemp("roserax_" + name), raw, seed=31 + len(_folders),
                                                std=0.03 if name.startswith("g") else 0.08, norm_jitter=0.2)
        return _folders[name]

    return get


def load(folder, page, pages, backend, max_seqs=4, hip_graph=False):
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.factory import load as load_model

    device, dtype = backend
    cfg = EngineConfig(page_size=page, num_pages=pages, max_num_seqs=max_seqs, dtype=dtype, device=device,
                       hip_graph=hip_graph)
    return load_model(folder, cfg, ops=TorchOps() if device == "cpu" else None)


def plain_logits(folder, requests):
    cfg, w = P.load(folder)
    out = {}
    for rid, toks in requests.items():
        logits = P.forward(cfg, w, toks).float()
        for p in range(len(toks)):
            out[(rid, p)] = logits[p]
    return out


def check(got, want, dtype, noise=0.2):
    """float32: to rounding of float32 sums, everywhere. bfloat16: as noise relative to the logits'
    own spread, their root mean square under a quarter of ``noise`` and no position over ``noise``,
    one in a hundred aside: a retention head's read-out is divided by its root mean square, so at a
    sequence's first positions, where the state is one outer product, it is a fixed vector times
    the sign of ``k . q``, and that sign may fall the other way in 8 bits. A wrong window, state or
    portion shows in float32, where the bound is rounding."""
    if dtype == "float32":
        traces.compare(got, want, atol=2e-4, rtol=2e-4)
        return
    keys = sorted(want)
    assert set(got) == set(want)
    w = torch.stack([want[k].double() for k in keys])
    err = torch.stack([got[k].double() for k in keys]) - w
    std = float(w.std())
    per_pos = err.abs().amax(dim=1)
    good = per_pos < noise * std
    assert int((~good).sum()) <= len(keys) // 100, \
        f"{int((~good).sum())} of {len(keys)} positions over the bound, the first {keys[int((~good).nonzero()[0])]}"
    rms = float(err[good].pow(2).mean().sqrt())
    assert rms < 0.25 * noise * std, f"rms error {rms:.4f} against a logit deviation of {std:.3f}"


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("name", ["a", "b", "c", "d", "e"])
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_cuttings_match_plain(folder, backend, name, cut):
    """Whole prompts; the last tokens one by one (across window edges); portions down to two tokens;
    up to four live requests mixed in a pool of the peak's size, so that pages and slots are used
    again (freed pages are poisoned first; a slot is zeroed when it is taken)."""
    raw, page = CONFIGS[name]()
    reqs = traces.make_requests(raw["vocab"], LENGTHS[name] + ([30, 9] if cut == "mixed" else []), seed=5)
    steps = getattr(traces, cut)(reqs)
    loaded = load(folder(name, backend[1]), page, traces.peak_tokens(steps, unit=page) // page, backend)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, plain_logits(folder(name, backend[1]), reqs), backend[1], NOISE[name])
    assert (len(loaded.cache.groups) == 0) == (name == "c")


def test_the_stream_after_every_layer_matches_plain(folder):
    """Layer by layer: the engine's residual stream after each layer (the pending sub-layer output
    applied through its norm) against the plain one, for a short prompt."""
    from qwen3_runtime_amd.engine.batch import StepEntry

    raw, page = config_a()
    toks = traces.make_requests(raw["vocab"], [33], seed=3)["r0"]
    cfg, w = P.load(folder("a"))
    _, want = P.forward(cfg, w, toks, return_layers=True)
    loaded = load(folder("a"), page, 8, ("cpu", "float32"))
    seen = []
    for block in loaded.model.blocks:
        inner = block.forward

        def spy(ctx, residual, delta, cache, inner=inner):
            residual, pending = inner(ctx, residual, delta, cache)
            y = pending.y.double().sum(0) if pending.y.dim() == 3 else pending.y.double()
            seen.append(residual.double() + P.rms_norm(y, pending.weight.double(), pending.eps))
            return residual, pending

        block.forward = spy
    loaded.cache.admit("x")
    loaded.runner.step([StepEntry("x", toks, [len(toks) - 1])])
    loaded.cache.release("x")
    assert len(seen) == len(raw["layers"])
    for i, (got, ref) in enumerate(zip(seen, want)):
        torch.testing.assert_close(got, ref, atol=2e-4, rtol=2e-4, msg=lambda m, i=i: f"after layer {i}: {m}")


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_of_a_real_model_s_proportions(folder, dtype):
    """A 330-token prompt in one step, then in portions with its last tokens one by one, beside a
    second request: prompt kernels with full tiles, the window passing, experts by expert."""
    raw, page = config_g()
    reqs = traces.make_requests(raw["vocab"], [330, 40], seed=9)
    want = plain_logits(folder("g", dtype), reqs)
    for steps in (traces.whole(reqs), traces.mixed(reqs, seed=2, decode_tail=12)):
        loaded = load(folder("g", dtype), page, traces.peak_tokens(steps, unit=page) // page, ("cuda:0", dtype))
        check(traces.replay(loaded, steps, poison_freed=True), want, dtype, NOISE["g"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding_in_a_pool_of_one_window(folder, backend):
    """A request far longer than the windowed pool, decoded token by token: the windowed caches give
    their pages back as the window passes and keep those of the first tokens; the state has none."""
    raw, page = config_b()
    raw["layers"] = raw["layers"][1:]  # windowed attention and retention: nothing grows with the length
    from qwen3_runtime_amd.weights import write_model_folder
    import tempfile

    with tempfile.TemporaryDirectory() as tmp:
        if backend[1] == "bfloat16":
            raw = every_expert(lambda: (raw, page))()[0]
        where = write_model_folder(tmp, raw, seed=12, std=0.08, norm_jitter=0.2)
        reqs = traces.make_requests(raw["vocab"], [300], seed=8)
        steps = traces.tail_one_by_one(reqs, tail=290)
        loaded = load(where, page, 7, backend)   # 17 kept tokens: 3 pages; a window of 9: 3 pages; one to spare
        got = traces.replay(loaded, steps, poison_freed=True)
        check(got, plain_logits(where, reqs), backend[1], NOISE["b"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_decoded_tokens_over_a_long_context_beside_prompt_portions(folder, backend):
    """One request decodes past 1,000 tokens while another is read in portions in the same steps: the
    attention of the few rows with the long context is cut over many blocks in a launch of its own,
    whose parts a merge joins (with the sink, after the kept first keys), beside the portions'."""
    raw, page = config_e()
    reqs = traces.make_requests(raw["vocab"], [1085, 700], seed=11)
    a, b = reqs["r0"], reqs["r1"]
    steps = [{"step": 0, "entries": [{"id": "r0", "tokens": a[:1060], "want": [0, 500, 1059]}], "end": []}]
    for i in range(25):
        steps.append({"step": i + 1, "end": ["r0", "r1"] if i == 24 else [], "entries": [
            {"id": "r0", "tokens": a[1060 + i: 1061 + i], "want": [0]},
            {"id": "r1", "tokens": b[28 * i: 28 * (i + 1)], "want": [0, 27]}]})
    loaded = load(folder("e", backend[1]), page, traces.peak_tokens(steps, unit=page) // page, backend)
    got = traces.replay(loaded, steps, poison_freed=True)
    want = plain_logits(folder("e", backend[1]), reqs)
    check(got, {k: want[k] for k in got}, backend[1], NOISE["e"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_batch_mates_do_not_change_a_request(folder, backend):
    """Unequal requests in one batch against each alone: the same logits within rounding."""
    raw, page = config_a()
    reqs = traces.make_requests(raw["vocab"], [9, 60, 121, 33], seed=2)
    together = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in reqs.items()],
                 "end": list(reqs)}]
    loaded = load(folder("a", backend[1]), page, 64, backend)
    both = traces.replay(loaded, together)
    alone = traces.replay(loaded, traces.whole(reqs))
    if backend[1] == "float32":
        traces.compare(both, alone, atol=2e-5, rtol=2e-5)
    else:
        check(both, alone, "bfloat16", NOISE["a"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_restarted_request_computes_the_same_again(folder, backend):
    """Preemption by recompute: pages back, state zeroed, the slot kept; the second pass over the
    same tokens gives the first one's logits."""
    from qwen3_runtime_amd.engine.batch import StepEntry

    raw, page = config_e()
    toks = traces.make_requests(raw["vocab"], [70], seed=3)["r0"]
    loaded = load(folder("e"), page, 16, backend)
    loaded.cache.admit("x")
    first = loaded.runner.step([StepEntry("x", toks[:50], [49])]).float().cpu()
    loaded.runner.step([StepEntry("x", toks[50:], [0])])
    loaded.cache.restart("x")
    again = loaded.runner.step([StepEntry("x", toks[:50], [49])]).float().cpu()
    loaded.cache.release("x")
    torch.testing.assert_close(again, first, atol=1e-6 if backend[1] == "float32" else 1e-2, rtol=0)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,graphs", [("float32", False), ("bfloat16", True), ("bfloat16", False)])
@pytest.mark.parametrize("name", ["a", "c", "e"])
def test_greedy_generation_through_the_entry_point(folder, name, dtype, graphs):
    """``LLM.generate`` (scheduler with a small token budget, sampler, graphs where they apply): the
    tokens chosen greedily are, by the plain model given the same context, the best ones or within
    rounding of the best. Requests of unequal lengths, more of them than fit at once."""
    from qwen3_runtime_amd.llm import LLM

    raw, page = CONFIGS[name]()
    llm = LLM(str(folder(name, dtype)), dtype=dtype, block_size=page, num_kv_blocks=64, max_num_seqs=3,
              max_num_batched_tokens=48, cuda_graph=graphs)
    prompts = list(traces.make_requests(raw["vocab"], [5, 61, 20, 90], seed=4).values())
    outs = llm.generate(prompts, max_tokens=40)
    cfg, w = P.load(folder(name, dtype))
    for prompt, tokens in zip(prompts, outs):
        assert len(tokens) == 40
        logits = P.forward(cfg, w, list(prompt) + list(tokens))[len(prompt) - 1: -1]
        below = logits.max(-1).values - logits[range(40), list(tokens)]
        bound = 1e-3 if dtype == "float32" else 2 * NOISE[name] * float(logits.std())
        assert int((below >= bound).sum()) == 0, (float(below.max()), int(below.argmax()))


def test_greedy_generation_on_the_host(folder):
    """The same entry point's scheduler and sampler over the plain torch ops."""
    from qwen3_runtime_amd.engine.batch import StepEntry

    raw, page = config_d()
    cfg, w = P.load(folder("d"))
    loaded = load(folder("d"), page, 32, ("cpu", "float32"))
    prompt = traces.make_requests(raw["vocab"], [12], seed=4)["r0"]
    loaded.cache.admit("x")
    tokens, feed = [], list(prompt)
    for _ in range(24):
        logits = loaded.runner.step([StepEntry("x", feed, [len(feed) - 1])])
        feed = [int(logits[0].argmax())]
        tokens += feed
    loaded.cache.release("x")
    ref = P.forward(cfg, w, list(prompt) + tokens)[len(prompt) - 1: -1]
    below = ref.max(-1).values - ref[range(24), tokens]
    assert float(below.max()) < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_command_line_and_trace_replay(folder, tmp_path, dtype):
    """As a user runs them: ``python -m qwen3_runtime_amd.cli --model DIR`` generates greedily, and
    ``bin/trace_run`` replays a mixed schedule of seven requests from standard input, four live at
    most, with a pool that only holds what is live and state slots for four."""
    import ast
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    raw, page = config_e()
    where = folder("e", dtype)
    cfg, w = P.load(where)
    prompt = [5, 17, 3, 140, 9, 77, 2]
    proc = subprocess.run([sys.executable, "-m", "qwen3_runtime_amd.cli", "--model", str(where), "--dtype", dtype,
                           "--prompt-tokens", *map(str, prompt), "--max-tokens", "8"],
                          capture_output=True, text=True, timeout=600, cwd=str(root))
    assert proc.returncode == 0, proc.stderr[-3000:]
    lines = dict(line.split(" ", 1) for line in proc.stdout.splitlines() if " " in line)
    tokens = ast.literal_eval(lines["runtime"])
    assert len(tokens) == 8
    logits = P.forward(cfg, w, prompt + tokens)[len(prompt) - 1: -1]
    below = logits.max(-1).values - logits[range(8), tokens]
    assert float(below.max()) < (1e-3 if dtype == "float32" else 2 * NOISE["e"] * float(logits.std()))

    reqs = traces.make_requests(raw["vocab"], [70, 9, 41, 100, 35, 1, 66], seed=6)
    steps = traces.mixed(reqs, seed=1)
    out = tmp_path / "logits"
    proc = subprocess.run([str(root / "bin" / "trace_run"), "--model", str(where), "--dtype", dtype, "--out", str(out),
                           "--max-tokens", str(traces.peak_tokens(steps))],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True,
                          timeout=600, cwd=str(root))
    assert proc.returncode == 0, proc.stderr[-3000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    got, pos = {}, {r: 0 for r in reqs}
    for s in steps:
        wanted = sum(len(e["want"]) for e in s["entries"])
        rows = np.fromfile(out / f"{s['step']}.f32", dtype="<f4").reshape(wanted, raw["vocab"]) if wanted else None
        i = 0
        for e in s["entries"]:
            for k in e["want"]:
                got[(e["id"], pos[e["id"]] + k)] = torch.from_numpy(rows[i].copy())
                i += 1
            pos[e["id"]] += len(e["tokens"])
    check(got, plain_logits(where, reqs), dtype, NOISE["e"])


# ------------------------------------------------------------------ configuration and plan
def test_config_reader_and_plan():
    from qwen3_runtime_amd.config.model import ConfigError
    from qwen3_runtime_amd.config.roserax import RoseraxConfig
    from qwen3_runtime_amd.engine.factory import build_model

    raw, _ = config_e()
    cfg = RoseraxConfig.from_dict(raw)
    assert RoseraxConfig.from_dict(cfg.to_dict()) == cfg
    assert (cfg.embedding_scale, cfg.logit_scale) == (9.0, 2.0)
    _, built = build_model(raw)
    plan = built.plan
    assert [len(s.cache_ids()) for s in plan.order] == [1, 1, 1, 1, 1]
    kinds = [plan.caches[s.cache_ids()[0]] for s in plan.order]
    assert [c.kind for c in kinds] == ["paged_kv"] * 4 + ["state"]
    # equal windows share a pool of pages; another window, and the latent's one head, have their own
    assert kinds[0].group_key() == kinds[2].group_key() != kinds[3].group_key()
    assert (kinds[1].heads, kinds[1].head_dim, kinds[1].window) == (1, 32 + 16, None)
    assert (kinds[0].window, kinds[0].keep_first) == (24, 6) and kinds[4].shape == (4, 32, 32)
    names = {d.file_name for d in built.tensor_decls()}
    assert {"embed", "final.norm", "l0.norm1b", "l0.norm2b", "l0.mix.q.norm", "l1.mix.dkv.norm", "l1.mlp.e15.down", "l1.mlp.router",
            "l4.mix.g", "l0.mlp.up"} <= names
    assert "l3.norm2" not in names and "l3.norm2" in plan.ignorable and "lm_head" not in names
    # what a file leaves out is not there: a key head per query head, values as wide as keys, none kept, one group
    small, _ = config_d()
    read = RoseraxConfig.from_dict(small)
    assert (read.layers[3].mixer.kv_heads, read.layers[3].mixer.vdim, read.layers[0].mixer.keep_first) == (2, 6, 0)
    assert read.logit_scale == 1.0 and RoseraxConfig.from_dict(config_b()[0]).embedding_scale == 1.0
    assert RoseraxConfig.from_dict(config_a()[0]).layers[3].feed_forward.groups == 1
    for bad in ({**raw, "layers": [{"type": "convolution", "mixer": {}, "mlp": None}]},
                {**raw, "layers": [{"type": "retention", "mixer": retention(2, 8, 8, (0.9,), 4, 10.0), "mlp": None}]},
                {**raw, "layers": [{"type": "latent_attention", "mixer": {**latent(2, 8, 4, 8, 8, 8, 0.1, 10.0), "rot": {"dims": 6, "base": 10.0}},
                                    "mlp": None}]},
                {**raw, "layers": [{"type": "attention", "mixer": attention(3, 2, 8, 8, 0.1, 4, 0), "mlp": None}]},
                {**raw, "layers": [{"type": "attention", "mixer": attention(2, 2, 8, 8, 0.1, 4, 0), "mlp": moe(8, 6, 3, (4, 2))}]},
                {**raw, "layers": []}, {k: v for k, v in raw.items() if k != "norm"}):
        with pytest.raises((ConfigError, ValueError, TypeError)):
            RoseraxConfig.from_dict(bad)


def test_presets_are_registered_and_run():
    from qwen3_runtime_amd.engine.factory import build_model
    from qwen3_runtime_amd.registry import preset_config, preset_names

    assert {"roserax_tiny_a", "roserax_tiny_b", "roserax_4b"} <= set(preset_names())
    for name in ("roserax_tiny_a", "roserax_tiny_b"):
        raw = preset_config(name)
        assert raw["architecture"] == "Roserax"
        build_model(raw)
