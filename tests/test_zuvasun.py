"""Zuvasun: every mechanism alone against its plain function, and whole models under every cutting.

Each test runs with the plain torch ops on the CPU (which pins the host side: plan, packing,
pages, windows, a cache that two layers read, the loop) and with the HIP ops on the GPU (marked
``gpu``; float32 and bfloat16). The oracle is ``plain/zuvasun_plain.py``: whole sequences, no cache,
float64. Configurations are made here and differ from each other in every size and option, also
in values that a model may happen to make equal or 1. Where random weights would hide a fault (a
key far back, the edge of a window, a correction that changes the router's choice), one token's
key or value, or the correction, is made to stand out.
"""

from __future__ import annotations

import math

import pytest
import torch

import traces
from drivers import BACKENDS, DT, DictFetch, MixerDriver, f64, in_steps, make_ops, rnd, rounded
from plain import zuvasun_plain as P
from plain.ops_ref import TorchOps


def row_bound(want, dtype):
    """Per row: float32 sums' rounding; in bfloat16 a twentieth of the row's largest element (queries,
    probabilities and values rounded to 8 bits move a row by about a hundredth of it; where a marked
    token or a temperature makes the scores large, their rounding moves the probabilities by more)."""
    top = want.abs().amax(1)
    return 2e-4 + 2e-4 * top if dtype == "float32" else 0.05 + 0.05 * top


def assert_rows(got, want, dtype, what=""):
    worst = (got.double() - want).abs().amax(1) / row_bound(want, dtype)
    assert float(worst.max()) <= 1.0, (what, int(worst.argmax()), float(worst.max()))


# ------------------------------------------------------------------ rotation of neighbours, stretched frequencies
STRETCH = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}


@pytest.mark.parametrize("dims,base,scaling", [(16, 100.0, None), (16, 100.0, STRETCH), (6, 1e4, {**STRETCH, "factor": 1.0}),
                                               (24, 3e4, {"factor": 16.0, "original": 4096, "fast": 32.0, "slow": 2.0})])
def test_stretched_frequencies(dims, base, scaling):
    """The frequencies the mixer computes against the plain function's, and the ramp's two ends:
    fast pairs keep their frequency, slow ones have it divided by the factor."""
    from qwen3_runtime_amd.parts.latent import stretched_frequencies

    how = None if scaling is None else tuple(scaling[k] for k in ("factor", "original", "fast", "slow"))
    got, mag = stretched_frequencies(dims, base, how)
    want, want_mag = P.yarn_frequencies(dims, base, scaling)
    torch.testing.assert_close(got.double(), want, atol=0, rtol=1e-6)
    assert abs(mag - want_mag) < 1e-12
    plain = base ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)
    if scaling is None or scaling["factor"] == 1.0:
        torch.testing.assert_close(want, plain)
        assert mag == 1.0
    else:
        assert abs(float(want[0] / plain[0]) - 1.0) < 1e-9 and abs(float(want[-1] / plain[-1]) - 1.0 / scaling["factor"]) < 1e-9
        assert mag == pytest.approx(0.1 * math.log(scaling["factor"]) + 1.0)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("heads,width,dims,scaling", [(3, 16, 16, STRETCH), (2, 24, 6, None), (5, 8, 8, STRETCH), (1, 64, 32, None)])
def test_neighbours_turn_against_each_other(backend, heads, width, dims, scaling):
    """The rotating copy with pairs of neighbours, from columns of one matrix into columns of another,
    at positions up to several thousand."""
    from qwen3_runtime_amd.parts.latent import stretched_frequencies

    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    t, lead, out_lead = 40, 5, 3
    how = None if scaling is None else tuple(scaling[k] for k in ("factor", "original", "fast", "slow"))
    freq, mag = stretched_frequencies(dims, 300.0, how)
    pos = torch.tensor([0, 1, 2, 3, 63, 64, 65, 511, 4095, 6000] * 4, dtype=torch.int32)
    x = rnd(t, heads * (lead + width), seed=1).to(dt)
    out = torch.zeros(t, heads * (out_lead + width) + 2, dtype=dt, device=device)
    ops.rotate_half(x.to(device), lead + width, lead, out, out_lead + width, out_lead, heads, width, pos.to(device),
                    freq.to(device), neighbours=True, magnitude=mag)
    src = x.float().view(t, heads, lead + width)[:, :, lead:].double()
    want = P.rotate_pairs(src, pos.tolist(), dims, 300.0, scaling)
    got = out[:, : heads * (out_lead + width)].float().cpu().view(t, heads, out_lead + width)
    # the angle is a float32 product of position and frequency: its rounding grows with the position
    bound = dict(atol=2e-3, rtol=1e-3) if dtype == "float32" else dict(atol=3e-2, rtol=2e-2)
    torch.testing.assert_close(got[:, :, out_lead:].double(), want, **bound)
    assert float(got[:, :, :out_lead].abs().max()) == 0.0 and float(out[:, -2:].abs().max()) == 0.0
    if dims < width:
        assert torch.equal(got[:, :, out_lead + dims:], x.float().view(t, heads, lead + width)[:, :, lead + dims:])


# ------------------------------------------------------------------ attention through a latent, over a window
def latent_weights(width, n, d, r, dv, kv_rank, seed=0, own=True):
    s = 0.3
    w = {"q": rnd(n * (d + r), width, seed=seed + 1, scale=s), "uk": rnd(n * d, kv_rank, seed=seed + 6, scale=s),
         "uv": rnd(n * dv, kv_rank, seed=seed + 7, scale=s), "o": rnd(width, n * dv, seed=seed + 9, scale=s)}
    if own:
        w.update({"dkv": rnd(kv_rank + r, width, seed=seed + 4, scale=s), "dkv.norm": 1 + rnd(kv_rank, seed=seed + 5, scale=0.2)})
    return w


def latent_mixer(width, sizes, eps, w, device, dt, cache_window=..., own=True):
    from qwen3_runtime_amd.parts.latent import LatentAttention

    names = {n: n for n in ("q", "uk", "uv", "o")} | ({"dkv": "dkv", "dkv_norm": "dkv.norm"} if own else {})
    sc = sizes["rot"].get("scaling")
    window = (sizes.get("mask") or {}).get("size")
    mixer = LatentAttention(width, sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], None, sizes["kv_rank"],
                            sizes["scale"], eps, sizes["rot"]["dims"], sizes["rot"]["base"], output_gate=False, window=window,
                            cache_window=window if cache_window is ... else cache_window, rotation="pairs",
                            rot_scaling=None if sc is None else (sc["factor"], sc["original"], sc["fast"], sc["slow"]),
                            own_latent=own, tensors=names)
    mixer.load(DictFetch(w, device, dt))
    return mixer


def latent_sizes(n, d, r, dv, kv_rank, window, dims=None, base=200.0, scaling=None):
    rot = {"dims": r if dims is None else dims, "base": base}
    if scaling:
        rot["scaling"] = scaling
    sizes = {"heads": n, "dim": d, "rot_dim": r, "vdim": dv, "kv_rank": kv_rank, "scale": 0.6 / math.sqrt(d + r), "rot": rot}
    if window:
        sizes["mask"] = {"size": window}
    return sizes


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("n,d,r,dv,kv_rank,window,dims,scaling,page", [
    (4, 32, 16, 32, 48, 40, None, STRETCH, 16),
    (3, 16, 8, 24, 40, 21, 6, None, 8),        # fewer turning elements than the part has; a row of 48
    (1, 64, 64, 16, 64, 70, None, STRETCH, 16),  # one head, as many turning elements as plain ones
    (5, 24, 8, 8, 64, 9, 2, STRETCH, 8),       # one pair turns; a row of 72, no multiple of 16
    (2, 32, 16, 48, 112, 1, None, None, 16),   # a window of the query itself
    (6, 16, 32, 16, 32, None, None, STRETCH, 16),  # no window
    (8, 32, 32, 64, 96, 33, None, STRETCH, 32),
])
def test_latent_attention_over_a_window(backend, n, d, r, dv, kv_rank, window, dims, scaling, page):
    """The latent mixer (full-rank queries, neighbour pairs turned by stretched frequencies, a window)
    over pages that hold only the latent and the shared turning key part and go back to the pool
    behind the window: against the plain mixer, which builds every head's keys and values. One
    token's input is scaled: its latent is normed and stays, its turning key part grows, so the heads
    whose queries point its way give it nearly all their weight while they see it. The queries pass
    its window's edge one by one and inside a portion."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, eps = 56, 1e-5
    reach = window or 60
    t = 3 * reach + 60
    sizes = latent_sizes(n, d, r, dv, kv_rank, window, dims, scaling=scaling)
    w = rounded(latent_weights(width, n, d, r, dv, kv_rank), dt)
    h = rnd(t, width, seed=8)
    marked = t - reach - 25
    h[marked] *= 6.0
    h = h.to(dt).float()
    want, _ = P.latent_attention(h.double(), f64(w), sizes, eps)
    edge = marked + reach  # the first query that no longer sees the marked token (with a window)
    pages = -(-(reach + 64) // page) + 2 if window else -(-t // page)
    for cuts in (in_steps(edge - 3, (64, 5)) + [(p, 1) for p in range(edge - 3, edge + 4)] + [(edge + 4, t - edge - 4)],
                 in_steps(edge - 10, (7, 2, 30)) + [(edge - 10, 20)] + in_steps(t, (1,), edge + 10)):
        driver = MixerDriver(latent_mixer(width, sizes, eps, w, device, dt), device, dt, ops, page, pages)
        got = driver.run("a", h, cuts)
        assert driver.cache.groups[0].pool.num_free == pages
        assert_rows(got, want, dtype)
    if window and window > 1:
        assert (want[edge - 1] - want[edge]).abs().max() > 5 * float(row_bound(want, dtype)[edge - 1])  # the edge shows
        for other in (window - 1, window + 1):  # and a window one token off would show, in the last rows too
            off, _ = P.latent_attention(h.double(), f64(w), {**sizes, "mask": {"size": other}}, eps)
            assert (off - want).abs().amax(1).max() > 5 * float(row_bound(want, dtype).max())
    # the rotation takes part: turned the other way (a sign of the position wrong) the rows differ
    if window != 1:
        still, _ = P.latent_attention(h.double(), f64(w), {**sizes, "rot": {**sizes["rot"], "dims": 0}}, eps)
        assert (still - want).abs().amax(1).max() > 5 * float(row_bound(want, dtype).max())


class TwoReaders:
    """The layer that owns a latent cache and one that reads it, run one after the other on the same
    input as two steps of a plan's order would: outputs side by side."""

    def __init__(self, owner, reader):
        self.owner, self.reader = owner, reader

    def cache_specs(self):
        return self.owner.cache_specs()

    def forward(self, ctx, x, cache):
        from dataclasses import replace

        first = self.owner.forward(ctx, x, cache)
        second = self.reader.forward(ctx, x, replace(cache, writes=False))
        flat = lambda y: y.sum(0) if y.dim() == 3 else y  # noqa: E731
        return torch.cat([flat(first).float(), flat(second).float()], dim=1)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("own_window,read_window,page", [(13, 22, 8), (30, 7, 16), (None, 12, 8), (16, None, 16), (24, 24, 8)])
def test_a_layer_reads_the_latent_another_layer_cached(backend, own_window, read_window, page):
    """A second latent layer without ``dkv``: other heads, sizes, matrices and window, the first one's
    cached latent and turning key part. The cache keeps what the wider of the two windows sees."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, eps, t, kv_rank, r = 48, 1e-6, 130, 40, 8
    own = latent_sizes(3, 16, r, 24, kv_rank, own_window, scaling=STRETCH)
    read = latent_sizes(5, 8, r, 16, kv_rank, read_window, scaling=STRETCH)
    read["scale"] = 0.25
    w1 = rounded(latent_weights(width, 3, 16, r, 24, kv_rank, seed=0), dt)
    w2 = rounded(latent_weights(width, 5, 8, r, 16, kv_rank, seed=50, own=False), dt)
    keep = None if own_window is None or read_window is None else max(own_window, read_window)
    h = rnd(t, width, seed=3)
    h[60] *= 3.0
    h = h.to(dt).float()
    want1, shared = P.latent_attention(h.double(), f64(w1), own, eps)
    want2, _ = P.latent_attention(h.double(), f64(w2), read, eps, shared)
    want = torch.cat([want1, want2], dim=1)
    pair = TwoReaders(latent_mixer(width, own, eps, w1, device, dt, cache_window=keep),
                      latent_mixer(width, read, eps, w2, device, dt, cache_window=keep, own=False))
    pages = -(-t // page) if keep is None else -(-(keep + 40) // page) + 2
    for cuts in (in_steps(t, (40, 3, 2, 17, 1, 1, 1)), in_steps(t, (1,)), [(0, t)][: 1 if keep is None else 0] or in_steps(t, (33,))):
        driver = MixerDriver(pair, device, dt, ops, page, pages)
        got = driver.run("a", h, cuts)
        assert_rows(got, want, dtype)
    with pytest.raises(ValueError):
        latent_mixer(width, {**read, "mask": {"size": 50}}, eps, w2, device, dt, cache_window=20, own=False)


# ------------------------------------------------------------------ attention whose values are its keys
def key_value_weights(width, nq, nkv, d, seed=0):
    s = 0.3
    return {"q": rnd(nq * d, width, seed=seed + 1, scale=s), "k": rnd(nkv * d, width, seed=seed + 2, scale=s),
            "q.b": rnd(nq * d, seed=seed + 3, scale=0.2), "k.b": rnd(nkv * d, seed=seed + 4, scale=0.2),
            "q.norm": 1 + rnd(nq * d, seed=seed + 5, scale=0.2), "k.norm": 1 + rnd(nkv * d, seed=seed + 6, scale=0.2),
            "o": rnd(width, nq * d, seed=seed + 7, scale=s)}


def key_value_mixer(width, sizes, eps, w, device, dt):
    from qwen3_runtime_amd.parts.attention import GroupedQueryAttention

    names = {"q": "q", "k": "k", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "q_norm": "q.norm", "k_norm": "k.norm"}
    temp = sizes.get("q_temp")
    mixer = GroupedQueryAttention(width, sizes["heads"], sizes["kv_heads"], sizes["dim"], qk_norm_eps=eps, scale=sizes["scale"],
                                  qk_norm_scope="projection", values_are_keys=True, bias=True,
                                  q_temp=None if temp is None else (temp["coef"], temp["every"]), tensors=names)
    mixer.load(DictFetch(w, device, dt))
    return mixer


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("nq,nkv,d,temp,page", [
    (4, 2, 32, (0.5, 7), 16),
    (6, 2, 16, (0.8, 1), 8),      # the temperature grows at every position
    (2, 2, 64, None, 16),         # a key head per query head, no temperature
    (3, 1, 48, (0.25, 64), 8),    # ... which first moves at position 63
    (8, 1, 24, (0.5, 1000), 16),  # ... never within the sequence; heads of 24
    (2, 1, 128, (0.7, 16), 32),
])
def test_values_are_the_keys(backend, nq, nkv, d, temp, page):
    """Biases, one norm over all query heads and one over all key heads, the queries' temperature, no
    rotation, every earlier key in sight, the keys as projected for values: against the plain mixer,
    in portions down to two tokens and token by token, a second request beside the first in other
    steps. An early token's input is scaled: its normed key stays, its value, the raw key, grows,
    and shows in every later row, hundreds of keys on."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, eps, t = 40, 1e-5, 330
    sizes = {"heads": nq, "kv_heads": nkv, "dim": d, "scale": 1.0 / math.sqrt(d)}
    if temp:
        sizes["q_temp"] = {"coef": temp[0], "every": temp[1]}
    w = rounded(key_value_weights(width, nq, nkv, d), dt)
    plainer = rnd(t, width, seed=8).to(dt).float()
    h = plainer.clone()
    h[5] *= 200.0
    h = [h.to(dt).float(), rnd(70, width, seed=9).to(dt).float()]
    want = [P.key_value_attention(x.double(), f64(w), sizes, eps) for x in h]
    without = P.key_value_attention(plainer.double(), f64(w), sizes, eps)
    far = (without - want[0])[100:].abs().amax(1) / row_bound(want[0], dtype)[100:]
    assert float(far.max()) > 5  # the far key's value shows, a hundred and more keys on
    if temp and temp[1] < t:
        cold = P.key_value_attention(h[0].double(), f64(w), {**sizes, "q_temp": {"coef": temp[0], "every": temp[1] + 1}}, eps)
        moved = (cold - want[0]).abs().amax(1) / row_bound(want[0], "float32")
        assert float(moved.max()) > 5  # where the temperature moves shows (to the float32 runs, which hold it to rounding)
    mixer = key_value_mixer(width, sizes, eps, w, device, dt)
    pages = -(-t // page) + -(-70 // page)
    driver = MixerDriver(mixer, device, dt, ops, page, pages)
    driver.admit("a")
    driver.admit("b")
    got = {"a": [], "b": []}
    plan = in_steps(t, (64, 2, 7, 33, 1, 1, 120))
    other = in_steps(70, (1, 1, 9, 2))
    for i in range(max(len(plan), len(other))):
        spans = []
        if i < len(plan):
            spans.append(("a", h[0][plan[i][0]: plan[i][0] + plan[i][1]]))
        if i < len(other):
            spans.append(("b", h[1][other[i][0]: other[i][0] + other[i][1]]))
        for (rid, _), out in zip(spans, driver.step(spans)):
            got[rid].append(out)
    driver.release("a")
    driver.release("b")
    assert driver.cache.groups[0].pool.num_free == pages
    assert_rows(torch.cat(got["a"]), want[0], dtype, "beside another")
    assert_rows(torch.cat(got["b"]), want[1], dtype, "the other")
    # the pages are used again, token by token from the start
    driver = MixerDriver(mixer, device, dt, ops, page, -(-100 // page))
    assert_rows(driver.run("c", h[0][:100], in_steps(100, (1,))), want[0][:100], dtype, "one by one")
    # long portions, whose values are stored eight tokens at a time: from a page's start, and from its third place
    for cuts in ([(0, t)], [(0, 3), (3, 300), (303, t - 303)]):
        driver = MixerDriver(mixer, device, dt, ops, page, -(-t // page))
        assert_rows(driver.run("d", h[0], cuts), want[0], dtype, f"portions {cuts}")


def test_attention_options_that_do_not_go_together():
    from qwen3_runtime_amd.parts.attention import GroupedQueryAttention

    names = {"q": "q", "k": "k", "o": "o", "q_norm": "qn", "k_norm": "kn"}
    with pytest.raises(NotImplementedError):
        GroupedQueryAttention(32, 2, 1, 16, qk_norm_eps=1e-5, values_are_keys=True, tensors=names)
    with pytest.raises(ValueError):
        GroupedQueryAttention(32, 2, 1, 16, qk_norm_eps=1e-5, qk_norm_scope="projection", values_are_keys=True, value_dim=8, tensors=names)
    with pytest.raises(ValueError):
        GroupedQueryAttention(32, 2, 1, 16, qk_norm_eps=None, qk_norm_scope="projection", tensors=names)
    with pytest.raises(ValueError):
        GroupedQueryAttention(32, 2, 1, 16, qk_norm_eps=1e-5, qk_norm_scope="projection", q_temp=(0.5, 0), tensors=names)
    decls = GroupedQueryAttention(32, 2, 1, 16, qk_norm_eps=1e-5, qk_norm_scope="projection", values_are_keys=True, bias=True,
                                  tensors={**names, "q_bias": "qb", "k_bias": "kb"}).tensor_decls()
    assert {d.file_name: d.shape for d in decls} == {"q": (32, 32), "k": (16, 32), "o": (32, 32), "qb": (32,), "kb": (16,),
                                                     "qn": (32,), "kn": (16,)}


# ------------------------------------------------------------------ the mixture of squared-relu experts
def mixture_weights(width, ff, experts, seed=0):
    w = {"router": rnd(experts, width, seed=seed + 1, scale=0.5), "correction": rnd(experts, seed=seed + 2, scale=0.3)}
    for e in range(experts):
        w[f"e{e}.up"] = rnd(ff, width, seed=seed + 10 + 2 * e, scale=0.3)
        w[f"e{e}.down"] = rnd(width, ff, seed=seed + 11 + 2 * e, scale=0.3)
    return w


def mixture_part(width, ff, experts, top, scale, w, device, dt):
    from qwen3_runtime_amd.parts.moe import RoutedSwiGLU

    names = {"router": "router", "correction": "correction", "up": "e{e}.up", "down": "e{e}.down"}
    part = RoutedSwiGLU(width, ff, experts, top, router_bias=False, scoring="softmax_all", activation="relu2", correction=True,
                        renormalise=True, weight_scale=scale, tensors=names)
    part.load(DictFetch(w, device, dt))
    return part


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("experts,top,scale", [(10, 3, 2.0), (5, 1, 1.0), (4, 4, 0.5), (70, 6, 1.7)])
def test_the_correction_moves_the_choice_and_not_the_weights(backend, experts, top, scale):
    """The router alone. A correction of several times the scores' spread decides who is chosen;
    the weights are the chosen experts' own scores, renormalised and scaled."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    width, t = 48, 60
    x = rnd(t, width, seed=1).to(dt)
    router = rnd(experts, width, seed=2, scale=0.3).to(dt).float()
    correction = rnd(experts, seed=3, scale=0.5)
    index, weight = ops.route_top(x.to(device), router.to(device), None, top, scoring="softmax_all",
                                  correction=correction.to(device), renormalise=True, weight_scale=scale)
    want_i, want_w = P.route(x.double(), router.double(), correction.double(), top, scale)
    plain_i, _ = P.route(x.double(), router.double(), torch.zeros(experts, dtype=torch.float64), top, scale)
    if top < experts:
        assert (want_i.sort(-1).values != plain_i.sort(-1).values).any()  # the correction changes somebody's experts
    got_i, order = index.cpu().long().sort(-1)
    ref_i, ref_order = want_i.sort(-1)
    assert torch.equal(got_i, ref_i)
    torch.testing.assert_close(weight.cpu().double().gather(1, order), want_w.gather(1, ref_order), atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(weight.cpu().sum(-1).double(), torch.full((t,), scale, dtype=torch.float64), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width,ff,experts,top,scale", [(48, 40, 6, 2, 1.5), (64, 24, 10, 3, 2.0), (40, 56, 4, 4, 0.5), (72, 16, 5, 1, 1.0)])
def test_mixture_of_squared_relu_experts(backend, width, ff, experts, top, scale):
    """Router and experts together at every step size (one token, a few, tens, hundreds: pair by
    pair, expert by expert on the device, expert by expert through the engine's products)."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    w = rounded(mixture_weights(width, ff, experts), dt)
    w["router"] = w["router"] * 0.2  # scores far from a tie in 8 bits
    part = mixture_part(width, ff, experts, top, scale, w, device, dt)
    mlp = {"router": {"experts": experts, "top": top, "scale": scale}}
    ctx = lambda: None  # noqa: E731
    for t in (1, 3, 17, 70, 300):
        x = rnd(t, width, seed=t).to(dt)
        holder = type("Ctx", (), {"ops": ops, "num_tokens": t, "dtype": dt})()
        got = part.forward(holder, x.to(device))
        got = (got.sum(0) if got.dim() == 3 else got).float().cpu()
        want = P.mixture(x.double(), f64(w), mlp)
        assert_rows(got, want, dtype, f"{t} tokens")


# ------------------------------------------------------------------ the scaled sum into the stream
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("width", [70, 200, 4100])
def test_scaled_outputs_join_the_stream_in_one_sum(backend, width):
    """``x += s1 * y1 + s2 * y2`` and the norm of the sum: one term, two terms, a term in planes, all rows
    and chosen rows (which leave the stream alone)."""
    device, dtype = backend
    ops, dt = make_ops(device), DT[dtype]
    t, eps = 9, 1e-5
    x0 = rnd(t, width, seed=1)
    y1, y2 = rnd(t, width, seed=2).to(dt), rnd(3, t, width, seed=3)
    s1, s2, w = 1 + rnd(width, seed=4, scale=0.3), rnd(width, seed=5), 1 + rnd(width, seed=6, scale=0.2)
    dev = lambda a: a.to(device)  # noqa: E731
    for parts, total in (([(y1, s1)], y1.double() * s1), ([(y1, s1), (y2, s2)], y1.double() * s1 + y2.double().sum(0) * s2),
                         ([(y2[0].to(dt), s2), (y1, s1)], y2[0].to(dt).double() * s2 + y1.double() * s1)):
        new = x0.double() + total
        want = P.rms_norm(new, w.double(), eps)
        for rows in (None, torch.tensor([7, 0, 3], dtype=torch.int32)):
            x = dev(x0.clone())
            got = ops.scaled_add_rmsnorm(x, [(dev(y), dev(s)) for y, s in parts], dev(w), eps, dt,
                                         None if rows is None else dev(rows))
            ref = want if rows is None else want[rows.long()]
            torch.testing.assert_close(got.float().cpu().double(), ref, **(dict(atol=2e-5, rtol=2e-5) if dtype == "float32"
                                                                          else dict(atol=2e-2, rtol=2e-2)))
            torch.testing.assert_close(x.cpu().double(), new if rows is None else x0.double(), atol=1e-5, rtol=1e-6)


# ------------------------------------------------------------------ whole models
def latent(n, d, r, dv, kv_rank, scale, window=None, dims=None, base=1000.0, scaling=None, kv_from=None):
    m = {"heads": n, "dim": d, "rot_dim": r, "vdim": dv, "kv_rank": kv_rank, "scale": scale,
         "rot": {"dims": r if dims is None else dims, "base": base}}
    if scaling:
        m["rot"]["scaling"] = scaling
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def attention(nq, nkv, d, scale, temp=None):
    m = {"heads": nq, "kv_heads": nkv, "dim": d, "vdim": d, "scale": scale}
    if temp:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return m


def moe(ff, experts, top, scale):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale}}


def model(vocab, width, eps, layers):
    return {"architecture": "Zuvasun", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "layers": [{"type": kind, "mixer": mixer, "mlp": mlp} for kind, mixer, mlp in layers]}


def config_a():
    """Every kind of layer; the reader's window is the wider one; a layer without feed-forward."""
    s = {"factor": 8.0, "original": 32, "fast": 4.0, "slow": 1.0}
    return model(210, 80, 1e-5, [
        ("latent_attention", latent(3, 16, 16, 24, 32, 0.2, 13, scaling=s), moe(24, 10, 3, 2.0)),
        ("attention", attention(6, 2, 16, 0.3, (0.4, 5)), moe(40, 6, 2, 1.5)),
        ("latent_attention", latent(5, 8, 16, 16, 32, 0.3, 22, scaling=s, kv_from=0), None),
        ("attention", attention(4, 4, 32, 0.15), moe(24, 10, 3, 2.0)),
    ]), 16


def config_b():
    """A latent without window, read by two layers with windows; one expert a token; all experts a token."""
    return model(150, 64, 1e-6, [
        ("latent_attention", latent(2, 32, 8, 16, 24, 0.15, None, dims=6, base=1e4), None),
        ("latent_attention", latent(4, 16, 8, 32, 24, 0.25, 9, dims=6, base=1e4, kv_from=0), moe(32, 5, 1, 1.0)),
        ("attention", attention(2, 1, 48, 0.12, (1.0, 1)), moe(48, 4, 4, 0.5)),
        ("latent_attention", latent(1, 8, 8, 8, 24, 0.4, 30, dims=6, base=1e4, kv_from=0), moe(16, 3, 2, 3.0)),
    ]), 8


def config_c():
    """Latent layers alone, windows all round: nothing grows with the length. Two owners, each with a reader."""
    s = {"factor": 2.0, "original": 16, "fast": 2.0, "slow": 0.5}
    return model(97, 48, 1e-5, [
        ("latent_attention", latent(2, 16, 8, 16, 40, 0.3, 17, scaling=s), moe(16, 4, 2, 1.0)),
        ("latent_attention", latent(3, 8, 16, 8, 16, 0.3, 6, base=50.0), moe(16, 4, 2, 1.0)),
        ("latent_attention", latent(3, 8, 16, 24, 16, 0.2, 11, base=50.0, kv_from=1), None),
        ("latent_attention", latent(4, 8, 8, 8, 40, 0.5, 5, scaling=s, kv_from=0), moe(8, 7, 3, 0.7)),
    ]), 8


def config_d():
    """Sizes that are multiples of nothing."""
    return model(131, 50, 1e-5, [
        ("attention", attention(3, 1, 10, 0.4, (0.3, 3)), moe(18, 3, 2, 1.3)),
        ("latent_attention", latent(3, 6, 6, 10, 14, 0.5, 7, dims=4, base=30.0), moe(10, 5, 2, 0.9)),
        ("latent_attention", latent(2, 10, 6, 6, 14, 0.4, 12, dims=4, base=30.0, kv_from=1), None),
    ]), 8


def config_g():
    """Layers of a real model's proportions, narrow: heads of 64 and 128, a latent row of 160."""
    s = {"factor": 4.0, "original": 128, "fast": 16.0, "slow": 1.0}
    return model(500, 256, 1e-6, [
        ("latent_attention", latent(4, 64, 32, 64, 128, 0.1, 100, base=1e4, scaling=s), moe(128, 8, 2, 2.0)),
        ("latent_attention", latent(4, 64, 32, 64, 128, 0.1, 100, base=1e4, scaling=s, kv_from=0), moe(128, 8, 2, 2.0)),
        ("attention", attention(4, 2, 128, 0.2, (0.4, 100)), moe(128, 8, 2, 2.0)),
        ("attention", attention(8, 2, 64, 0.25, (0.4, 100)), moe(128, 8, 2, 2.0)),
    ]), 16


CONFIGS = {"a": config_a, "b": config_b, "c": config_c, "d": config_d, "g": config_g}
LENGTHS = {"a": [70, 1, 23], "b": [64, 40, 2], "c": [90, 5], "d": [37, 20], "g": [330, 40]}
NOISE = {"a": 0.2, "b": 0.2, "c": 0.2, "d": 0.2, "g": 0.2}


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    """Model folders with random weights, written once per configuration. For runs in bfloat16 the
    corrections of the routers' choice are spread out further than scores can differ (a
    permutation of multiples of 1.5 per layer): the choice is then the correction's, and no expert is
    chosen on a call that 8 bits could turn, which would move that position's logits by a large
    part of their spread; the weights are still the scores'. The choice by scores is held to the
    plain one in float32 here, and in both types in the router's own test."""
    from safetensors.torch import load_file, save_file

    from qwen3_runtime_amd.weights import write_model_folder

    made = {}

    def get(name, dtype="float32"):
        key = (name, dtype == "bfloat16")
        if key not in made:
            raw, _ = CONFIGS[name]()
            where = write_model_folder(tmp_path_factory.mktemp("zuvasun_" + name), raw, seed=41 + len(CONFIGS) + sorted(CONFIGS).index(name),
                                       std=0.03 if name == "g" else 0.08, norm_jitter=0.2)
            if key[1]:
                tensors = load_file(str(where / "model.safetensors"))
                for i, (tensor_name, x) in enumerate(sorted(tensors.items())):
                    if tensor_name.endswith(".mlp.correction"):
                        order = torch.randperm(x.numel(), generator=torch.Generator().manual_seed(i))
                        tensors[tensor_name] = (1.5 * order).to(x.dtype)
                save_file(tensors, str(where / "model.safetensors"))
            made[key] = where
        return made[key]

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
    own spread: no position over ``noise``, one in a hundred aside (an expert chosen on a close call),
    and the root mean square under a quarter of it. A wrong window, cache or portion shows in
    float32, where the bound is rounding."""
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
@pytest.mark.parametrize("name", ["a", "b", "c", "d"])
@pytest.mark.parametrize("cut", ["whole", "tail_one_by_one", "portions", "mixed"])
def test_cuttings_match_plain(folder, backend, name, cut):
    """Whole prompts; the last tokens one by one (across window edges); portions down to two tokens;
    up to four live requests mixed in a pool of the peak's size, so that pages are used again
    (freed pages are poisoned first)."""
    raw, page = CONFIGS[name]()
    reqs = traces.make_requests(raw["vocab"], LENGTHS[name] + ([30, 9] if cut == "mixed" else []), seed=5)
    steps = getattr(traces, cut)(reqs)
    loaded = load(folder(name, backend[1]), page, traces.peak_tokens(steps, unit=page) // page, backend)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, plain_logits(folder(name, backend[1]), reqs), backend[1], NOISE[name])


def test_the_stream_after_every_layer_matches_plain(folder):
    """Layer by layer: the engine's residual stream after each layer (the pending scaled sum
    applied) against the plain one, for a short prompt."""
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
            total = residual.double()
            for y, scale in pending.parts:
                total = total + (y.double().sum(0) if y.dim() == 3 else y.double()) * scale.double()
            seen.append(total)
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
    reqs = traces.make_requests(raw["vocab"], LENGTHS["g"], seed=9)
    want = plain_logits(folder("g", dtype), reqs)
    for steps in (traces.whole(reqs), traces.mixed(reqs, seed=2, decode_tail=12)):
        loaded = load(folder("g", dtype), page, traces.peak_tokens(steps, unit=page) // page, ("cuda:0", dtype))
        check(traces.replay(loaded, steps, poison_freed=True), want, dtype, NOISE["g"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_long_decoding_in_a_pool_of_one_window(folder, backend):
    """A request far longer than the pool, decoded token by token: every cache is windowed and gives
    its pages back as the window passes, also the one that two layers read."""
    raw, page = config_c()
    reqs = traces.make_requests(raw["vocab"], [300], seed=8)
    steps = traces.tail_one_by_one(reqs, tail=290)
    loaded = load(folder("c", backend[1]), page, 5, backend)   # a window of 17 touches 3 pages, a step's tokens one more
    assert all(g.window is not None for g in loaded.cache.groups)
    got = traces.replay(loaded, steps, poison_freed=True)
    check(got, plain_logits(folder("c", backend[1]), reqs), backend[1], NOISE["c"])


@pytest.mark.parametrize("backend", BACKENDS)
def test_batches_of_unequal_requests_against_each_alone(folder, backend):
    """A long prompt's portion, a short prompt and two single tokens in one step give what each gives
    alone (float32: to the last bits)."""
    from qwen3_runtime_amd.engine.batch import StepEntry

    raw, page = config_a()
    reqs = traces.make_requests(raw["vocab"], [61, 9, 30, 25], seed=2)
    name = folder("a", backend[1])

    def run(batches):
        loaded = load(name, page, 24, backend)
        out = {}
        for rid in reqs:
            loaded.cache.admit(rid)
        done = {rid: 0 for rid in reqs}
        for batch in batches:
            entries = [StepEntry(rid, reqs[rid][done[rid]: done[rid] + n], [n - 1]) for rid, n in batch]
            logits = loaded.runner.step(entries).float().cpu()
            for (rid, n), row in zip(batch, logits):
                done[rid] += n
                out[(rid, done[rid] - 1)] = row
        return out

    first = [[("r2", 29)], [("r3", 24)]]
    together = run(first + [[("r0", 40), ("r1", 9), ("r2", 1), ("r3", 1)], [("r0", 21)]])
    alone = run(first + [[("r0", 40)], [("r1", 9)], [("r2", 1)], [("r3", 1)], [("r0", 21)]])
    assert set(together) == set(alone)
    if backend[1] == "float32":
        traces.compare(together, alone, atol=2e-5, rtol=2e-5)
    else:
        check(together, alone, "bfloat16", NOISE["a"])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,graphs", [("float32", False), ("bfloat16", True), ("bfloat16", False)])
@pytest.mark.parametrize("name", ["a", "b"])
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
    """The engine's own scheduler (admission, portions under a small token budget, two requests at
    a time of three) and step function over the plain torch ops; the greedy choice is made here,
    the sampler being a kernel."""
    from qwen3_runtime_amd.config.engine import EngineConfig
    from qwen3_runtime_amd.engine.batch import StepEntry
    from qwen3_runtime_amd.engine.request import Request
    from qwen3_runtime_amd.engine.scheduler import Scheduler

    raw, page = config_d()
    cfg, w = P.load(folder("d"))
    loaded = load(folder("d"), page, 32, ("cpu", "float32"), max_seqs=2)
    prompts = list(traces.make_requests(raw["vocab"], [12, 3, 30], seed=4).values())
    engine = EngineConfig(page_size=page, num_pages=32, max_num_seqs=2, max_num_batched_tokens=10, dtype="float32", device="cpu")
    scheduler = Scheduler(engine, loaded.cache, 100_000)
    lengths = [16, 9, 16]  # the second ends first, and the third one's prompt is read beside the first one's decoding
    requests = [Request(list(p), max_tokens=n) for p, n in zip(prompts, lengths)]
    for r in requests:
        scheduler.add(r)
    sizes = set()
    while not scheduler.is_finished():
        batch = scheduler.schedule()
        entries, caught = [], []
        for r in batch:
            at = loaded.cache.length(r.request_id)
            upto = at + r.grant
            caught.append(upto >= len(r.token_ids))
            entries.append(StepEntry(r.request_id, r.token_ids[at:upto], [r.grant - 1] if caught[-1] else []))
        sizes.add(tuple(sorted(r.grant for r in batch)))
        logits = loaded.runner.step(entries)
        rows = iter(logits if logits is not None else [])
        scheduler.settle(batch, [int(next(rows).argmax()) if c else None for c in caught])
    assert any(len(x) == 2 and x[0] == 1 and x[1] > 1 for x in sizes)  # a decoded token beside a prompt's portion
    for prompt, r, n in zip(prompts, requests, lengths):
        tokens = list(r.output_tokens)
        assert len(tokens) == n
        ref = P.forward(cfg, w, list(prompt) + tokens)[len(prompt) - 1: -1]
        below = ref.max(-1).values - ref[range(n), tokens]
        assert float(below.max()) < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_command_line_and_trace_replay(folder, tmp_path, dtype):
    """As a user runs them: ``python -m qwen3_runtime_amd.cli --model DIR`` generates greedily, and
    ``bin/trace_run`` replays a mixed schedule of seven requests from standard input, four live at
    most, with a pool that only holds what is live."""
    import ast
    import json
    import subprocess
    import sys
    from pathlib import Path

    import numpy as np

    root = Path(__file__).resolve().parents[1]
    raw, page = config_a()
    where = folder("a", dtype)
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
    assert float(below.max()) < (1e-3 if dtype == "float32" else 2 * NOISE["a"] * float(logits.std()))

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
    check(got, plain_logits(where, reqs), dtype, NOISE["a"])


# ------------------------------------------------------------------ configuration and plan
def test_config_reader_and_plan():
    from qwen3_runtime_amd.config.model import ConfigError
    from qwen3_runtime_amd.config.zuvasun import ZuvasunConfig
    from qwen3_runtime_amd.engine.factory import build_model

    raw, _ = config_a()
    cfg = ZuvasunConfig.from_dict(raw)
    assert ZuvasunConfig.from_dict(cfg.to_dict()) == cfg
    _, built = build_model(raw)
    plan = built.plan
    # three caches for four layers: the third layer reads the first one's, which keeps the wider window
    assert [(s.cache, s.writes_cache) for s in plan.order] == [(0, True), (1, True), (0, False), (2, True)]
    assert (plan.caches[0].heads, plan.caches[0].head_dim, plan.caches[0].window) == (1, 32 + 16, 22)
    assert (plan.caches[1].heads, plan.caches[1].head_dim, plan.caches[1].window) == (2, 16, None)
    assert built.blocks[0].mixer.window == 13 and built.blocks[2].mixer.window == 22
    names = {d.file_name for d in built.tensor_decls()}
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.ls1", "l0.ls2", "l0.mix.dkv", "l0.mix.dkv.norm", "l1.mix.q.b",
            "l1.mix.k.norm", "l1.mlp.correction", "l0.mlp.e9.down", "l2.mix.uk", "l2.ls1"} <= names
    assert not {"l2.mix.dkv", "l2.mix.dkv.norm", "l2.ls2", "l1.mix.v", "l0.mlp.e0.gate", "l0.norm2"} & names
    assert "l2.ls2" in plan.ignorable
    # what a file leaves out is not there
    read = ZuvasunConfig.from_dict(config_b()[0])
    assert read.layers[0].mixer.window is None and read.layers[0].mixer.rot.scaling is None
    assert read.layers[2].mixer.kv_heads == 1 and ZuvasunConfig.from_dict(raw).layers[3].mixer.temp_coef is None
    bare = model(50, 16, 1e-5, [("attention", {"heads": 2, "dim": 8, "scale": 0.3},
                                 {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 2, "top": 1}})])
    read = ZuvasunConfig.from_dict(bare)
    assert read.layers[0].mixer.kv_heads == 2 and read.layers[0].feed_forward.scale == 1.0
    lat = latent(2, 8, 4, 8, 8, 0.1)
    for bad in ({**raw, "layers": [{"type": "retention", "mixer": {}, "mlp": None}]},
                model(50, 16, 1e-5, [("latent_attention", {**lat, "rot": {"dims": 6, "base": 10.0}}, None)]),
                model(50, 16, 1e-5, [("latent_attention", {**lat, "kv_from": 0}, None)]),          # reads itself
                model(50, 16, 1e-5, [("latent_attention", lat, None), ("latent_attention", {**lat, "kv_rank": 16, "kv_from": 0}, None)]),
                model(50, 16, 1e-5, [("attention", attention(2, 2, 8, 0.1), None), ("latent_attention", {**lat, "kv_from": 0}, None)]),
                model(50, 16, 1e-5, [("latent_attention", lat, None), ("latent_attention", {**lat, "kv_from": 0}, None),
                                     ("latent_attention", {**lat, "kv_from": 1}, None)]),           # a reader's reader
                model(50, 16, 1e-5, [("attention", attention(3, 2, 8, 0.1), None)]),
                model(50, 16, 1e-5, [("attention", {**attention(2, 2, 8, 0.1), "vdim": 4}, None)]),
                model(50, 16, 1e-5, [("attention", attention(2, 2, 8, 0.1), moe(8, 2, 3, 1.0))]),
                model(50, 16, 1e-5, [("attention", attention(2, 2, 8, 0.1), {"kind": "dense", "ff": 8})]),
                {**raw, "layers": []}, {k: v for k, v in raw.items() if k != "norm"}):
        with pytest.raises((ConfigError, ValueError, TypeError)):
            ZuvasunConfig.from_dict(bad)


def test_presets_are_registered_and_run():
    from qwen3_runtime_amd.engine.factory import build_model
    from qwen3_runtime_amd.registry import preset_config, preset_names

    assert {"zuvasun_tiny_a", "zuvasun_tiny_b"} <= set(preset_names())
    for name in ("zuvasun_tiny_a", "zuvasun_tiny_b"):
        raw = preset_config(name)
        assert raw["architecture"] == "Zuvasun"
        build_model(raw)
