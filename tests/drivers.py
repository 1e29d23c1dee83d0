"""What the tests of single mechanisms share: the backends they run on, tensors from seeds, a
fetcher that hands a part its tensors from a dict, and a driver that steps one mixer through a
cache manager of its own as the engine's step function would."""

from __future__ import annotations

import pytest
import torch

from plain.ops_ref import TorchOps

GPU = pytest.mark.gpu
BACKENDS = [pytest.param(("cpu", "float32"), id="host-f32"),
            pytest.param(("cuda:0", "float32"), id="gpu-f32", marks=GPU),
            pytest.param(("cuda:0", "bfloat16"), id="gpu-bf16", marks=GPU)]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def make_ops(device):
    if device == "cpu":
        return TorchOps()
    from qwen3_runtime_amd.ops.hip import HipOps

    return HipOps()


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def tol(dtype):
    return dict(atol=3e-5, rtol=3e-5) if dtype == "float32" else dict(atol=4e-2, rtol=4e-2)


def in_steps(total, sizes, first=0):
    """Cut positions ``first .. total`` into portions of the given sizes, repeated."""
    out, p, i = [], first, 0
    while p < total:
        n = min(sizes[i % len(sizes)], total - p)
        out.append((p, n))
        p += n
        i += 1
    return out


class DictFetch:
    """Hands a part its tensors from a dict, placed as the loader would place them."""

    def __init__(self, tensors, device, dtype):
        self.t, self.device, self.dtype = tensors, device, dtype

    def matrix(self, name):
        return self.t[name].to(self.dtype).to(self.device).contiguous()

    def fused(self, names, dim=0):
        return torch.cat([self.t[n] for n in names], dim=dim).to(self.dtype).to(self.device).contiguous()

    def vector_f32(self, name):
        return self.t[name].float().to(self.device)

    def constant(self, tensor):
        return tensor.to(self.device).contiguous()


class MixerDriver:
    """Steps one mixer over requests' inputs through a cache manager of its own: pages reserved and
    committed as the engine's step does (a window gives its early pages back, except those of the
    first tokens it keeps), a state slot per request. Pages are poisoned before anyone holds them
    and whenever they go back to the pool."""

    def __init__(self, mixer, device, dt, ops, page, pages, max_requests=2):
        from qwen3_runtime_amd.cache import CacheManager

        self.mixer, self.device, self.dt, self.ops, self.page = mixer, device, dt, ops, page
        self.cache = CacheManager(mixer.cache_specs(), page_size=page, num_pages=pages, max_requests=max_requests,
                                  device=device, dtype=dt)
        self.slot = {}
        self._poison()

    def _poison(self):
        for g in self.cache.groups:
            held = {p for t in g.tables.values() for p in t if p >= 0}
            free = torch.tensor([p for p in range(g.pool.num_pages) if p not in held], dtype=torch.long, device=self.device)
            for i, store in enumerate(g.storage):
                store[:, free] = float("nan") if i % 2 == 0 else float("inf")

    def admit(self, rid):
        self.slot[rid] = self.cache.admit(rid)

    def release(self, rid):
        self.cache.release(rid)
        self._poison()

    def step(self, spans):
        """``spans``: [(request, its next rows [n, width])]. Returns their outputs, [n, width] each."""
        from qwen3_runtime_amd.parts.base import GroupView, StepContext

        cache, dev = self.cache, self.device
        rids = [r for r, _ in spans]
        starts = [cache.length(r) for r in rids]
        lens = [x.shape[0] for _, x in spans]
        for r, n in zip(rids, lens):
            cache.reserve(r, n)
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=dev)  # noqa: E731
        cu = [0]
        for n in lens:
            cu.append(cu[-1] + n)
        kv = [s + n for s, n in zip(starts, lens)]
        ctx = StepContext(ops=self.ops, dtype=self.dt, device=torch.device(dev), num_tokens=cu[-1], num_seqs=len(spans),
                          positions=i32([s + i for s, n in zip(starts, lens) for i in range(n)]), cu_q=i32(cu), kv_lens=i32(kv),
                          seq_of_token=i32([j for j, n in enumerate(lens) for _ in range(n)]),
                          state_slots=i32([self.slot[r] for r in rids]), first_span=i32([int(s == 0) for s in starts]),
                          q_lens_host=list(lens), kv_lens_host=kv, max_q_len=max(lens), max_kv_len=max(kv))
        groups = []
        for gi, g in enumerate(cache.groups):
            table = torch.full((len(rids), cache.table_width(rids)), -1, dtype=torch.int32)
            cache.fill_tables(gi, rids, table.numpy())
            slots = torch.cat([torch.from_numpy(cache.token_slots(gi, r, s, n)) for r, s, n in zip(rids, starts, lens)])
            groups.append(GroupView(g.page_size, g.window, table.to(dev), slots.to(dev), g.chunk, g.keep_first))
        ctx.groups = groups
        views = [cache.view(c, groups) for c in range(len(cache.specs))]
        out = self.mixer.forward(ctx, torch.cat([x for _, x in spans]).to(self.dt).to(dev),
                                 views[0] if len(views) == 1 else tuple(views))
        out = (out.sum(0) if out.dim() == 3 else out).float().cpu()
        for r, n in zip(rids, lens):
            cache.commit(r, n)
        self._poison()
        cache.check()
        return [out[a:b] for a, b in zip(cu[:-1], cu[1:])]

    def run(self, rid, h, cuts):
        """One request alone, cut at ``cuts`` [(start, n)]; returns [T, width]."""
        self.admit(rid)
        got = torch.cat([self.step([(rid, h[p: p + n])])[0] for p, n in cuts])
        self.release(rid)
        return got


def rounded(w, dt):
    return {n: x.to(dt).float() for n, x in w.items()}


def f64(w):
    return {n: x.double() for n, x in w.items()}
