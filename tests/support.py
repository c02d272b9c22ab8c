"""Shared helpers of the GPU parity tests: one layer's pages for several sequences over shuffled page tables, written
through the kernels module under test, read back through the CPU oracle."""
import math

import torch

from oracle import append as oracle_append
from oracle import attend as oracle_attend

STORE = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp8": torch.float8_e4m3fn, "fp8:row": torch.float8_e4m3fn,
         "int8": torch.int8}
KINDS = list(STORE)


def kernels():
    import crit_amd.paged_kv_attention as pk
    return pk


def bits(t):
    return t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t


class Cache:
    """As the reference's test helper (kernels/techniques/attention/paged-kv-attention/tests/
    test_paged_kv_attention.py:19-68): pages of one layer, each sequence over shuffled pages, written by pk.write."""

    def __init__(self, kind, hkv, d, dv, page, lengths, seed=0, multipliers=(0.02, 0.03), dev="cuda", scale=1.0,
                 extra_pages=3):
        self.pk = kernels()
        g = torch.Generator().manual_seed(seed)
        self.kind, self.hkv, self.d, self.dv, self.page, self.dev = kind, hkv, d, dv, page, dev
        self.multipliers = multipliers if kind == "fp8" else (1.0, 1.0)
        width = max(math.ceil(n / page) for n in lengths) + 1
        n_pages = width * len(lengths) + extra_pages
        self.k = torch.zeros(n_pages, page, hkv, d, dtype=STORE[kind], device=dev)
        self.v = torch.zeros(n_pages, page, hkv, dv, dtype=STORE[kind], device=dev)
        self.ks = self.vs = None
        if kind in ("fp8:row", "int8"):
            self.ks = torch.zeros(n_pages, page, hkv, dtype=torch.float32, device=dev)
            self.vs = torch.zeros_like(self.ks)
        order = torch.randperm(n_pages, generator=g)
        self.tables = order[:width * len(lengths)].view(len(lengths), width).to(torch.int32).to(dev)
        self.lengths = list(lengths)
        for s, n in enumerate(lengths):
            keys = (torch.randn(n, hkv, d, generator=g) * scale).to(dev)
            values = (torch.randn(n, hkv, dv, generator=g) * scale).to(dev)
            self.write(s, 0, keys, values)

    def slots(self, s, positions):
        positions = torch.as_tensor(positions, device=self.dev)
        return self.tables[s][positions // self.page].long() * self.page + positions % self.page

    def write(self, s, start, keys, values):
        slots = self.slots(s, torch.arange(start, start + keys.shape[0], device=self.dev))
        m = self.multipliers
        if torch.is_tensor(m):
            m = m.to(self.dev)
        self.pk.write(keys, values, slots, self.k, self.v, self.kind, self.ks, self.vs, multipliers=m)

    def cpu(self):
        """(key pages, value pages, key scales, value scales, tables) on the CPU, for the oracle."""
        c = lambda t: None if t is None else t.cpu()
        return c(self.k), c(self.v), c(self.ks), c(self.vs), self.tables.cpu()

    def want(self, q, s, first, count, scale=None, sliding=0, parents=None, blocks=None, block_size=None, fresh=None,
             int8_qk=False):
        """The oracle's float64 (out, lse) of one window row over the STORED values."""
        k, v, ks, vs, tables = self.cpu()
        q_dtype = torch.float16 if self.kind == "fp16" else torch.bfloat16
        m = self.multipliers
        if torch.is_tensor(m):
            m = (m[0].cpu(), m[1].cpu())
        return oracle_attend.window_reference(q.cpu().float(), k, v, self.kind, tables[s], first, count, self.page,
                                              scale if scale is not None else self.d ** -0.5, ks, vs, m,
                                              sliding=sliding, q_dtype=q_dtype, parents=parents, blocks=blocks,
                                              block_size=block_size, fresh=fresh, int8_qk=int8_qk)

    def attend(self, q, rows, starts, firsts, columns, **kw):
        q_dtype = torch.float16 if self.kind == "fp16" else torch.bfloat16
        t = lambda x, dt: x if torch.is_tensor(x) else torch.tensor(x, dtype=dt, device=self.dev)
        m = self.multipliers
        if torch.is_tensor(m):
            m = m.to(self.dev)
        return self.pk.attend(q.to(q_dtype), self.k, self.v, self.kind, self.tables, t(rows, torch.int32),
                              t(starts, torch.int32), t(firsts, torch.int64), columns, self.page,
                              key_scales=self.ks, value_scales=self.vs, multipliers=m, **kw)


def rand_q(tokens, hq, d, seed, dev="cuda"):
    return torch.randn(tokens, hq, d, generator=torch.Generator().manual_seed(seed)).to(dev)


def expected_pages(kind, keys, values, slots, n_slots, multipliers):
    """The oracle's pages after one write into zeroed storage: (k, v, ks, vs) on the CPU."""
    hkv, d, dv = keys.shape[1], keys.shape[2], values.shape[2]
    k = torch.zeros(n_slots, hkv, d, dtype=STORE[kind])
    v = torch.zeros(n_slots, hkv, dv, dtype=STORE[kind])
    ks = vs = None
    if kind in ("fp8:row", "int8"):
        ks, vs = torch.zeros(n_slots, hkv), torch.zeros(n_slots, hkv)
    oracle_append.write(keys.cpu(), values.cpu(), slots.cpu(), k, v, kind, ks, vs, multipliers)
    return k, v, ks, vs
