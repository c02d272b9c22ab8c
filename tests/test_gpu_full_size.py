"""The benchmark configurations at their full sizes (Llama-3-8B-shaped bf16 decode, FP8 decode at batch 128, 200k-token
split-K decode, chunked prefill mixed with decode): every row of every launch against textbook float64 attention over
the STORED values, computed densely by torch on the GPU (the oracle's reference() formula), and in every configuration
sampled rows of the launch directly against the CPU oracle (oracle.attend.window_reference over the pages copied
back), plus what does not depend on size: a fused launch and each row alone give the split
launch's bits, every chunk size of the contiguous splits agrees, appended bytes read back equal the oracle's encoding.
Tolerances: 2e-2 for 16-bit pages, 5e-2 for FP8 pages (outputs), 2e-3 for the log-sum-exp."""
import math

import pytest
import torch

from oracle import append as oracle_append
from oracle import attend as oracle_attend
from tests import harness
from tests.support import kernels

pytestmark = pytest.mark.gpu
dev = "cuda"
PAGE, HKV, D = 16, 8, 128


class Pool:
    """One layer's pages for sequences of the given lengths over a seeded permutation of a pool 1.25 times the pages
    needed, filled on the GPU."""

    def __init__(self, kind, lengths, seed, outliers=False, room=1):
        self.pk = kernels()
        self.kind, self.lengths = kind, list(lengths)
        g = torch.Generator(device=dev).manual_seed(seed)
        held = [math.ceil((n + room) / PAGE) for n in lengths]
        self.width = (max(held) + 15) // 16 * 16
        self.pages, self.held = int(sum(held) * 1.25) + 1, held
        order = torch.randperm(self.pages, device=dev, generator=g).to(torch.int32)
        self.tables = torch.full((len(lengths), self.width), self.pages, dtype=torch.int32, device=dev)      # (the dump page)
        at = 0
        for s, w in enumerate(held):
            self.tables[s, :w] = order[at:at + w]
            at += w
        store = torch.bfloat16 if kind == "bf16" else torch.float8_e4m3fn
        self.k = torch.zeros(self.pages + 1, PAGE, HKV, D, dtype=store, device=dev)
        self.v = torch.zeros(self.pages + 1, PAGE, HKV, D, dtype=store, device=dev)
        self.mult = (1.0, 1.0)

        def rows_of(s, n):      # sequence s's keys and values, the same at every call
            gs = torch.Generator(device=dev).manual_seed(seed * 100003 + s)
            keys = torch.randn(n, HKV, D, device=dev, generator=gs)
            values = torch.randn(n, HKV, D, device=dev, generator=gs)
            if outliers:
                keys = torch.where(torch.rand(n, HKV, D, device=dev, generator=gs) < 0.01, keys * 20, keys)
                values = torch.where(torch.rand(n, HKV, D, device=dev, generator=gs) < 0.01, values * 20, values)
            else:
                keys, values = keys * 0.5, values * 0.5
            return keys.bfloat16(), values.bfloat16()
        if kind == "fp8":      # per-(layer, KV head) multipliers: amax / 448 over the rows appended (N(0,1), 1 % x 20)
            top = torch.zeros(2, HKV, device=dev)
            for s, n in enumerate(lengths):
                keys, values = rows_of(s, n)
                top[0] = torch.maximum(top[0], keys.float().abs().amax((0, 2)))
                top[1] = torch.maximum(top[1], values.float().abs().amax((0, 2)))
            self.mult = (top / 448.0).contiguous()
        for s, n in enumerate(lengths):
            keys, values = rows_of(s, n)
            self.pk.write(keys, values, self.slots(s, 0, n), self.k, self.v, kind, multipliers=self.mult)

    def view(self, window=16):
        """The pool as crit's attention plugin reads it: each sequence's page ids on the host, the dump page, the window."""
        host = self.tables.cpu()
        tables = {s: host[s, :w].tolist() for s, w in enumerate(self.held)}
        return harness.PoolView(self.kind, PAGE, self.pages, window, tables, (self.k, self.v), self.mult, dev)

    def slots(self, s, start, n):
        p = torch.arange(start, start + n, device=dev)
        return self.tables[s][p // PAGE].long() * PAGE + p % PAGE

    def oracle_rows(self, q, tokens, s, first, tol, out, lse, what):
        """Tokens `tokens` of q / out / lse (consecutive columns of one window row of sequence s, the first at position
        `first`) against the CPU oracle over the pages as they are stored."""
        if not hasattr(self, "_cpu"):
            self._cpu = (self.k.cpu(), self.v.cpu(), self.tables.cpu())
        k, v, tables = self._cpu
        mult = (1.0, 1.0) if self.kind != "fp8" else (self.mult[0].cpu(), self.mult[1].cpu())
        count = tokens.stop - tokens.start
        want, want_lse = oracle_attend.window_reference(q[tokens].float().cpu(), k, v, self.kind, tables[s], first, count,
                                                        PAGE, D ** -0.5, multipliers=mult)
        torch.testing.assert_close(out[tokens].double().cpu(), want, atol=tol, rtol=tol, msg=lambda m: f"{what} vs the oracle: {m}")
        torch.testing.assert_close(lse[tokens].double().cpu(), want_lse, atol=2e-3, rtol=1e-3, msg=lambda m: f"{what} lse vs the oracle: {m}")

    def stored(self, s, n):
        """Positions 0 .. n - 1 of sequence s as float64 (keys, values) [n][HKV][D]: the codes times their multiplier."""
        at = self.slots(s, 0, n)
        k = self.k.view(-1, HKV, D)[at].double()
        v = self.v.view(-1, HKV, D)[at].double()
        if self.kind == "fp8":
            k, v = k * self.mult[0].double()[None, :, None], v * self.mult[1].double()[None, :, None]
        return k, v


def dense(q, keys, values, position, scale):
    """Float64 attention of a chunk q [T][HQ][D] whose token t sits at position + t and sees positions 0 .. position + t
    of keys / values [n][HKV][D] (n >= position + T): (out [T][HQ][D], lse [T][HQ]); the oracle's reference(), all
    heads at once."""
    T, hq, _ = q.shape
    g = hq // HKV
    n = position + T
    qq = q.double().view(T, HKV, g, D)
    s = torch.einsum("thgd,nhd->thgn", qq, keys[:n]) * scale
    seen = torch.arange(n, device=q.device)[None, :] <= (position + torch.arange(T, device=q.device))[:, None]
    s = s.masked_fill(~seen[:, None, None, :], float("-inf"))
    lse = torch.logsumexp(s, -1)
    out = torch.einsum("thgn,nhd->thgd", torch.softmax(s, -1), values[:n])
    return out.reshape(T, hq, D), lse.reshape(T, hq)


def check(out, lse, want, want_lse, tol, what):
    torch.testing.assert_close(out.double(), want, atol=tol, rtol=tol, msg=lambda m: f"{what}: {m}")
    torch.testing.assert_close(lse.double(), want_lse, atol=2e-3, rtol=1e-3, msg=lambda m: f"{what} lse: {m}")


def decode_all(pool, q, firsts, **kw):
    B = len(pool.lengths)
    rows = torch.arange(B, dtype=torch.int32, device=dev)
    lse = torch.empty(B, q.shape[1], device=dev)
    out = pool.pk.attend(q, pool.k, pool.v, pool.kind, pool.tables, rows, rows.clone(), firsts, 1, PAGE,
                         multipliers=pool.mult, lse=lse, **kw)
    return out, lse


@pytest.mark.parametrize("kind,B,low,high,tol", [("bf16", 64, 1024, 8192, 2e-2), ("fp8", 128, 2048, 16384, 5e-2)])
def test_a_decode_step_of_the_8b_shape_at_its_batch_and_lengths(kind, B, low, high, tol):
    pk = kernels()
    hq = 32
    lengths = torch.randint(low, high + 1, (B,), generator=torch.Generator().manual_seed(7)).tolist()
    lengths[0], lengths[1] = low, high
    pool = Pool(kind, lengths, 8, outliers=kind == "fp8")
    g = torch.Generator(device=dev).manual_seed(9)
    # the step's append: one token a sequence at its length; the bytes read back equal the oracle's encoding
    keys = torch.randn(B, HKV, D, device=dev, generator=g).bfloat16()
    values = torch.randn(B, HKV, D, device=dev, generator=g).bfloat16()
    slots = torch.stack([pool.slots(s, n, 1)[0] for s, n in enumerate(lengths)])
    pk.write(keys, values, slots, pool.k, pool.v, kind, multipliers=pool.mult)
    for given, pages, which in ((keys, pool.k, 0), (values, pool.v, 1)):
        m = 1.0 if kind == "bf16" else pool.mult[which].cpu()
        want, _ = oracle_append.encode(given.cpu(), kind, m)
        got = pages.view(-1, HKV, D)[slots].cpu()
        assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), "appended bytes"
    q = torch.randn(B, hq, D, device=dev, generator=g).bfloat16()
    firsts = torch.tensor(lengths, dtype=torch.int64, device=dev)
    # the launch crit's plugin makes of this step: a StepBatch of one token a sequence, every row a window row, tables cut
    # at the rows' pages in widths of sixteen, partials packed by the tokens
    batch = harness.StepBatch.build([(s, n, 1) for s, n in enumerate(lengths)], dev)
    out, lse = harness.forward(pk, q, pool.view(), batch, lse=True)
    assert harness.forward.launched == {"attend": 1, "prefill": 0}
    # the same rows over the pool's whole tables, laid out by columns, and in three launches where the partials run out
    plain, plain_lse = decode_all(pool, q, firsts)
    assert torch.equal(out, plain) and torch.equal(lse, plain_lse)
    cut, cut_lse = harness.forward(pk, q, pool.view(), batch, lse=True, partial_rows=B // 3 + 1)
    assert harness.forward.launched == {"attend": 3, "prefill": 0} and torch.equal(out, cut) and torch.equal(lse, cut_lse)
    scale = D ** -0.5
    for s, n in enumerate(lengths):
        k, v = pool.stored(s, n + 1)
        want, want_lse = dense(q[s:s + 1], k, v, n, scale)
        check(out[s:s + 1], lse[s:s + 1], want, want_lse, tol, f"row {s} of {n + 1} positions")
    # the launch's shortest and longest rows and one between, directly against the CPU oracle
    for s in (0, 1, B // 2):
        pool.oracle_rows(q, slice(s, s + 1), s, lengths[s], tol, out, lse, f"row {s}")
    # what does not depend on size: the fused launch and a row alone give the split launch's bits
    fused, fused_lse = decode_all(pool, q, firsts, fused=True)
    assert torch.equal(out, fused) and torch.equal(lse, fused_lse)
    for s in (1, B - 1):
        alone = pk.attend(q[s:s + 1], pool.k, pool.v, kind, pool.tables, torch.tensor([s], dtype=torch.int32, device=dev),
                          torch.zeros(1, dtype=torch.int32, device=dev), firsts[s:s + 1], 1, PAGE, multipliers=pool.mult)
        assert torch.equal(alone, out[s:s + 1])


@pytest.mark.parametrize("B,context", [(1, 200000), (4, 131072), (2, 32768)])
def test_long_contexts_through_contiguous_splits_and_their_merge(B, context):
    hq = 40
    pool = Pool("bf16", [context - 1] * B, 10)
    g = torch.Generator(device=dev).manual_seed(11)
    q = torch.randn(B, hq, D, device=dev, generator=g).bfloat16()
    firsts = torch.full((B,), context - 1, dtype=torch.int64, device=dev)
    scale = D ** -0.5
    wants = [dense(q[s:s + 1], *pool.stored(s, context), context - 1, scale) for s in range(B)]
    found = {}
    for chunk in (None, 512, 1024, 2048):
        out, lse = decode_all(pool, q, firsts, **({} if chunk is None else dict(flash=True, chunk=chunk)))
        for s in range(B):
            check(out[s:s + 1], lse[s:s + 1], wants[s][0], wants[s][1], 2e-2, f"chunk {chunk} row {s}")
        if B == 1 or chunk is None:      # a row of each context directly against the CPU oracle (200k: every reader)
            pool.oracle_rows(q, slice(B - 1, B), B - 1, context - 1, 2e-2, out, lse, f"chunk {chunk} row {B - 1}")
        found[chunk] = (out, lse)
    # every cut of the positions gives the same sum to rounding: the log-sum-exp of any two chunk sizes agrees far
    # inside the bound against the reference
    for chunk in (512, 2048):
        torch.testing.assert_close(found[chunk][1], found[1024][1], atol=1e-4, rtol=1e-5)


def test_prompt_chunks_on_prefixes_mixed_with_decode_rows():
    pk = kernels()
    hq, T = 32, 512
    prefixes = [1229, 6096, 6373, 0, 1175, 5023, 8192, 4769]
    decodes = torch.randint(1024, 8193, (56,), generator=torch.Generator().manual_seed(12)).tolist()
    pool = Pool("bf16", [p + T for p in prefixes] + [n + 1 for n in decodes], 13, room=0)
    g = torch.Generator(device=dev).manual_seed(14)
    tokens = 8 * T + 56
    q = torch.randn(tokens, hq, D, device=dev, generator=g).bfloat16()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    # the step as crit's plugin launches it: the rows of up to the pool's window (the decode rows) in one attend(), each
    # prompt row through prefill() over its sequence's own table
    batch = harness.StepBatch.build([(c, p, T) for c, p in enumerate(prefixes)] + [(8 + r, n, 1) for r, n in enumerate(decodes)], dev)
    out, lse = harness.forward(pk, q, pool.view(), batch, lse=True)
    assert harness.forward.launched == {"attend": 1, "prefill": 8}
    # every chunk in one launch (prefill_rows) and the decode rows over the pool's whole tables give the same bits
    once, once_lse = torch.empty_like(out), torch.empty_like(lse)
    pk.prefill_rows(q, pool.k, pool.v, "bf16", pool.tables, i32(list(range(8))), i32([c * T for c in range(8)]),
                    i32([T] * 8), torch.tensor(prefixes, dtype=torch.int64, device=dev), T, PAGE, out=once, lse=once_lse)
    rows = i32(list(range(8, 64)))
    pk.attend(q, pool.k, pool.v, "bf16", pool.tables, rows, i32([8 * T + r for r in range(56)]),
              torch.tensor(decodes, dtype=torch.int64, device=dev), 1, PAGE, out=once, lse=once_lse)
    assert torch.equal(out, once) and torch.equal(lse, once_lse)
    scale = D ** -0.5
    for c, p in enumerate(prefixes):
        k, v = pool.stored(c, p + T)
        want, want_lse = dense(q[c * T:(c + 1) * T], k, v, p, scale)
        check(out[c * T:(c + 1) * T], lse[c * T:(c + 1) * T], want, want_lse, 2e-2, f"chunk {c} on a prefix of {p}")
    for r, n in enumerate(decodes):
        k, v = pool.stored(8 + r, n + 1)
        t = 8 * T + r
        want, want_lse = dense(q[t:t + 1], k, v, n, scale)
        check(out[t:t + 1], lse[t:t + 1], want, want_lse, 2e-2, f"decode row {r}")
    # directly against the CPU oracle: the chunk that starts its sequence, the last columns of the one on the longest
    # prefix, and a decode row
    pool.oracle_rows(q, slice(3 * T, 3 * T + T), 3, 0, 2e-2, out, lse, "chunk 3")
    pool.oracle_rows(q, slice(6 * T + T - 3, 6 * T + T), 6, prefixes[6] + T - 3, 2e-2, out, lse, "chunk 6's last columns")
    pool.oracle_rows(q, slice(8 * T + 5, 8 * T + 6), 8 + 5, decodes[5], 2e-2, out, lse, "decode row 5")
    # a prompt token's output is the same position decoded, to the readers' rounding
    c, t = 2, 300
    one = pk.attend(q[c * T + t:c * T + t + 1], pool.k, pool.v, "bf16", pool.tables, i32([c]), i32([0]),
                    torch.tensor([prefixes[c] + t], dtype=torch.int64, device=dev), 1, PAGE)
    torch.testing.assert_close(one.float(), out[c * T + t:c * T + t + 1].float(), atol=8e-3, rtol=2e-2)
