"""Seeded sweeps over the geometry of the attention entry points: every case draws its page kind, head widths (keys' and
values'), KV heads and GQA group, page size (powers of two and not), rows' lengths, window widths and live columns,
sliding window, draft tree, piece and partitions from its seed, and is checked against float64 attention over the stored
values (2e-2, as everywhere) with the split launch and the fused launch bit for bit the same. What the hand-picked
shapes of the other files leave between them (a value row narrower than a wavefront under many partitions was one such
gap) is met here by chance rather than by foresight."""
import math
import random

import pytest
import torch

from tests.support import KINDS, Cache, kernels, rand_q

pytestmark = pytest.mark.gpu
dev = "cuda"
ATOL, RTOL = 8e-3, 2e-2


def _rows(draw, lengths, cols):
    rows, starts, firsts, counts, at = [], [], [], [], 0
    for s, n in enumerate(lengths):
        c = draw.randint(1, min(cols, n))
        rows.append(s), starts.append(at), firsts.append(n - c), counts.append(c)
        at += cols
    return rows, starts, firsts, counts, at


def _multipliers(draw, kind, hkv, seed):
    if kind == "fp8" and draw.random() < 0.5:      # one multiplier a KV head
        return torch.rand(2, hkv, generator=torch.Generator().manual_seed(seed)) * 0.04 + 0.01
    return 0.02, 0.03


@pytest.mark.parametrize("seed", range(60))
def test_windows_of_any_geometry(seed):
    draw = random.Random(seed)
    kind = draw.choice(KINDS)
    d = draw.choice([16, 32, 64, 64, 128, 128, 256])
    dv = d if draw.random() < 0.7 else draw.choice([16, 32, 64, 128, 256])
    hkv, g = draw.choice([1, 2, 3, 4, 6, 8]), draw.choice([1, 2, 3, 4, 5, 7, 8, 12, 16])
    page = draw.choice([16, 16, 32, 64, 128, 48, 24, 8, 1, 256])
    lengths = [draw.choice([1, 2, 15, 16, 17, 63, 64, 65, 300, 1023, 1025, 2500]) + draw.randint(0, 40)
               for _ in range(draw.randint(1, 4))]
    cols = draw.choice([1, 1, 2, 3, 5, 8, 13])
    rows, starts, firsts, counts, tokens = _rows(draw, lengths, cols)
    cache = Cache(kind, hkv, d, dv, page, lengths, seed=seed, multipliers=_multipliers(draw, kind, hkv, seed))
    q = rand_q(tokens, hkv * g, d, seed + 1000)
    sliding = draw.choice([0, 0, 0, 7, 200])
    fused = draw.random() < 0.4
    kw = dict(counts=torch.tensor(counts, dtype=torch.int32, device=dev), fused=fused)
    parents = None
    if sliding:
        kw["sliding"] = sliding
    elif cols > 1 and draw.random() < 0.4:
        parents = torch.tensor([[draw.randint(-1, c - 1) for c in range(cols)] for _ in rows], dtype=torch.int32)
        kw["parents"] = parents.to(dev).flatten()
    if draw.random() < 0.3:
        kw["piece"] = draw.choice([32, 64, 256, 1024])
    if draw.random() < 0.3:
        kw["partitions"] = draw.choice([1, 3, 8, 20, 64])
    lse = torch.empty(tokens, hkv * g, device=dev)
    out = cache.attend(q, rows, starts, firsts, cols, lse=lse, **kw)
    other = cache.attend(q, rows, starts, firsts, cols, **{**kw, "fused": not fused})
    for i, (s, start, first, count) in enumerate(zip(rows, starts, firsts, counts)):
        span = slice(start, start + count)
        assert torch.equal(out[span], other[span]), (seed, i, "the fused launch's bits are the split launch's")
        want, want_lse = cache.want(q[span], s, first, count, sliding=sliding,
                                    parents=None if parents is None else parents[i][:count])
        torch.testing.assert_close(out[span].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=lambda m: f"seed {seed} row {i}: {m}")
        torch.testing.assert_close(lse[span].double().cpu(), want_lse, atol=1e-3, rtol=1e-4, msg=lambda m: f"seed {seed} lse {i}: {m}")


@pytest.mark.parametrize("seed", range(30))
def test_block_lists_of_any_geometry(seed):
    draw = random.Random(seed)
    kind = draw.choice(KINDS)
    d = draw.choice([16, 32, 64, 128, 128, 256])
    hkv, g = draw.choice([1, 2, 3, 4, 8]), draw.choice([1, 2, 3, 4, 5, 8])
    page = draw.choice([16, 16, 32, 64, 8, 48])
    lengths = [draw.choice([5, 16, 17, 64, 300, 1023, 2500, 6000]) + draw.randint(0, 40) for _ in range(draw.randint(1, 3))]
    cols = draw.choice([1, 1, 2, 3, 5])
    block_size, width = draw.choice([1, 4, 8, 16, 24, 32, 64, 80, 128]), draw.choice([1, 2, 5, 12, 40, 100])
    rows, starts, firsts, counts, tokens = _rows(draw, lengths, cols)
    blocks = torch.full((tokens, width), -1, dtype=torch.int32)      # each token's own list, gaps of -1 anywhere
    for i, n in enumerate(lengths):
        nblk = math.ceil(n / block_size)
        for c in range(cols):
            k = draw.randint(0, min(width, nblk))
            chosen = draw.sample(range(nblk), k)
            for place, b in zip(sorted(draw.sample(range(width), k)), chosen):
                blocks[i * cols + c, place] = b
    cache = Cache(kind, hkv, d, d, page, lengths, seed=seed, multipliers=_multipliers(draw, kind, hkv, seed))
    q_dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    q = rand_q(tokens, hkv * g, d, seed + 1000)
    kw = dict(counts=torch.tensor(counts, dtype=torch.int32, device=dev), blocks=blocks.to(dev), block_size=block_size)
    parents = None
    if cols > 1 and draw.random() < 0.4:
        parents = torch.tensor([[draw.randint(-1, c - 1) for c in range(cols)] for _ in rows], dtype=torch.int32)
        kw["parents"] = parents.to(dev).flatten()
    if draw.random() < 0.4:
        kw["piece"] = draw.choice([32, 64, 256, 1024])
    if draw.random() < 0.5:
        kw["partitions"] = draw.choice([1, 3, 4, 16, 64])
    lse = torch.empty(tokens, hkv * g, device=dev)
    out = cache.attend(q, rows, starts, firsts, cols, lse=lse, **kw)
    for i, (s, start, first, count) in enumerate(zip(rows, starts, firsts, counts)):
        span = slice(start, start + count)
        want, want_lse = cache.want(q[span].to(q_dtype), s, first, count, blocks=blocks[span], block_size=block_size,
                                    parents=None if parents is None else parents[i][:count].tolist())
        sees_nothing = torch.isinf(want_lse) & (want_lse < 0)      # (an empty list: zeros and -inf)
        want = torch.where(sees_nothing[..., None], torch.zeros_like(want), want)
        torch.testing.assert_close(out[span].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=lambda m: f"seed {seed} row {i}: {m}")
        torch.testing.assert_close(lse[span].double().cpu(), want_lse, atol=1e-3, rtol=1e-4, msg=lambda m: f"seed {seed} lse {i}: {m}")


@pytest.mark.parametrize("seed", range(40))
def test_prompt_chunks_of_any_geometry(seed):
    draw = random.Random(seed)
    pk = kernels()
    kind = draw.choice(KINDS)
    d = draw.choice([16, 32, 64, 64, 128, 128, 256])
    hkv, g = draw.choice([1, 2, 3, 4, 8]), draw.choice([1, 2, 3, 4, 6, 8])
    page = draw.choice([16, 16, 32, 64, 8, 48, 128])
    position = draw.choice([0, 1, 15, 100, 511, 1000, 3000]) + draw.randint(0, 30)
    T = draw.choice([1, 2, 17, 63, 64, 65, 100, 200, 333])
    sliding = draw.choice([0, 0, 0, 7, 200])
    int8_qk = kind == "int8" and draw.random() < 0.5
    cache = Cache(kind, hkv, d, d, page, [position + T], seed=seed, multipliers=_multipliers(draw, kind, hkv, seed))
    q_dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    q = rand_q(T, hkv * g, d, seed + 1000)
    m = cache.multipliers.to(dev) if torch.is_tensor(cache.multipliers) else cache.multipliers
    kw = dict(key_scales=cache.ks, value_scales=cache.vs, multipliers=m)
    if sliding:
        kw["sliding"] = sliding
    if int8_qk:
        kw["int8_qk"] = True
    fresh = None
    if draw.random() < 0.35:      # the chunk's own rows from `first` on, as the projections gave them
        rows = torch.Generator().manual_seed(seed + 5)
        fk = torch.randn(T, hkv, d, generator=rows).to(q_dtype).to(dev)
        fv = torch.randn(T, hkv, d, generator=rows).to(q_dtype).to(dev)
        first = position + draw.randint(0, T)
        kw["fresh"] = (fk, fv, first)
        fresh = (fk.cpu(), fv.cpu(), position, first)
    table = cache.tables[0] if draw.random() < 0.5 else cache.tables[0].long()
    lse = torch.empty(T, hkv * g, device=dev)
    out = pk.prefill(q.to(q_dtype), cache.k, cache.v, kind, table, position, page, lse=lse, **kw)
    for t in sorted({0, T // 3, T // 2, T - 1, draw.randrange(T)}):
        want, want_lse = cache.want(q[t:t + 1], 0, position + t, 1, sliding=sliding, fresh=fresh, int8_qk=int8_qk)
        torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=lambda m: f"seed {seed} token {t}: {m}")
        torch.testing.assert_close(lse[t:t + 1].double().cpu(), want_lse, atol=2e-3, rtol=1e-4, msg=lambda m: f"seed {seed} lse {t}: {m}")
    if fresh is None and T > 1:      # a chunk cut in two anywhere: every token's bits stay
        cut = draw.randrange(1, T)
        head = pk.prefill(q[:cut].to(q_dtype), cache.k, cache.v, kind, table, position, page, **kw)
        tail = pk.prefill(q[cut:].to(q_dtype), cache.k, cache.v, kind, table, position + cut, page, **kw)
        assert torch.equal(torch.cat([head, tail]), out), (seed, cut)
