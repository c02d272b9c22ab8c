"""Seeded sweeps over the geometry of the entry points: paged windows, block lists, prompt chunks, latent windows and
index selection against float64; appends, plain and with the keys' rope and norm fused in, byte for byte. An attention
case draws its page kind, head widths (keys' and values'), KV heads and GQA group, page size (powers of two and not),
rows' lengths, window widths and live columns, sliding window, draft tree, piece and partitions from its seed, and is
checked against float64 attention over the stored values (2e-2, as everywhere) with the split launch and the fused
launch bit for bit the same. What the hand-picked shapes of the other files leave between them (a value row narrower
than a wavefront under many partitions was one such gap) is met here by chance rather than by foresight."""
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


@pytest.mark.parametrize("seed", range(40))
def test_latent_windows_of_any_geometry(seed):
    # every rank and rotary width the reference's module takes (the matrix-core kernels' shapes, the many-heads kernel
    # where it may read, and the shapes below the tiles), 16-bit and E4M3 caches with two scales a row or one
    from tests.test_gpu_latent import Cache as LatentCache, _q
    draw = random.Random(seed)
    if draw.random() < 0.4:
        rank, rope = 512, 64
    else:
        rank, rope = draw.choice([16, 32, 64, 128, 256, 512, 1024]), draw.choice([16, 32, 64, 128, 256])
    heads = draw.choice([1, 2, 3, 5, 8, 16, 16, 20, 40, 64, 128])
    if rank * heads > 512 * 128:
        heads = 16
    page = draw.choice([16, 16, 32, 64, 48, 8, 1, 128])
    coded = draw.choice([0, 0, 2, 1])
    dtype = draw.choice([torch.bfloat16, torch.float16])
    lengths = [draw.choice([1, 2, 31, 32, 33, 64, 255, 256, 257, 700, 1500, 3000]) + draw.randint(0, 20)
               for _ in range(draw.randint(1, 4))]
    cols = draw.choice([1, 1, 2, 3, 5, 8])
    rows, starts, firsts, counts, tokens = _rows(draw, lengths, cols)
    kw = dict(counts=torch.tensor(counts, dtype=torch.int32, device=dev))
    if draw.random() < 0.3:
        kw["piece"] = draw.choice([32, 64, 96, 256, 512, 1024])
    if draw.random() < 0.3:
        kw["partitions"] = draw.choice([1, 3, 8, 64])
    if (rank, rope) == (512, 64) and page % 16 == 0 and draw.random() < 0.5:
        kw["tile_rows"] = draw.choice([16, 128])
    scale = draw.choice([None, 0.07])
    kind = dict(dtype=torch.float8_e4m3fn, scales=coded) if coded else dict(dtype=dtype)
    cache = LatentCache(rank, rope, page, lengths, seed=seed, **kind)
    q = _q(tokens, heads, rank + rope, seed + 500, dtype)
    sinks = torch.randn(heads, generator=torch.Generator().manual_seed(seed)).to(dev) if draw.random() < 0.3 else None
    lse = torch.empty(tokens, heads, device=dev)
    out = cache.attend(q, rows, starts, firsts, cols, lse=lse, sinks=sinks, scale=scale, **kw)
    used = (rank + rope) ** -0.5 if scale is None else scale
    for s, start, first, count in zip(rows, starts, firsts, counts):
        cache.check(q, out, lse, s, start, first, count, used, sinks)
        j = draw.randrange(count)      # a token alone in a window of one column: the same bits
        alone = cache.attend(q[start + j:start + j + 1], [s], [0], [first + j], 1, sinks=sinks, scale=scale,
                             **{**kw, "counts": None})
        assert torch.equal(alone[0], out[start + j]), (seed, s, j)


@pytest.mark.parametrize("seed", range(40))
def test_index_selection_of_any_geometry(seed):
    import numpy as np

    from crit_amd import sparse_indexer as si
    from oracle import indexer as ref
    from tests.test_gpu_indexer import compressed
    draw = random.Random(seed)
    heads, width = draw.choice([1, 2, 4, 8, 16, 32, 64, 128]), draw.choice([64, 128, 256])
    e4m3 = draw.random() < 0.4
    dtype = draw.choice([torch.bfloat16, torch.float16])
    n = draw.choice([1, 5, 63, 64, 65, 200, 1000, 3000])
    groups = draw.choice([0, 0, 1, 1, 2, 3, 5])      # 0: the keys as they lie; 1: one list of slots; more: a list a group
    each = draw.choice([1, 2, 3, 4, 7, 8, 16, 20, 33])
    tokens = each * max(1, groups)
    k = draw.choice([1, 16, 64, 512])
    store_n = n + draw.choice([0, 10, 500])
    g = torch.Generator().manual_seed(seed)
    rows = torch.empty(store_n, width).normal_(0.0, 0.5, generator=g).to(dev).to(dtype)
    q = torch.empty(tokens, heads, width).normal_(0.0, 0.5, generator=g).to(dev).to(dtype)
    w = (torch.empty(tokens, heads).normal_(generator=g) / heads ** 0.5).to(dev)
    ends = (torch.rand(tokens, generator=g) * (n + 1)).long().clamp_(max=n).to(torch.int32).to(dev)
    keys, scales, values = compressed(rows, e4m3)
    kw, slots = {}, None
    if groups == 0:
        keys, values, scales = keys[:n], values[:n], None if scales is None else scales[:n]
    elif groups == 1:
        slots = torch.randperm(store_n, generator=g)[:n].to(dev)
        kw["slots"] = slots.to(torch.int32) if draw.random() < 0.5 else slots
    else:
        slots = torch.stack([torch.randperm(store_n, generator=g)[:n] for _ in range(groups)]).to(dev)
        kw["slots"] = slots
    got = si.scores(q, keys, w, ends, key_scales=scales, **kw)
    picks = si.topk(got, ends, k)
    if groups <= 1:
        assert torch.equal(si.select(q, keys, w, ends, k, key_scales=scales, **kw), picks), seed
    f = lambda x: x.double().cpu().numpy()
    for gi in range(max(1, groups)):
        span = slice(gi * each, (gi + 1) * each) if groups > 1 else slice(None)
        vals = values if slots is None else values[(slots if slots.dim() == 1 else slots[gi]).long()]
        want = ref.sparse_scores(f(q[span]), f(vals), f(w[span]), ends[span].cpu().numpy(), width ** -0.5)
        slack = ref.sparse_scores(f(q[span].abs()), f(vals.abs()), f(w[span].abs()), ends[span].cpu().numpy(), width ** -0.5) * 1e-4 + 1e-6
        found = got[span].cpu().numpy()
        seen = np.isfinite(want)
        assert np.array_equal(seen, np.isfinite(found)) and (found[~seen] == -np.inf).all(), (seed, "the causal ends")
        assert (np.abs(found.astype(np.float64)[seen] - want[seen]) <= slack[seen]).all(), (seed, "scores")
        exact = torch.from_numpy(ref.sparse_index(got[span].double().cpu().numpy(), ends[span].cpu().numpy(), k))
        assert torch.equal(picks[span].long().cpu(), exact), (seed, "picks")


def _same_bytes(got, want, what):
    """Stored tensors bit for bit; a NaN only as a NaN where `want` holds one (what a cast stores for it is the host's)."""
    from tests.support import bits
    got = got.cpu()
    nan = torch.isnan(want.float())
    assert torch.equal(torch.isnan(got.float()), nan), (what, "which are NaN")
    assert torch.equal(bits(got)[~nan], bits(want)[~nan]), (what, int((bits(got)[~nan] != bits(want)[~nan]).sum()), "differ")


@pytest.mark.parametrize("seed", range(60))
def test_appends_of_any_geometry_store_the_oracles_bytes(seed):
    # rows of any width (the scalar kernel's too), strided views of a wider projection output, keys only or values
    # only, FP32 / BF16 / FP16 inputs into every page kind, magnitudes from 1e-2 to 1e3 and one far outlier, per-head
    # multipliers, negative slots: every stored byte and row scale
    from tests.support import STORE, expected_pages
    draw = random.Random(seed)
    pk = kernels()
    kind = draw.choice(KINDS)
    d = draw.choice([8, 16, 20, 32, 40, 64, 96, 128, 128, 192, 256, 512])
    dv = d if draw.random() < 0.6 else draw.choice([8, 16, 24, 64, 128, 256])
    hkv = draw.choice([1, 2, 3, 4, 8, 16])
    T = draw.choice([1, 2, 3, 7, 64, 100, 257, 1000, 4152])
    n_slots = T + draw.choice([0, 5, 100])
    in_dtype = draw.choice([torch.float32, torch.bfloat16, torch.float16])
    which = draw.choice(["both", "both", "both", "keys", "values"])
    strided = draw.random() < 0.4
    g = torch.Generator().manual_seed(seed)
    if kind == "fp8" and draw.random() < 0.5:
        mult = torch.rand(2, hkv, generator=g) * 0.04 + 0.01
    else:
        mult = (draw.choice([1.0, 0.05, 0.013]), draw.choice([1.0, 0.07]))
    amp = draw.choice([0.01, 1.0, 30.0, 1000.0])
    keys = (torch.randn(T, hkv, d, generator=g) * amp).to(in_dtype)
    values = (torch.randn(T, hkv, dv, generator=g) * amp).to(in_dtype)
    if T > 2:
        keys[1] = 0.0
        values[2, 0] = 0.0
    if draw.random() < 0.3 and in_dtype != torch.float16:
        keys[0, 0, 0] = 1e30
    slots = torch.randperm(n_slots, generator=g)[:T]
    for i in range(T):
        if draw.random() < 0.05:
            slots[i] = -1 - draw.randint(0, 3)

    def on_device(x):
        if not strided:
            return x.to(dev)
        width = x.shape[2]      # a view into a wider row, as a fused projection's output is
        wide = torch.zeros(T, hkv * width + 8 * draw.randint(0, 3), dtype=x.dtype, device=dev)
        wide[:, :hkv * width] = x.reshape(T, hkv * width).to(dev)
        return wide[:, :hkv * width].view(T, hkv, width)
    k = torch.zeros(n_slots, hkv, d, dtype=STORE[kind], device=dev)
    v = torch.zeros(n_slots, hkv, dv, dtype=STORE[kind], device=dev)
    ks = vs = None
    if kind in ("fp8:row", "int8"):
        ks, vs = torch.zeros(n_slots, hkv, device=dev), torch.zeros(n_slots, hkv, device=dev)
    given = mult.to(dev) if torch.is_tensor(mult) else mult
    if which == "both":
        pk.write(on_device(keys), on_device(values), slots.to(dev), k, v, kind, ks, vs, multipliers=given)
    elif which == "keys":
        pk.write(on_device(keys), None, slots.to(dev), k, None, kind, ks, None, multipliers=given)
    else:
        pk.write(None, on_device(values), slots.to(dev), None, v, kind, None, vs, multipliers=given)
    want = expected_pages(kind, keys, values, slots, n_slots, (mult[0], mult[1]) if torch.is_tensor(mult) else mult)
    for at, (name, got, exact) in enumerate(zip(("keys", "values", "key scales", "value scales"), (k, v, ks, vs), want)):
        if exact is None:
            continue
        if (which == "keys" and at in (1, 3)) or (which == "values" and at in (0, 2)):
            exact = torch.zeros_like(exact)      # (the part not given stays untouched)
        _same_bytes(got, exact, (seed, name))


@pytest.mark.parametrize("seed", range(40))
def test_appends_with_the_keys_rope_and_norm_fused_in_store_the_oracles_bytes(seed):
    # rope() or rms_norm_rope() of the keys and then the append, against the oracle's two steps: magnitudes from 1e-20
    # to 1e15, zeros of both signs, infinities, subnormals, NaNs, positions past the table, both pair styles, a scale
    # on cos and sin, the weight in FP32 or in the inputs' type, values wider or narrower than the keys
    from oracle import append as oracle_append
    from tests.support import STORE, expected_pages
    draw = random.Random(seed)
    pk = kernels()
    kind = draw.choice(KINDS)
    d, dv = draw.choice([64, 128, 256]), draw.choice([64, 128, 256])
    in_dtype = draw.choice([torch.float32, torch.bfloat16, torch.float16])
    if kind == "fp16" and in_dtype == torch.bfloat16:
        in_dtype = torch.float16
    style = draw.choice(["half", "interleaved"])
    normed = draw.random() < 0.6
    g = torch.Generator().manual_seed(seed)
    T, hkv, P = draw.choice([1, 7, 70, 300]), draw.choice([1, 2, 3, 8]), 500
    mag = draw.choice([1e-20, 1e-3, 1.0, 30.0, 1e4, 1e15 if in_dtype != torch.float16 else 3e3])
    keys = torch.randn(T, hkv, d, generator=g) * mag
    flat = keys.view(-1)
    for special in (0.0, -0.0, float("inf"), float("-inf"), 1e-40, -1e-40, 65504.0):
        if draw.random() < 0.4:
            flat[torch.randint(0, flat.numel(), (3,), generator=g)] = special
    if draw.random() < 0.3:
        flat[torch.randint(0, flat.numel(), (2,), generator=g)] = float("nan")
    if draw.random() < 0.3:
        keys[0] = 0
    keys = keys.to(in_dtype)
    values = torch.randn(T, hkv, dv, generator=g).to(in_dtype)
    half = d // 2
    angle = torch.arange(P, dtype=torch.float64)[:, None] / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))[None, :]
    table = torch.cat([angle.cos(), angle.sin()], 1).float()
    positions = torch.randint(-3, P + 10, (T,), generator=g)
    n_slots = T + 9
    slots = torch.randperm(n_slots, generator=g)[:T]
    if T > 2:
        slots[1] = -1
    mult = (draw.choice([0.05, 1.0, 3.7e-3]), 0.07)
    scale = draw.choice([1.0, 0.75, 1.3])
    k = torch.zeros(n_slots, hkv, d, dtype=STORE[kind], device=dev)
    v = torch.zeros(n_slots, hkv, dv, dtype=STORE[kind], device=dev)
    ks = vs = None
    if kind in ("fp8:row", "int8"):
        ks, vs = torch.zeros(n_slots, hkv, device=dev), torch.zeros(n_slots, hkv, device=dev)
    rope = (table.to(dev), positions.to(dev), style, scale)
    if normed:
        weight = torch.randn(d, generator=g) * 0.3 + 1
        eps, offset = draw.choice([1e-6, 1e-5, 0.0 if mag >= 1e-3 else 1e-6]), draw.choice([0.0, 1.0])
        weight = weight if draw.random() < 0.5 else weight.to(in_dtype)
        pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs, multipliers=mult, rope=rope,
                 norm=(weight.to(dev), eps, offset))
        turned = oracle_append.rms_norm_rope(keys, weight, eps, positions, table, offset, style, scale)
    else:
        pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs, multipliers=mult, rope=rope)
        turned = oracle_append.rope(keys, positions, table, style, scale)
    want = expected_pages(kind, turned, values, slots, n_slots, mult)
    for name, got, exact in zip(("keys", "values", "key scales", "value scales"), (k, v, ks, vs), want):
        if exact is not None:
            _same_bytes(got, exact, (seed, name))


@pytest.mark.parametrize("seed", range(24))
def test_windows_at_the_launchs_limits(seed):
    # launches of hundreds to 1,500 rows (past the rows a workgroup lists in LDS), windows of up to 64 columns under GQA
    # groups of up to 32 (dozens of tiles a KV head), thousands of partitions of the shortest pieces, rows of no column
    draw = random.Random(7000 + seed)
    kind = draw.choice(KINDS)
    d = draw.choice([64, 128, 128, 256, 32])
    hkv, g = draw.choice([1, 2, 4, 8]), draw.choice([1, 4, 8, 16, 32])
    g = min(g, 128 // hkv)
    page = draw.choice([16, 16, 64, 256])
    mode = ("many rows", "wide windows", "many partitions", "empty rows")[seed % 4]
    if mode == "many rows":
        lengths, cols = [draw.randint(1, 60) for _ in range(draw.choice([300, 700, 1500]))], draw.choice([1, 2])
    elif mode == "wide windows":
        lengths = [draw.choice([64, 100, 700, 3000]) + draw.randint(0, 30) for _ in range(draw.randint(1, 3))]
        cols = draw.choice([16, 33, 64])
    elif mode == "many partitions":
        lengths, cols = [draw.choice([5000, 20000]) + draw.randint(0, 100) for _ in range(draw.randint(1, 2))], draw.choice([1, 3])
    else:
        lengths, cols = [draw.choice([1, 5, 300]) for _ in range(draw.randint(2, 6))], draw.choice([1, 4])
    rows, starts, firsts, counts, tokens = [], [], [], [], 0
    for s, n in enumerate(lengths):
        c = 0 if mode == "empty rows" and draw.random() < 0.4 else draw.randint(1, min(cols, n))
        rows.append(s), starts.append(tokens), firsts.append(n - max(c, 1)), counts.append(c)
        tokens += cols
    fused = draw.random() < 0.4
    kw = dict(counts=torch.tensor(counts, dtype=torch.int32, device=dev), fused=fused)
    if mode == "many partitions":
        kw["partitions"], kw["piece"] = draw.choice([200, 1000, 5000]), draw.choice([16, 32, 64])
    sliding = draw.choice([0, 0, 50])
    if sliding:
        kw["sliding"] = sliding
    cache = Cache(kind, hkv, d, d, page, lengths, seed=seed)
    q = rand_q(tokens, hkv * g, d, seed + 1000)
    lse = torch.full((tokens, hkv * g), 7.0, device=dev)
    out = cache.attend(q, rows, starts, firsts, cols, lse=lse, **kw)
    other = cache.attend(q, rows, starts, firsts, cols, **{**kw, "fused": not fused})
    for i, (start, count) in enumerate(zip(starts, counts)):
        assert torch.equal(out[start:start + count], other[start:start + count]), (seed, i)
        assert bool((lse[start + count:start + cols] == 7.0).all()), (seed, i, "tokens past the row's count are not written")
    for i in (range(len(rows)) if len(rows) <= 8 else draw.sample(range(len(rows)), 8)):
        s, start, first, count = rows[i], starts[i], firsts[i], counts[i]
        if count:
            some = sorted({0, count - 1, draw.randrange(count)})
            want, want_lse = cache.want(q[start:start + count], s, first, count, sliding=sliding)
            torch.testing.assert_close(out[start:start + count].double().cpu()[some], want[some], atol=ATOL, rtol=RTOL)
            torch.testing.assert_close(lse[start:start + count].double().cpu()[some], want_lse[some], atol=1e-3, rtol=1e-4)
