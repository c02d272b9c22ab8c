"""Chunked prefill over paged KV (the matrix-core path) on the GPU against the CPU oracle. Mirrors the reference's
kernels/techniques/attention/paged-kv-attention/tests/test_paged_kv_attention.py:459-480, 515-536 and the prompt-row
call sites of inference/attention-state/code/device_attention.py:901-916 (int64 tables, sliced outputs)."""
import pytest
import torch

from tests.support import KINDS, Cache, kernels, rand_q

pytestmark = pytest.mark.gpu
dev = "cuda"
ATOL, RTOL = 8e-3, 2e-2


def _check(cache, q, out, lse, position, tokens, sliding=0):
    for t in tokens:
        want, want_lse = cache.want(q[t:t + 1], 0, position + t, 1, sliding=sliding)
        torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"token {t}")
        if lse is not None:
            torch.testing.assert_close(lse[t:t + 1].double().cpu(), want_lse, atol=1e-3, rtol=1e-4, msg=f"lse {t}")


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (32, 8, 128), (40, 8, 128), (12, 2, 64), (24, 2, 256), (24, 4, 256)])
def test_prompt_chunks_match_float64_attention(kind, hq, hkv, d):
    # (256-wide heads: the matrix-core kernel with one workgroup a compute unit; INT8 pages there go through window rows)
    pk = kernels()
    cache = Cache(kind, hkv, d, d, 16, [300])
    q = rand_q(100, hq, d, 4)
    lse = torch.empty(100, hq, device=dev)
    q_dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    out = pk.prefill(q.to(q_dtype), cache.k, cache.v, kind, cache.tables[0], 200, 16, key_scales=cache.ks,
                     value_scales=cache.vs, multipliers=cache.multipliers, lse=lse)
    _check(cache, q, out, lse, 200, (0, 37, 63, 64, 99))


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
@pytest.mark.parametrize("hq,hkv,d", [(24, 4, 256), (4, 2, 32), (6, 1, 16)])
def test_prompt_chunks_at_the_other_head_widths(kind, hq, hkv, d):
    # 256-wide heads on the matrix-core kernel; 16 and 32, which it does not take, as window rows of up to 64 columns
    # read by the decode reader's fused launch (what crit does with prompt_reader decode); the same contract, fresh
    # rows included.
    pk = kernels()
    cache = Cache(kind, hkv, d, d, 16, [300])
    q = rand_q(150, hq, d, 4)
    lse = torch.empty(150, hq, device=dev)
    out = pk.prefill(q.bfloat16(), cache.k, cache.v, kind, cache.tables[0].long(), 150, 16, key_scales=cache.ks,
                     value_scales=cache.vs, lse=lse)
    _check(cache, q, out, lse, 150, (0, 63, 64, 127, 128, 149))
    position = torch.tensor([150], dtype=torch.int64, device=dev)
    assert torch.equal(pk.prefill(q.bfloat16(), cache.k, cache.v, kind, cache.tables[0], position, 16,
                                  key_scales=cache.ks, value_scales=cache.vs), out)
    g = torch.Generator().manual_seed(8)
    fk, fv = torch.randn(150, hkv, d, generator=g).bfloat16().to(dev), torch.randn(150, hkv, d, generator=g).bfloat16().to(dev)
    got = pk.prefill(q.bfloat16(), cache.k, cache.v, kind, cache.tables[0], 150, 16, key_scales=cache.ks,
                     value_scales=cache.vs, fresh=(fk, fv, 200))
    for t in (0, 49, 50, 149):
        want, _ = cache.want(q[t:t + 1], 0, 150 + t, 1, fresh=(fk.cpu(), fv.cpu(), 150, 200))
        torch.testing.assert_close(got[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"fresh token {t}")


@pytest.mark.parametrize("position,T", [(0, 1), (0, 512), (1, 17), (1000, 512), (8191, 33)])
def test_chunks_at_any_position_and_length(position, T):
    pk = kernels()
    cache = Cache("bf16", 8, 128, 128, 16, [position + T], seed=3, scale=0.5)
    q = rand_q(T, 32, 128, 5)
    lse = torch.empty(T, 32, device=dev)
    out = pk.prefill(q.bfloat16(), cache.k, cache.v, "bf16", cache.tables[0].long(), position, 16, lse=lse)
    picks = sorted({0, T // 3, T - 1})
    _check(cache, q, out, lse, position, picks)


def test_a_tokens_bits_follow_its_own_positions_only():
    # The same tokens read as one chunk, as two chunks, and at a device position: every bit equal.
    pk = kernels()
    cache = Cache("bf16", 2, 128, 128, 16, [700])
    q = rand_q(200, 8, 128, 6).bfloat16()
    table = cache.tables[0]
    whole = pk.prefill(q, cache.k, cache.v, "bf16", table, 500, 16)
    first = pk.prefill(q[:77], cache.k, cache.v, "bf16", table, 500, 16)
    second = pk.prefill(q[77:], cache.k, cache.v, "bf16", table, 577, 16)
    assert torch.equal(torch.cat([first, second]), whole)
    position = torch.tensor([500], dtype=torch.int64, device=dev)
    assert torch.equal(pk.prefill(q, cache.k, cache.v, "bf16", table, position, 16), whole)
    sliced = torch.zeros(300, 8, 128, dtype=torch.bfloat16, device=dev)
    pk.prefill(q, cache.k, cache.v, "bf16", table, 500, 16, out=sliced[50:250])
    assert torch.equal(sliced[50:250], whole) and not bool(sliced[:50].any()) and not bool(sliced[250:].any())


def test_a_chunk_at_a_device_position_replays_from_one_graph():
    pk = kernels()
    cache = Cache("fp8:row", 4, 128, 128, 16, [700])
    q = rand_q(64, 16, 128, 12).to(torch.bfloat16)
    table = cache.tables[0]
    position = torch.zeros(1, dtype=torch.int64, device=dev)
    out = torch.empty_like(q)

    def launch(into, at):
        pk.prefill(q, cache.k, cache.v, "fp8:row", table, at, 16, key_scales=cache.ks, value_scales=cache.vs, out=into)
    launch(out, position)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch(out, position)
    for at in (0, 5, 300, 636):
        position.fill_(at)
        graph.replay()
        torch.cuda.synchronize()
        want = torch.empty_like(q)
        launch(want, at)
        assert torch.equal(out, want), at


def test_several_chunks_in_one_launch_equal_one_launch_each():
    # the mixed batch's prefill part: chunks of different lengths on prefixes of different lengths, one launch
    pk = kernels()
    lengths = [512 + 0, 512 + 1000, 300 + 4097, 512 + 8192]
    counts = [512, 512, 300, 512]
    cache = Cache("bf16", 8, 128, 128, 16, lengths, seed=9, scale=0.5)
    starts = [0, 512, 1024, 1324]
    q = rand_q(sum(counts), 32, 128, 7).bfloat16()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    positions = torch.tensor([n - c for n, c in zip(lengths, counts)], dtype=torch.int64, device=dev)
    lse = torch.empty(q.shape[0], 32, device=dev)
    out = pk.prefill_rows(q, cache.k, cache.v, "bf16", cache.tables, i32([0, 1, 2, 3]), i32(starts), i32(counts),
                          positions, 512, 16, lse=lse)
    for s, (start, count, n) in enumerate(zip(starts, counts, lengths)):
        one = pk.prefill(q[start:start + count], cache.k, cache.v, "bf16", cache.tables[s], n - count, 16)
        assert torch.equal(out[start:start + count], one), s
    want, want_lse = cache.want(q[1324 + 511:1324 + 512].float(), 3, lengths[3] - 1, 1)
    torch.testing.assert_close(out[-1:].double().cpu(), want, atol=ATOL, rtol=RTOL)
    torch.testing.assert_close(lse[-1:].double().cpu(), want_lse, atol=1e-3, rtol=1e-4)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("window", [0, 300])
def test_launches_that_fill_the_chip_equal_one_launch_per_chunk(kind, window):
    # 128-wide heads: a launch with 256-row tiles for every compute unit or more (here 8 chunks x 8 KV heads x 4 tiles
    # = 256) runs eight wavefronts a workgroup, half of them a phase behind; a chunk launched alone runs four on
    # 128-row tiles. Every bit equal, every kind, ragged counts, with and without a window and sinks; and the oracle.
    pk = kernels()
    counts = [256, 255, 256, 129, 256, 1, 200, 256]
    prefixes = [0, 7, 64, 500, 1023, 1100, 63, 128]
    lengths = [p + c for p, c in zip(prefixes, counts)]
    cache = Cache(kind, 8, 128, 128, 16, lengths, seed=17, scale=0.5)
    starts = [sum(counts[:i]) for i in range(8)]
    q32 = rand_q(sum(counts), 32, 128, 19)
    q = q32.to(torch.float16 if kind == "fp16" else torch.bfloat16)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    positions = torch.tensor(prefixes, dtype=torch.int64, device=dev)
    sinks = torch.linspace(-1, 1, 32, device=dev) if window else None
    kw = dict(key_scales=cache.ks, value_scales=cache.vs, multipliers=cache.multipliers, sliding=window, sinks=sinks)
    lse = torch.empty(q.shape[0], 32, device=dev)
    out = pk.prefill_rows(q, cache.k, cache.v, kind, cache.tables, i32(list(range(8))), i32(starts), i32(counts),
                          positions, 256, 16, lse=lse, **kw)
    for s in range(8):
        rows = slice(starts[s], starts[s] + counts[s])
        one_lse = torch.empty(counts[s], 32, device=dev)
        one = pk.prefill(q[rows], cache.k, cache.v, kind, cache.tables[s], prefixes[s], 16, lse=one_lse, **kw)
        assert torch.equal(out[rows], one), s
        assert torch.equal(lse[rows], one_lse), s
    if not window:
        for s, t in ((0, 0), (3, 128), (4, 255), (5, 0), (7, 100)):
            row = starts[s] + t
            want, want_lse = cache.want(q32[row:row + 1], s, prefixes[s] + t, 1)
            torch.testing.assert_close(out[row:row + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"chunk {s} token {t}")
            torch.testing.assert_close(lse[row:row + 1].double().cpu(), want_lse, atol=1e-3, rtol=1e-4, msg=f"lse {s} {t}")


def test_a_group_of_five_query_heads_in_a_launch_that_fills_the_chip():
    # 40 query heads on 8 KV heads: a token's five rows straddle the 256-row tiles' edges (256 is no multiple of 5).
    pk = kernels()
    counts, prefixes = [256, 200, 256, 77, 256, 256, 13, 256], [0, 70, 64, 900, 511, 1100, 63, 128]
    cache = Cache("bf16", 8, 128, 128, 16, [p + c for p, c in zip(prefixes, counts)], seed=61, scale=0.5)
    starts = [sum(counts[:i]) for i in range(8)]
    q32 = rand_q(sum(counts), 40, 128, 62)
    q = q32.bfloat16()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    positions = torch.tensor(prefixes, dtype=torch.int64, device=dev)
    out = pk.prefill_rows(q, cache.k, cache.v, "bf16", cache.tables, i32(list(range(8))), i32(starts), i32(counts),
                          positions, 256, 16)
    for s in range(8):
        rows = slice(starts[s], starts[s] + counts[s])
        assert torch.equal(out[rows], pk.prefill(q[rows], cache.k, cache.v, "bf16", cache.tables[s], prefixes[s], 16)), s
    for s, t in ((0, 51), (3, 76), (5, 255)):
        row = starts[s] + t
        want, _ = cache.want(q32[row:row + 1], s, prefixes[s] + t, 1)
        torch.testing.assert_close(out[row:row + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"chunk {s} token {t}")


def test_prefill_agrees_with_the_decode_reader_within_the_readers_rounding():
    pk = kernels()
    cache = Cache("bf16", 2, 128, 128, 16, [400])
    q = rand_q(64, 8, 128, 8)
    chunk = pk.prefill(q.bfloat16(), cache.k, cache.v, "bf16", cache.tables[0], 336, 16)
    decode = cache.attend(q, [0], [0], [336], 64)
    torch.testing.assert_close(chunk.float(), decode.float(), atol=1.6e-2, rtol=2e-2)


@pytest.mark.parametrize("window", [1, 100, 1000])
def test_a_sliding_window_and_sinks(window):
    pk = kernels()
    cache = Cache("bf16", 2, 128, 128, 16, [1500])
    q = rand_q(130, 8, 128, 9)
    lse = torch.empty(130, 8, device=dev)
    out = pk.prefill(q.bfloat16(), cache.k, cache.v, "bf16", cache.tables[0], 1370, 16, sliding=window, lse=lse)
    _check(cache, q, out, lse, 1370, (0, 64, 129), sliding=window)
    sinks = torch.linspace(-2, 2, 8, device=dev)
    with_sinks = pk.prefill(q.bfloat16(), cache.k, cache.v, "bf16", cache.tables[0], 1370, 16, sliding=window, sinks=sinks)
    weight = torch.exp(lse) / (torch.exp(lse) + torch.exp(sinks)[None, :])
    torch.testing.assert_close(with_sinks.float(), out.float() * weight[..., None], atol=8e-3, rtol=2e-2)


def test_fp32_outputs_and_warm_up_shapes():
    pk = kernels()
    cache = Cache("bf16", 2, 128, 128, 16, [40])
    q = rand_q(9, 8, 128, 2)
    out = torch.empty(9, 8, 128, dtype=torch.float32, device=dev)
    pk.prefill(q.bfloat16(), cache.k, cache.v, "bf16", cache.tables[0], 31, 16, out=out)
    _check(cache, q, out, None, 31, (0, 8))
    # DeviceAttention's load-time call: one token at position 0 over a one-entry int64 table of the dump page
    dump = torch.full((1,), cache.k.shape[0] - 1, dtype=torch.int64, device=dev)
    one = pk.prefill(q[:1].bfloat16(), cache.k, cache.v, "bf16", dump, 0, 16)
    assert one.shape == (1, 8, 128)


def _fresh_rows(T, hkv, d, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(T, hkv, d, generator=g).to(dtype).to(dev), torch.randn(T, hkv, d, generator=g).to(dtype).to(dev))


@pytest.mark.parametrize("kind", KINDS)
def test_a_chunk_reads_its_own_positions_from_fresh_rows(kind):
    # fresh=(keys, values[, first]): the chunk's positions from `first` on (default: all its own) come from the 16-bit
    # rows given, unscaled, the earlier ones from the pages (the reference's prefill(fresh=), __init__.py:1250-1255):
    # against the oracle for every kind, a first at the chunk's start, inside a key block, at a block's edge, before
    # the chunk (clamped to it) and past it (no fresh position: the bits of the launch without fresh rows, up to the
    # place of FP8 pages' value multiplier); lse too.
    pk = kernels()
    position, T = 200, 150
    cache = Cache(kind, 2, 128, 128, 16, [position + T], seed=23)
    q = rand_q(T, 8, 128, 24)
    q_dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    fk, fv = _fresh_rows(T, 2, 128, 25, q_dtype)
    kw = dict(key_scales=cache.ks, value_scales=cache.vs, multipliers=cache.multipliers)
    plain_lse = torch.empty(T, 8, device=dev)
    plain = pk.prefill(q.to(q_dtype), cache.k, cache.v, kind, cache.tables[0], position, 16, lse=plain_lse, **kw)
    for first in (None, position + 37, 256, 3, position + T, 10 ** 9):
        lse = torch.empty(T, 8, device=dev)
        fresh = (fk, fv) if first is None else (fk, fv, first)
        out = pk.prefill(q.to(q_dtype), cache.k, cache.v, kind, cache.tables[0], position, 16, lse=lse, fresh=fresh, **kw)
        at = position if first is None else min(max(first, position), position + T)
        if at >= position + T:
            if kind == "fp8":      # (the values' multiplier goes into the state, not into the final division: other roundings)
                torch.testing.assert_close(out.float(), plain.float(), atol=ATOL, rtol=RTOL)
            else:
                assert torch.equal(out, plain), first
            assert torch.equal(lse, plain_lse), first
            continue
        for t in (0, 36, 37, 56, 149):
            want, want_lse = cache.want(q[t:t + 1], 0, position + t, 1, fresh=(fk.cpu(), fv.cpu(), position, at))
            torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"first {first} token {t}")
            torch.testing.assert_close(lse[t:t + 1].double().cpu(), want_lse, atol=1e-3, rtol=1e-4, msg=f"first {first} lse {t}")
    on_device = torch.tensor([position + 37], dtype=torch.int64, device=dev)
    a = pk.prefill(q.to(q_dtype), cache.k, cache.v, kind, cache.tables[0], position, 16, fresh=(fk, fv, on_device), **kw)
    b = pk.prefill(q.to(q_dtype), cache.k, cache.v, kind, cache.tables[0], position, 16, fresh=(fk, fv, position + 37), **kw)
    assert torch.equal(a, b)


def test_fresh_rows_from_position_zero_with_a_window_and_sinks_and_a_workspace_of_the_callers():
    # A first chunk (nothing in the pages below it), a sliding window that cuts into the fresh positions and below
    # them, sink logits, and the rows' states in a workspace the caller gives (too small a one is refused).
    pk = kernels()
    cache = Cache("fp8", 2, 128, 128, 16, [700], seed=29)
    q = rand_q(300, 8, 128, 30)
    fk, fv = _fresh_rows(300, 2, 128, 31, torch.bfloat16)
    kw = dict(multipliers=cache.multipliers)
    out = pk.prefill(q.bfloat16(), cache.k, cache.v, "fp8", cache.tables[0], 0, 16, fresh=(fk, fv), **kw)
    for t in (0, 63, 64, 299):
        want, _ = cache.want(q[t:t + 1], 0, t, 1, fresh=(fk.cpu(), fv.cpu(), 0, 0))
        torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"token {t}")
    ws = torch.empty(pk.prefill_state_floats(300, 8, 128), dtype=torch.float32, device=dev)
    for window in (50, 250):
        lse = torch.empty(300, 8, device=dev)
        out = pk.prefill(q.bfloat16(), cache.k, cache.v, "fp8", cache.tables[0], 400, 16, fresh=(fk, fv, 500),
                         sliding=window, lse=lse, workspace=ws, **kw)
        for t in (0, 99, 100, 149, 151, 299):
            want, want_lse = cache.want(q[t:t + 1], 0, 400 + t, 1, sliding=window, fresh=(fk.cpu(), fv.cpu(), 400, 500))
            torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"window {window} token {t}")
            torch.testing.assert_close(lse[t:t + 1].double().cpu(), want_lse, atol=1e-3, rtol=1e-4)
        sinks = torch.linspace(-2, 2, 8, device=dev)
        with_sinks = pk.prefill(q.bfloat16(), cache.k, cache.v, "fp8", cache.tables[0], 400, 16, fresh=(fk, fv, 500),
                                sliding=window, sinks=sinks, workspace=ws, **kw)
        weight = torch.exp(lse) / (torch.exp(lse) + torch.exp(sinks)[None, :])
        torch.testing.assert_close(with_sinks.float(), out.float() * weight[..., None], atol=8e-3, rtol=2e-2)
    with pytest.raises(ValueError):
        pk.prefill(q.bfloat16(), cache.k, cache.v, "fp8", cache.tables[0], 400, 16, fresh=(fk, fv), workspace=ws[:1000], **kw)
    with pytest.raises(ValueError):
        pk.prefill(q.bfloat16(), cache.k, cache.v, "fp8", cache.tables[0], 400, 16, fresh=(fk[:10], fv[:10]), **kw)
    with pytest.raises(ValueError):
        pk.prefill(q.bfloat16(), cache.k, cache.v, "fp8", cache.tables[0], 400, 16, fresh=(fk.float(), fv.float()), **kw)


@pytest.mark.parametrize("kind", ["bf16", "fp8", "int8"])
def test_several_chunks_with_fresh_rows_equal_one_launch_each(kind):
    # prefill_rows(fresh=(keys, values, firsts)): the rows parallel to q's tokens, a first per chunk on the device; a
    # launch that fills the chip (eight wavefronts a workgroup in both of its passes) equals one launch per chunk bit
    # for bit, and firsts of None every chunk's own positions.
    pk = kernels()
    counts = [256, 255, 256, 129, 256, 1, 200, 256]
    prefixes = [0, 7, 64, 500, 1023, 1100, 63, 128]
    firsts = [0, 100, 64, 10 ** 6, 1023 + 255, 1100, 0, 200]
    lengths = [p + c for p, c in zip(prefixes, counts)]
    cache = Cache(kind, 8, 128, 128, 16, lengths, seed=37, scale=0.5)
    starts = [sum(counts[:i]) for i in range(8)]
    q = rand_q(sum(counts), 32, 128, 38).bfloat16()
    fk, fv = _fresh_rows(sum(counts), 8, 128, 39, torch.bfloat16)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    positions = torch.tensor(prefixes, dtype=torch.int64, device=dev)
    kw = dict(key_scales=cache.ks, value_scales=cache.vs, multipliers=cache.multipliers)
    for given in (torch.tensor(firsts, dtype=torch.int64, device=dev), None):
        lse = torch.empty(q.shape[0], 32, device=dev)
        out = pk.prefill_rows(q, cache.k, cache.v, kind, cache.tables, i32(list(range(8))), i32(starts), i32(counts),
                              positions, 256, 16, lse=lse, fresh=(fk, fv, given), **kw)
        for s in range(8):
            rows = slice(starts[s], starts[s] + counts[s])
            one_lse = torch.empty(counts[s], 32, device=dev)
            first = prefixes[s] if given is None else firsts[s]
            one = pk.prefill(q[rows], cache.k, cache.v, kind, cache.tables[s], prefixes[s], 16, lse=one_lse,
                             fresh=(fk[rows], fv[rows], first), **kw)
            assert torch.equal(out[rows], one), s
            assert torch.equal(lse[rows], one_lse), s


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (12, 2, 64), (8, 2, 32), (4, 2, 16), (8, 2, 256)])
def test_int8_queries_against_int8_keys(hq, hkv, d):
    # int8_qk over INT8 pages: the scores are exact integer products of the query rows' INT8 codes (their own scale,
    # amax / 127, half away from zero) and the keys' codes, times both scales: against the oracle with the queries
    # rounded the same way, and within the reference's own bound of the launch that keeps the queries' 16 bits
    # (0.06, test_paged_kv_attention.py:476-479); with a negative scale, a sliding window and sinks; with fresh rows
    # (read in q's type after the pages' integer scores).
    pk = kernels()
    cache = Cache("int8", hkv, d, d, 16, [500], seed=41)
    q = rand_q(150, hq, d, 42)
    kw = dict(key_scales=cache.ks, value_scales=cache.vs)
    lse = torch.empty(150, hq, device=dev)
    out = pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 350, 16, int8_qk=True, lse=lse, **kw)
    exact = pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 350, 16, **kw)
    assert float((out.float() - exact.float()).abs().max()) < 0.06
    for t in (0, 63, 64, 149):
        want, want_lse = cache.want(q[t:t + 1], 0, 350 + t, 1, int8_qk=True)
        torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"token {t}")
        torch.testing.assert_close(lse[t:t + 1].double().cpu(), want_lse, atol=1e-3, rtol=1e-4, msg=f"lse {t}")
    sinks = torch.linspace(-1, 1, hq, device=dev)
    out = pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 350, 16, int8_qk=True, scale=-0.11,
                     sliding=70, lse=lse, **kw)
    for t in (0, 100):
        want, want_lse = cache.want(q[t:t + 1], 0, 350 + t, 1, int8_qk=True, scale=-0.11, sliding=70)
        torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"negative scale, token {t}")
        torch.testing.assert_close(lse[t:t + 1].double().cpu(), want_lse, atol=2e-3, rtol=1e-4)
    with_sinks = pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 350, 16, int8_qk=True, scale=-0.11,
                            sliding=70, sinks=sinks, **kw)
    weight = torch.exp(lse) / (torch.exp(lse) + torch.exp(sinks)[None, :])
    torch.testing.assert_close(with_sinks.float(), out.float() * weight[..., None], atol=8e-3, rtol=2e-2)
    # the chunk's own positions fresh: the pages' part in integers, the fresh part in 16 bits; with every position
    # fresh nothing is left of the integers and the launch equals the one without int8_qk
    fk, fv = _fresh_rows(150, hkv, d, 43, torch.bfloat16)
    mixed = pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 350, 16, int8_qk=True, fresh=(fk, fv), **kw)
    plain = pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 350, 16, fresh=(fk, fv), **kw)
    assert float((mixed.float() - plain.float()).abs().max()) < 0.06
    for t in (0, 1, 75, 149):      # (the oracle scores the pages' positions with the codes, the fresh ones with q itself)
        want, _ = cache.want(q[t:t + 1], 0, 350 + t, 1, int8_qk=True, fresh=(fk.cpu(), fv.cpu(), 350, 350))
        torch.testing.assert_close(mixed[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"int8_qk with fresh rows, token {t}")
    first = pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 0, 16, int8_qk=True, fresh=(fk, fv), **kw)
    assert torch.equal(first, pk.prefill(q.bfloat16(), cache.k, cache.v, "int8", cache.tables[0], 0, 16, fresh=(fk, fv), **kw))


def test_int8_queries_in_a_launch_that_fills_the_chip_equal_one_launch_per_chunk():
    pk = kernels()
    counts = [256, 255, 256, 129, 256, 1, 200, 256]
    prefixes = [0, 7, 64, 500, 1023, 1100, 63, 128]
    cache = Cache("int8", 8, 128, 128, 16, [p + c for p, c in zip(prefixes, counts)], seed=47, scale=0.5)
    starts = [sum(counts[:i]) for i in range(8)]
    q = rand_q(sum(counts), 32, 128, 48).bfloat16()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    positions = torch.tensor(prefixes, dtype=torch.int64, device=dev)
    kw = dict(key_scales=cache.ks, value_scales=cache.vs, int8_qk=True)
    out = pk.prefill_rows(q, cache.k, cache.v, "int8", cache.tables, i32(list(range(8))), i32(starts), i32(counts),
                          positions, 256, 16, **kw)
    for s in range(8):
        rows = slice(starts[s], starts[s] + counts[s])
        assert torch.equal(out[rows], pk.prefill(q[rows], cache.k, cache.v, "int8", cache.tables[s], prefixes[s], 16, **kw)), s


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (12, 2, 64), (8, 2, 256)])
def test_a_nan_query_in_a_prompt_chunk_reaches_its_own_tokens_output_only(hq, hkv, d):
    # a fault upstream shows instead of turning into zeros, and in its own row only (the reference's test_nonfinite.py),
    # at every head width of the matrix-core path
    pk = kernels()
    cache = Cache("bf16", hkv, d, d, 16, [300])
    q = rand_q(4, hq, d, 2).bfloat16()
    lse = torch.empty(4, hq, device=dev)
    clean = pk.prefill(q, cache.k, cache.v, "bf16", cache.tables[0], 200, 16)
    q[1, 0, 0] = float("nan")
    out = pk.prefill(q, cache.k, cache.v, "bf16", cache.tables[0], 200, 16, lse=lse)
    assert bool(torch.isnan(out[1, 0]).all()) and bool(torch.isnan(lse[1, 0]))
    assert torch.equal(out[0], clean[0]) and torch.equal(out[2:], clean[2:]) and torch.equal(out[1, 1:], clean[1, 1:])


def test_what_the_prompt_reader_does_not_take_is_refused():
    pk = kernels()
    cache = Cache("int8", 2, 128, 128, 16, [40])
    q = rand_q(4, 8, 128, 2).bfloat16()
    kw = dict(key_scales=cache.ks, value_scales=cache.vs)
    with pytest.raises(ValueError):      # derive= reads the value pages as keys too: with key pages it is refused
        pk.prefill(q, cache.k, cache.v, "int8", cache.tables[0], 36, 16, derive=(None, 1e-6, None, 0), **kw)
    row = Cache("fp8:row", 2, 128, 128, 16, [40])
    with pytest.raises(ValueError):      # INT8 queries against INT8 keys only
        pk.prefill(q, row.k, row.v, "fp8:row", row.tables[0], 36, 16, int8_qk=True, key_scales=row.ks, value_scales=row.vs)
    with pytest.raises(ValueError):
        pk.prefill(q.float(), cache.k, cache.v, "int8", cache.tables[0], 36, 16, **kw)


@pytest.mark.parametrize("n_chunks", [5, 70])
def test_chunks_are_taken_in_any_order_with_equal_lengths_and_past_the_ranked_limit(n_chunks):
    # Workgroups take the chunks longest first (ranked on the device for up to 64 chunks, ties by index; the caller's
    # order beyond that): whatever the order, every chunk gets its own rows. Equal lengths make every rank a tie.
    pk = kernels()
    lengths = [40 + 16 * (i % 3) for i in range(n_chunks)]
    lengths[1] = lengths[3] = lengths[0]
    counts = [min(n, 24) for n in lengths]
    cache = Cache("bf16", 2, 128, 128, 16, lengths, seed=3, scale=0.5)
    starts = [sum(counts[:i]) for i in range(n_chunks)]
    q = rand_q(sum(counts), 8, 128, 13).bfloat16()
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    positions = torch.tensor([n - c for n, c in zip(lengths, counts)], dtype=torch.int64, device=dev)
    out = pk.prefill_rows(q, cache.k, cache.v, "bf16", cache.tables, i32(list(range(n_chunks))), i32(starts),
                          i32(counts), positions, 32, 16)
    for s in range(n_chunks):
        one = pk.prefill(q[starts[s]:starts[s] + counts[s]], cache.k, cache.v, "bf16", cache.tables[s],
                         lengths[s] - counts[s], 16)
        assert torch.equal(out[starts[s]:starts[s] + counts[s]], one), s


@pytest.mark.parametrize("kind", ["bf16", "fp8", "fp8:row"])
def test_a_negative_or_large_scale_and_a_far_running_maximum(kind):
    # A negative softmax scale (its sign goes into the queries for pages with one scale, into the per-key scales
    # otherwise) and a scale large enough that a row's maximum moves by far more than the slack between key blocks.
    pk = kernels()
    cache = Cache(kind, 2, 128, 128, 16, [300])
    q = rand_q(70, 8, 128, 21)
    for scale in (-0.09, 0.9):
        lse = torch.empty(70, 8, device=dev)
        out = pk.prefill(q.bfloat16(), cache.k, cache.v, kind, cache.tables[0], 230, 16, key_scales=cache.ks,
                         value_scales=cache.vs, multipliers=cache.multipliers, lse=lse, scale=scale)
        for t in (0, 33, 69):
            want, want_lse = cache.want(q[t:t + 1], 0, 230 + t, 1, scale=scale)
            torch.testing.assert_close(out[t:t + 1].double().cpu(), want, atol=ATOL, rtol=RTOL, msg=f"{scale} token {t}")
            torch.testing.assert_close(lse[t:t + 1].double().cpu(), want_lse, atol=2e-3, rtol=1e-4, msg=f"{scale} lse {t}")
