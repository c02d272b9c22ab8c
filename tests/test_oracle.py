"""Pins the CPU oracle before anything is checked against it: reference-held golden vectors, closed forms,
library routines and brute force on tiny inputs. Runs without a GPU."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import append, attend, e4m3

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _vectors():
    pairs = []
    with open(os.path.join(GOLDEN, "e4m3_scale_vectors.txt"), encoding="utf-8") as f:
        for line in f:
            fields = line.split("#", 1)[0].split()
            if fields:
                pairs.append((int(fields[0], 16), int(fields[1], 16)))
    return pairs


# -- E4M3 ----------------------------------------------------------------------------------------------------------------
def test_the_golden_file_holds_the_24_reference_vectors():
    assert len(_vectors()) == 24


def test_integer_encoder_reproduces_every_reference_vector():
    bits = np.array([b for b, _ in _vectors()], dtype=np.uint32).view(np.float32)
    want = np.array([c for _, c in _vectors()], dtype=np.uint8)
    assert np.array_equal(e4m3.encode(bits), want)


def test_torch_cast_with_the_clamp_reproduces_every_reference_vector_and_needs_the_clamp():
    bits = torch.from_numpy(np.array([b for b, _ in _vectors()], dtype=np.uint32).view(np.float32).copy())
    want = torch.tensor([c for _, c in _vectors()], dtype=torch.uint8)
    got = bits.clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(got, want)
    unclamped = bits.to(torch.float8_e4m3fn).view(torch.uint8)
    assert not torch.equal(unclamped, want)        # 1e30 and +inf become NaN codes without it


def test_decoder_matches_the_closed_form_on_every_code():
    codes = np.arange(256, dtype=np.uint8)
    got = e4m3.decode(codes)
    for b in range(256):
        mag = e4m3.magnitude(b)
        if mag is None:
            assert math.isnan(got[b])
        else:
            assert got[b] == (-mag if b & 0x80 else mag), b
    assert e4m3.magnitude(0x7E) == 448.0 and e4m3.magnitude(0x08) == 2.0 ** -6 and e4m3.magnitude(0x01) == 2.0 ** -9


def test_decoder_matches_torchs_cast_back():
    codes = torch.arange(256, dtype=torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    got = e4m3.decode(codes.numpy())
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])


def test_encode_of_every_finite_code_value_is_the_code():
    codes = np.array([b for b in range(256) if (b & 0x7F) != 0x7F], dtype=np.uint8)
    assert np.array_equal(e4m3.encode(e4m3.decode(codes)), codes)      # -0.0 keeps 0x80


def test_integer_encoder_equals_torch_on_every_97th_bit_pattern_in_range():
    # The reference's own check of its encoder (kernels/core/tests/test_core_triton.py:68-77), both signs.
    top = np.float32(448.0).view(np.uint32)
    pos = np.arange(0, int(top) + 1, 97, dtype=np.uint32)
    bits = np.concatenate([pos, pos | np.uint32(0x80000000)])
    x = bits.view(np.float32)
    want = torch.from_numpy(x.copy()).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(e4m3.encode(x), want)


def test_special_values():
    x = np.array([-0.0, -(2.0 ** -10), 2.0 ** -10, 1e-30, 448.0, -448.0, 1e30, -np.inf, np.nan], dtype=np.float32)
    assert e4m3.encode(x).tolist() == [0x80, 0x80, 0x00, 0x00, 0x7E, 0xFE, 0x7E, 0xFE, 0x7F]
    t = torch.from_numpy(x.copy()).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    assert t.tolist() == [0x80, 0x80, 0x00, 0x00, 0x7E, 0xFE, 0x7E, 0xFE, 0x7F]


# -- append ----------------------------------------------------------------------------------------------------------------
def test_slot_math_closed_form_and_known_answers():
    table = [7, 2, 9]
    assert append.slot(table, 0, 16) == 112 and append.slot(table, 15, 16) == 127
    assert append.slot(table, 16, 16) == 32 and append.slot(table, 37, 16) == 9 * 16 + 5
    got = append.slots(torch.tensor(table), torch.arange(48), 16).tolist()
    assert got == [table[p // 16] * 16 + p % 16 for p in range(48)]      # test_rounds.py:34-36's rule
    assert len(set(got)) == 48


def test_bf16_and_fp16_appends_are_round_to_nearest_even():
    x = torch.tensor([1.00390625, 1.01171875, 3.3895313892515355e38, -1.00390625]).view(1, 1, 4)
    bits = append.encode(x, "bf16")[0].view(torch.int16).flatten().tolist()
    assert [b & 0xFFFF for b in bits] == [0x3F80, 0x3F82, 0x7F7F, 0xBF80]
    h = append.encode(torch.tensor([1.00048828125, 1.00146484375]).view(1, 1, 2), "fp16")[0]
    assert [b & 0xFFFF for b in h.view(torch.int16).flatten().tolist()] == [0x3C00, 0x3C02]


@pytest.mark.parametrize("mult", [0.05, 0.07, 1.0, 3.0])
def test_fp8_append_torch_cast_equals_the_integer_encoder(mult):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(64, 3, 128, generator=g) * 3
    x[0, 0, :8] = torch.tensor([0.0, -0.0, 1e30, -1e30, 448.0 * mult, 2.0 ** -10 * mult, float("inf"), 1e-30])
    a = append.encode(x, "fp8", mult)[0].view(torch.uint8)
    b = append.encode_fp8_integer(x, mult)
    assert torch.equal(a, b)


def test_fp8_append_with_one_multiplier_per_head_is_the_scalar_rule_head_by_head():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(10, 4, 64, generator=g) * 2
    mults = torch.tensor([0.01, 0.02, 0.5, 1.5])
    got = append.encode(x, "fp8", mults)[0].view(torch.uint8)
    for h in range(4):
        want = append.encode(x[:, h:h + 1], "fp8", float(mults[h]))[0].view(torch.uint8)
        assert torch.equal(got[:, h:h + 1], want)


def test_division_is_ieee_a_reciprocal_multiply_gives_other_codes():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(100_000, generator=g)
    s = torch.full_like(x, 0.05)
    exact, approx = x / s, x * (1.0 / s)
    assert float((exact != approx).float().mean()) > 0.05
    # The stored FP32 row scales show it directly: amax / 448 is not amax * (1 / 448) for many rows.
    amax = x.abs()
    assert not torch.equal(amax / torch.full_like(amax, 448.0), amax * (1.0 / 448.0))
    assert torch.equal(append.row_scales(x.view(-1, 1), 448.0), (amax / torch.full_like(amax, 448.0)).clamp(min=1e-30))


def test_row_scaled_encodings_follow_their_rules():
    g = torch.Generator().manual_seed(8)
    x = torch.randn(12, 2, 64, generator=g) * 4
    x[3] = 0.0
    codes, scale = append.fp8_rows(x)
    amax = x.abs().amax(-1)
    assert torch.equal(scale, torch.maximum(amax / 448.0, torch.tensor(1e-30)))    # x / 448.0 on CPU is IEEE too
    assert float(scale[3, 0]) == pytest.approx(1e-30) and not bool(codes[3].view(torch.uint8).any())
    back = torch.from_numpy(e4m3.decode(codes.view(torch.uint8).numpy())) * scale[..., None]
    assert float((back - x).abs().max()) <= float(amax.max()) / 16 + 1e-6       # 3 mantissa bits: half a step of 1/8
    # the row's largest magnitude lands on +-448 exactly
    top = codes.view(torch.uint8).view(12, 2, 64)[torch.arange(12) != 3] & 0x7F
    assert bool((top.amax(-1) == 0x7E).all())
    icodes, iscale = append.int8_rows(x)
    assert torch.equal(iscale, torch.maximum(amax / 127.0, torch.tensor(1e-30)))
    assert int(icodes.abs().max()) == 127
    want = torch.round(x / iscale[..., None]).clamp(-127, 127).to(torch.int8)
    assert torch.equal(icodes, want)
    assert torch.round(torch.tensor([0.5, 1.5, 2.5, -0.5])).tolist() == [0.0, 2.0, 2.0, -0.0]    # ties to even


@pytest.mark.parametrize("kind", ["bf16", "fp16", "fp8", "fp8:row", "int8"])
def test_write_places_rows_at_their_slots_and_skips_negative_ones(kind):
    g = torch.Generator().manual_seed(1)
    keys, values = torch.randn(40, 3, 32, generator=g) * 3, torch.randn(40, 3, 16, generator=g)
    k = torch.zeros(4, 16, 3, 32, dtype=append.STORAGE[kind])
    v = torch.zeros(4, 16, 3, 16, dtype=append.STORAGE[kind])
    ks = vs = None
    if kind in append.ROW_SCALED:
        ks, vs = torch.zeros(4, 16, 3), torch.zeros(4, 16, 3)
    ids = torch.randperm(64, generator=g)[:40]
    ids[7] = -1
    append.write(keys, values, ids, k, v, kind, ks, vs, multipliers=(0.05, 0.07))
    keep = ids >= 0
    for x, store, scales, m in ((keys, k, ks, 0.05), (values, v, vs, 0.07)):
        want, want_scale = append.encode(x[keep], kind, m)
        got = store.view(-1, 3, store.shape[-1])[ids[keep]]
        assert torch.equal(append._bytes(got), append._bytes(want))
        if want_scale is not None:
            assert torch.equal(scales.view(-1, 3)[ids[keep]], want_scale)
        untouched = torch.ones(64, dtype=torch.bool)
        untouched[ids[keep]] = False
        assert not bool(store.view(-1, 3, store.shape[-1])[untouched].float().abs().sum())
    # the torch path sends a skipped token to the dump slot instead
    k2 = torch.zeros_like(k)
    append.write(keys, None, ids, k2, None, kind, torch.zeros(4, 16, 3) if ks is not None else None, None,
                 multipliers=(0.05, 0.07), dump_slot=63)
    assert bool(k2.view(-1, 3, 32)[63].float().abs().sum()) or bool((ids == 63).any())


# -- attention ---------------------------------------------------------------------------------------------------------------
def _brute(q, keys, values, seen, scale, group):
    out, lse = [], []
    for h in range(len(q)):
        kv = h // group
        scores = [sum(a * b for a, b in zip(q[h], keys[n][kv])) * scale for n in range(len(keys)) if seen[n]]
        vals = [values[n][kv] for n in range(len(keys)) if seen[n]]
        top = max(scores)
        w = [math.exp(s - top) for s in scores]
        total = sum(w)
        out.append([sum(wi / total * v[c] for wi, v in zip(w, vals)) for c in range(len(vals[0]))])
        lse.append(top + math.log(total))
    return out, lse


def test_reference_attention_equals_brute_force_and_maps_gqa_heads_by_division():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(4, 8, generator=g, dtype=torch.float64)
    keys = torch.randn(9, 2, 8, generator=g, dtype=torch.float64)
    values = torch.randn(9, 2, 5, generator=g, dtype=torch.float64)
    seen = torch.tensor([True] * 6 + [False] * 3)
    out, lse = attend.reference(q, keys, values, seen, 0.3)
    want, want_lse = _brute(q.tolist(), keys.tolist(), values.tolist(), seen.tolist(), 0.3, 2)
    assert torch.allclose(out, torch.tensor(want, dtype=torch.float64), atol=1e-12)
    assert torch.allclose(lse, torch.tensor(want_lse, dtype=torch.float64), atol=1e-12)
    # heads 0,1 read KV head 0 and heads 2,3 read KV head 1: changing KV head 1 moves only heads 2 and 3
    keys2 = keys.clone()
    keys2[:, 1] += 1.0
    out2, _ = attend.reference(q, keys2, values, seen, 0.3)
    assert torch.equal(out2[:2], out[:2]) and not torch.equal(out2[2:], out[2:])


def test_zero_queries_average_the_values_and_unseen_rows_give_zero_and_minus_infinity():
    keys = torch.randn(7, 1, 4, dtype=torch.float64)
    values = torch.arange(14, dtype=torch.float64).view(7, 1, 2)
    out, lse = attend.reference(torch.zeros(2, 4, dtype=torch.float64), keys, values, torch.ones(7, dtype=torch.bool), 1.0)
    assert torch.allclose(out[0], values[:, 0].mean(0)) and float(lse[0]) == pytest.approx(math.log(7))
    out, lse = attend.reference(torch.zeros(2, 4, dtype=torch.float64), keys, values, torch.zeros(7, dtype=torch.bool), 1.0)
    assert not bool(out.any()) and bool(torch.isinf(lse).all()) and bool((lse < 0).all())
    # the attention-state README's worked example (README.md:224-238): zero query over values 2 and 10 -> 6, then 2
    kv = torch.tensor([[[1.0, 0.0]], [[0.0, 1.0]]], dtype=torch.float64)
    vv = torch.tensor([[[2.0]], [[10.0]]], dtype=torch.float64)
    z = torch.zeros(1, 2, dtype=torch.float64)
    assert float(attend.reference(z, kv, vv, torch.tensor([True, True]), 1.0)[0]) == 6.0
    assert float(attend.reference(z, kv, vv, torch.tensor([True, False]), 1.0)[0]) == 2.0


def _pool(kind, hkv, d, dv, page, lengths, seed=0, multipliers=(0.02, 0.03)):
    """One layer's pages over shuffled page tables, written by the oracle's append."""
    g = torch.Generator().manual_seed(seed)
    width = max(math.ceil(n / page) for n in lengths) + 1
    n_pages = width * len(lengths) + 3
    k = torch.zeros(n_pages, page, hkv, d, dtype=append.STORAGE[kind])
    v = torch.zeros(n_pages, page, hkv, dv, dtype=append.STORAGE[kind])
    ks = vs = None
    if kind in append.ROW_SCALED:
        ks, vs = torch.zeros(n_pages, page, hkv), torch.zeros(n_pages, page, hkv)
    tables = torch.randperm(n_pages, generator=g)[:width * len(lengths)].view(len(lengths), width).to(torch.int32)
    raw = []
    for s, n in enumerate(lengths):
        keys, values = torch.randn(n, hkv, d, generator=g), torch.randn(n, hkv, dv, generator=g)
        append.write(keys, values, append.slots(tables[s], torch.arange(n), page), k, v, kind, ks, vs, multipliers)
        raw.append((keys, values))
    return k, v, ks, vs, tables, raw


@pytest.mark.parametrize("kind", ["fp32", "bf16", "fp8", "fp8:row", "int8"])
def test_the_sdpa_cpu_path_and_the_dense_window_agree_with_float64_over_the_stored_values(kind):
    hq, hkv, d, page = 8, 2, 128, 16
    lengths = [64, 200, 333, 512]
    mult = (0.02, 0.03) if kind == "fp8" else (1.0, 1.0)
    k, v, ks, vs, tables, _ = _pool(kind, hkv, d, d, page, lengths, multipliers=mult)
    compute = torch.float32 if kind == "fp32" else torch.bfloat16
    g = torch.Generator().manual_seed(3)
    rows = [(0, 1, 63), (1, 1, 199), (2, 3, 330), (5, 2, 510)]          # (first token, count, first position)
    q = torch.randn(7, hq, d, generator=g)
    scale = d ** -0.5

    def gather_row(r, n):
        return attend.gather(k, v, tables[r], n, page, kind, compute, ks, vs, mult)
    out = attend.sdpa_rows(q, rows, gather_row, scale, torch.empty(7, hq, d))
    tol = 1e-5 if kind == "fp32" else 2e-2
    for r, (first, count, position) in enumerate(rows):
        want, want_lse = attend.window_reference(q[first:first + count], k, v, kind, tables[r], position, count, page,
                                                 scale, ks, vs, mult, q_dtype=compute)
        assert torch.allclose(out[first:first + count].double(), want, atol=tol, rtol=tol)
        keys, values = attend.stored_rows(k, v, tables[r], position + count, page, kind, ks, vs, mult)
        dense, dense_lse = attend.windows_dense(q[first:first + count].to(compute), keys.float(), values.float(),
                                                position, scale)
        assert torch.allclose(dense.double(), want, atol=1e-4, rtol=1e-4)
        assert torch.allclose(dense_lse.double(), want_lse, atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
def test_the_online_fallback_over_page_tables_is_float64_attention_whatever_its_passes(kind):
    # windows_online (the reference's windows_torch) against float64 attention over the stored values: a row whose
    # positions span three passes, verify windows, a sliding window, sinks; passes of another size agree to FP32
    # rounding, and passes past a column's positions leave its sums bit for bit as they were.
    hq, hkv, d, page = 4, 2, 32, 16
    lengths = [40, 700, 333]
    k, v, ks, vs, tables, _ = _pool(kind, hkv, d, d, page, lengths)
    g = torch.Generator().manual_seed(13)
    q = torch.randn(8, hq, d, generator=g).bfloat16().float()
    rows, starts, counts, firsts = [2, 0, 1], [0, 3, 5], [3, 1, 2], [330, 39, 698]
    scale = d ** -0.5
    sinks = torch.tensor([0.5, -1.0, float("-inf"), 2.0])
    for sliding, sink in ((0, None), (24, None), (0, sinks)):
        out, lse = attend.windows_online(q, k, v, kind, tables, rows, starts, counts, firsts, 4, page, scale, ks, vs,
                                         sliding=sliding, sinks=sink, chunk=256)
        for r in range(3):
            span = slice(starts[r], starts[r] + counts[r])
            want, want_lse = attend.window_reference(q[span], k, v, kind, tables[rows[r]], firsts[r], counts[r], page, scale,
                                                     ks, vs, sliding=sliding)
            if sink is not None:      # a sink is one more position with no value: out shrinks by e^lse / (e^lse + e^sink)
                total = torch.logaddexp(want_lse, sink.double()[None, :])
                want, want_lse = want * torch.exp(want_lse - total)[..., None], total
            torch.testing.assert_close(out[span].double(), want, atol=2e-5, rtol=1e-4)
            torch.testing.assert_close(lse[span].double(), want_lse, atol=2e-5, rtol=1e-5)
        assert out[7].eq(0).all() and lse[7].eq(float("-inf")).all()      # a token no window holds
        other, other_lse = attend.windows_online(q, k, v, kind, tables, rows, starts, counts, firsts, 4, page, scale, ks, vs,
                                                 sliding=sliding, sinks=sink, chunk=64)
        torch.testing.assert_close(other, out, atol=2e-5, rtol=1e-4)
        short, short_lse = attend.windows_online(q, k, v, kind, tables, rows[1:2], starts[1:2], counts[1:2], firsts[1:2], 4,
                                                 page, scale, ks, vs, sliding=sliding, sinks=sink, chunk=64, extent=40)
        assert torch.equal(short[3], other[3]) and torch.equal(short_lse[3], other_lse[3])


def test_derived_keys_are_the_normed_weighted_rows_turned_by_their_positions():
    # against rms_norm_rope (pinned above by a scalar loop and torch's rms_norm) where the rotation spans the head, by a
    # scalar float64 loop where it does not, and by what a rotation keeps: each pair's length, and position 0 turns nothing
    g = torch.Generator().manual_seed(23)
    rows = torch.randn(6, 2, 32, generator=g, dtype=torch.float64) * 3
    weight = 1.0 + 0.3 * torch.randn(32, generator=g)
    freqs = (10000.0 ** (-torch.arange(0, 32, 2, dtype=torch.float64) / 32)).float()
    keys = attend.derived_keys(rows, weight, 1e-6, freqs, 32, start=7)
    angle = (torch.arange(7, 13, dtype=torch.float32)[:, None] * freqs[None, :])
    table = torch.cat([angle.double().cos(), angle.double().sin()], 1).float()
    want = append.rms_norm_rope(rows.float(), weight, 1e-6, torch.arange(6), table)
    torch.testing.assert_close(keys.float(), want, atol=2e-6, rtol=2e-6)
    part = attend.derived_keys(rows, None, 1e-6, freqs[:4] * 3, 8, start=2)
    for n in range(6):
        for h in range(2):
            r = rows[n, h]
            y = r / math.sqrt(float((r * r).mean()) + 1e-6)
            for i in range(4):
                t = float(torch.tensor(float(n + 2), dtype=torch.float32) * (freqs[i] * 3))
                assert abs(float(part[n, h, i]) - (float(y[i]) * math.cos(t) - float(y[i + 4]) * math.sin(t))) < 1e-12
                assert abs(float(part[n, h, i + 4]) - (float(y[i + 4]) * math.cos(t) + float(y[i]) * math.sin(t))) < 1e-12
            assert torch.equal(part[n, h, 8:], y[8:])
    still = attend.derived_keys(rows, weight, 0.0, freqs, 32, start=0)
    normed = rows / torch.sqrt((rows * rows).mean(-1, keepdim=True)) * weight.double()
    torch.testing.assert_close(still[0], normed[0], atol=1e-14, rtol=1e-14)
    torch.testing.assert_close(still[..., :16] ** 2 + still[..., 16:] ** 2, normed[..., :16] ** 2 + normed[..., 16:] ** 2, atol=1e-12, rtol=1e-12)


def test_latent_attention_is_attention_over_latent_and_rotary_keys_with_the_latent_as_value():
    from oracle import latent as oracle_latent
    g = torch.Generator().manual_seed(29)
    T, H, R, P, N = 3, 4, 8, 4, 11
    ql, qr = torch.randn(T, H, R, generator=g, dtype=torch.float64), torch.randn(T, H, P, generator=g, dtype=torch.float64)
    c, k = torch.randn(N, R, generator=g, dtype=torch.float64), torch.randn(N, P, generator=g, dtype=torch.float64)
    seen = torch.arange(N)[None, :] <= torch.tensor([4, 10, 0])[:, None]
    seen[2, 0] = False                                       # a token that sees nothing
    scale = 0.3
    out, lse = oracle_latent.latent_attention(ql, qr, c, k, seen, scale)
    for t in range(T):
        # ordinary attention with one KV head: keys the whole rows, values their latents
        want, want_lse = attend.reference(torch.cat([ql[t], qr[t]], -1), torch.cat([c, k], -1)[:, None], c[:, None], seen[t], scale)
        torch.testing.assert_close(out[t], want, atol=1e-12, rtol=1e-12)
        torch.testing.assert_close(lse[t], want_lse, atol=1e-12, rtol=1e-12)
    # a scalar loop
    t, h = 1, 2
    scores = [scale * (sum(float(ql[t, h, i]) * float(c[n, i]) for i in range(R)) + sum(float(qr[t, h, i]) * float(k[n, i]) for i in range(P)))
              for n in range(N)]
    top = max(scores)
    w = [math.exp(x - top) for x in scores]
    for i in range(R):
        assert abs(float(out[t, h, i]) - sum(wn * float(c[n, i]) for n, wn in enumerate(w)) / sum(w)) < 1e-12
    assert abs(float(lse[t, h]) - (top + math.log(sum(w)))) < 1e-12
    assert out[2].eq(0).all() and lse[2].eq(float("-inf")).all()
    # a sink is one more position with no value: out shrinks by e^lse / (e^lse + e^sink), lse grows to their logaddexp
    sinks = torch.tensor([0.5, float("-inf"), -2.0, 3.0], dtype=torch.float64)
    with_sinks, sink_lse = oracle_latent.latent_attention(ql, qr, c, k, seen, scale, sinks)
    total = torch.logaddexp(lse, sinks[None, :])
    torch.testing.assert_close(sink_lse, total, atol=1e-12, rtol=1e-12)
    torch.testing.assert_close(with_sinks[:2], (out * torch.exp(lse - total)[..., None])[:2], atol=1e-12, rtol=1e-12)
    assert with_sinks[2].eq(0).all() and sink_lse[2, 1] == float("-inf") and sink_lse[2, 0] == 0.5


def test_a_latent_caches_rows_are_the_latent_then_the_rotary_key_each_part_coded_at_its_own_scale():
    from oracle import latent as oracle_latent
    g = torch.Generator().manual_seed(31)
    n, R, P, page = 9, 16, 8, 4
    latent, rope = torch.randn(n, R, generator=g), torch.randn(n, P, generator=g) * 5
    latent[3] = 0                                            # a row of zeros: the floor of 1e-30
    table = torch.tensor([2, 0, 3])
    slots = table[torch.arange(n) // page] * page + torch.arange(n) % page
    cache = torch.zeros(4, page, R + P, dtype=torch.bfloat16)
    oracle_latent.write(latent, rope, slots, cache)
    got_l, got_r = oracle_latent.stored(cache, None, table, n, page, R)
    assert torch.equal(got_l, latent.bfloat16().double()) and torch.equal(got_r, rope.bfloat16().double())
    codes, scales = torch.zeros(4, page, R + P, dtype=torch.float8_e4m3fn), torch.zeros(4, page, 2)
    oracle_latent.write(latent, rope, slots, codes, scales)
    flat, sc = codes.view(-1, R + P).view(torch.uint8), scales.view(-1, 2)
    for i, s in enumerate(slots.tolist()):
        for part, lo, hi, which in ((latent[i], 0, R, 0), (rope[i], R, R + P, 1)):
            want, scale = append.encode(part[None, None, :], "fp8:row")      # the pool's rule for a row: amax / 448, IEEE
            assert torch.equal(flat[s, lo:hi], want.view(torch.uint8)[0, 0]) and float(sc[s, which]) == float(scale[0, 0])
    assert float(sc[slots[3], 0]) == 1e-30 or abs(float(sc[slots[3], 0]) - 1e-30) < 1e-37
    got_l, got_r = oracle_latent.stored(codes, scales, table, n, page, R)
    torch.testing.assert_close(got_l.float(), latent, atol=0.07, rtol=0.07)


def test_the_transactional_state_follows_the_references_known_answers():
    from oracle.state import KVState
    state = KVState(capacity=3, key_width=2, value_width=1)      # README.md:224-238, test_techniques.py:471-482
    state.stage((1.0, 0.0), (2.0,))
    state.stage((0.0, 1.0), (10.0,))
    assert state.attend((0.0, 0.0), include_pending=True) == (6.0,)
    state.commit(1)
    assert state.attend((0.0, 0.0)) == (2.0,) and state.pending == []
    state.stage((1.0, 1.0), (99.0,))
    state.rollback()
    assert len(state.committed) == 1 and state.attend((0.0, 0.0)) == (2.0,)
    one = KVState(1, 1, 1)                                         # test_techniques.py:484-494
    with pytest.raises(ValueError):
        one.attend((1,))
    one.stage((1,), (2,))
    with pytest.raises(ValueError):
        one.stage((2,), (3,))
    with pytest.raises(ValueError):
        one.commit(2)
    assert len(one.pending) == 1
    for bad in ((0, 1, 1), (1, 1.0, 1)):
        with pytest.raises(ValueError):
            KVState(*bad)
    with pytest.raises(ValueError):
        one.stage((float("nan"),), (1,))
    # its softmax is float64 attention over the rows it holds
    g = torch.Generator().manual_seed(17)
    keys, values = torch.randn(9, 4, generator=g, dtype=torch.float64), torch.randn(9, 3, generator=g, dtype=torch.float64)
    query = torch.randn(4, generator=g, dtype=torch.float64)
    state = KVState(16, 4, 3)
    for key, value in zip(keys.tolist(), values.tolist()):
        state.stage(key, value)
    state.commit(6)
    want, _ = attend.reference(query[None], keys[:6, None], values[:6, None], torch.ones(6, dtype=torch.bool), 0.5)
    torch.testing.assert_close(torch.tensor(state.attend(query.tolist()), dtype=torch.float64), want[0], atol=1e-12, rtol=1e-12)
    assert state.pending == [] and len(state.committed) == 6      # the rejected suffix is gone


def test_a_sliding_window_sees_only_its_last_positions():
    k, v, ks, vs, tables, _ = _pool("bf16", 1, 16, 16, 16, [100])
    q = torch.randn(2, 2, 16, generator=torch.Generator().manual_seed(4))
    out, _ = attend.window_reference(q, k, v, "bf16", tables[0], 98, 2, 16, 0.25, sliding=8)
    keys, values = attend.stored_rows(k, v, tables[0], 100, 16, "bf16")
    for c in range(2):
        seen = torch.zeros(100, dtype=torch.bool)
        seen[98 + c - 7:98 + c + 1] = True
        want, _ = attend.reference(q[c].bfloat16().double(), keys, values, seen, 0.25)
        assert torch.equal(out[c], want)
    dense, _ = attend.windows_dense(q.bfloat16(), keys.float(), values.float(), 98, 0.25, sliding=8)
    assert torch.allclose(dense.double(), out, atol=1e-5)


# -- online softmax steps and merges -------------------------------------------------------------------------------------
@pytest.mark.parametrize("cuts", [[5], [1, 2, 3], [0, 7], [3, 3]])
def test_folding_any_cut_of_the_scores_equals_one_pass(cuts):
    g = torch.Generator().manual_seed(9)
    s = torch.randn(3, 11, generator=g, dtype=torch.float64) * 4
    s[1, :] = float("-inf")                                       # a row that sees nothing
    s[2, 4:] = float("-inf")
    vals = torch.randn(11, 5, generator=g, dtype=torch.float64)
    bounds = [0] + cuts + [11]
    m_run = torch.full((3,), float("-inf"), dtype=torch.float64)
    l_run = torch.zeros(3, dtype=torch.float64)
    acc_run = torch.zeros(3, 5, dtype=torch.float64)
    for a, b in zip(bounds[:-1], bounds[1:]):
        m = torch.full((3,), float("-inf"), dtype=torch.float64)
        if b > a:
            p, alpha, m = attend.step(s[:, a:b], m)
            l, acc = p.sum(1), p @ vals[a:b]
        else:
            l, acc = torch.zeros(3, dtype=torch.float64), torch.zeros(3, 5, dtype=torch.float64)
        m_run, l_run, keep, take = attend.fold(m_run, l_run, m, l)
        acc_run = acc_run * keep[:, None] + acc * take[:, None]
    out, lse = attend.finish(acc_run, l_run), attend.lse(m_run, l_run)
    want = torch.softmax(s[[0, 2]], 1) @ vals
    assert torch.allclose(out[[0, 2]], want, atol=1e-12)
    assert torch.allclose(lse[[0, 2]], torch.logsumexp(s[[0, 2]], 1), atol=1e-12)
    assert not bool(out[1].any()) and float(lse[1]) == float("-inf") and not bool(torch.isnan(out).any())


def test_merge_reproduces_the_readme_worked_example_and_the_host_oracle():
    # inference/partitioned-attention/README.md:48-62: four ranks share two tokens, two are empty -> 5.0
    rows = ((0, (1., 0.), (2.,)), (1, (0., 1.), (8.,)))
    parts = [attend.attention_partial((1., 1.), [r for r in rows if attend.owner(r[0], 4) == rank], 1, 1)
             for rank in range(4)]
    assert attend.merge_partials(parts)[0] == (5.,)
    assert attend.global_position(3, 4, 1) == 13
    assert attend.attention_partial((1., 1.), rows, 1, 0)[0] == (2.,)
    with pytest.raises(ValueError):
        attend.merge_partials([((0.0,), -math.inf)] * 2)
    outs = [torch.tensor(o).view(1, 1, 1) for o, _ in parts]
    lses = [torch.tensor(l).view(1, 1) for _, l in parts]
    out, lse = attend.merge(outs, lses)
    assert float(out) == pytest.approx(5.0) and float(lse) == pytest.approx(attend.merge_partials(parts)[1])


def test_merge_skips_parts_without_keys_and_gives_zero_for_a_token_no_part_saw():
    # inference/partitioned-attention/tests/test_device.py:70-77
    outs = [torch.ones(2, 1, 3), torch.zeros(2, 1, 3)]
    lses = [torch.tensor([[0.5], [float("-inf")]]), torch.full((2, 1), float("-inf"))]
    out, lse = attend.merge(outs, lses)
    assert out[0].tolist() == [[1.0, 1.0, 1.0]]
    assert (out[1].tolist(), lse[1].tolist()) == ([[0.0, 0.0, 0.0]], [float("-inf")])
    assert float(lse[0, 0]) == pytest.approx(0.5, abs=1e-6)


@pytest.mark.parametrize("cut", [1, 120, 299])
def test_merged_shards_equal_attention_over_the_whole_whatever_the_cut(cut):
    g = torch.Generator().manual_seed(1)
    keys, values = torch.randn(300, 2, 64, generator=g).double(), torch.randn(300, 2, 64, generator=g).double()
    q = torch.randn(4, 64, generator=g).double()
    every = torch.ones(300, dtype=torch.bool)
    want, want_lse = attend.reference(q, keys, values, every, 0.125)
    a = attend.reference(q, keys[:cut], values[:cut], every[:cut], 0.125)
    b = attend.reference(q, keys[cut:], values[cut:], every[cut:], 0.125)
    out, lse = attend.merge([a[0][None].float(), b[0][None].float()], [a[1][None].float(), b[1][None].float()])
    assert torch.allclose(out[0].double(), want, atol=1e-5) and torch.allclose(lse[0].double(), want_lse, atol=1e-5)


def test_a_draft_tree_column_sees_what_its_path_alone_would_hold():
    # Pins seen_by(): the reference's tree of its own tests (tests/test_cuda.py:113) against an independent statement
    # of the rule. A column's attention over the tree equals plain causal attention over a sequence that holds the
    # prefix and then only the column's path (root .. column) at consecutive positions, which is what the reference's
    # pool makes of an accepted path (pages.py:662-684); a chain is the causal window; a star sees the root and itself.
    k, v, ks, vs, tables, _ = _pool("bf16", 1, 16, 16, 16, [48])
    q = torch.randn(8, 2, 16, generator=torch.Generator().manual_seed(5))
    parents = [-1, 0, 0, 1, 1, 2, 5, 3]
    first = 40
    out, lse = attend.window_reference(q, k, v, "bf16", tables[0], first, 8, 16, 0.25, parents=parents)
    keys, values = attend.stored_rows(k, v, tables[0], 48, 16, "bf16")
    paths = {0: [0], 1: [0, 1], 2: [0, 2], 3: [0, 1, 3], 4: [0, 1, 4], 5: [0, 2, 5], 6: [0, 2, 5, 6], 7: [0, 1, 3, 7]}
    for c, path in paths.items():
        index = torch.tensor(list(range(first)) + [first + a for a in path])
        want, want_lse = attend.reference(q[c].bfloat16().double(), keys[index], values[index],
                                          torch.ones(len(index), dtype=torch.bool), 0.25)
        assert torch.allclose(out[c], want, atol=1e-12, rtol=1e-12), c
        assert torch.allclose(lse[c], want_lse, atol=1e-12, rtol=1e-12), c
        assert attend.seen_by(first, 8, c, 48, parents).sum() == first + len(path)
    chain, _ = attend.window_reference(q, k, v, "bf16", tables[0], first, 8, 16, 0.25, parents=list(range(-1, 7)))
    plain, _ = attend.window_reference(q, k, v, "bf16", tables[0], first, 8, 16, 0.25)
    assert torch.equal(chain, plain)
    star = attend.seen_by(first, 8, 5, 48, [-1, 0, 0, 0, 0, 0, 0, 0])
    assert star.nonzero().flatten().tolist() == list(range(first)) + [first, first + 5]
    slid = attend.seen_by(first, 8, 6, 48, parents, sliding=3)       # positions > 40 + 6 - 3 of the path 0, 2, 5, 6
    assert slid.nonzero().flatten().tolist() == [first + 5, first + 6]


def test_a_block_list_sees_what_a_sequence_of_only_its_blocks_would_hold():
    # Pins listed() and its use in window_reference(): a token with a list of KV blocks attends as a plain token would
    # over a sequence that holds only the listed blocks' positions up to the token's own, in any order of the list;
    # ids of -1, blocks past the token's position and blocks past the sequence add nothing; every block listed is
    # plain causal attention; an empty list gives zeros and -inf. Block sizes that divide the page, that do not, and
    # one larger than a page (the reference tests 4, 16 and 80: test_paged_kv_attention.py:374).
    k, v, ks, vs, tables, _ = _pool("bf16", 1, 16, 16, 16, [200])
    q = torch.randn(2, 2, 16, generator=torch.Generator().manual_seed(6))
    keys, values = attend.stored_rows(k, v, tables[0], 200, 16, "bf16")
    first = 150
    for bs in (4, 16, 80, 7):
        nblk = math.ceil(200 / bs)
        lists = [[nblk - 1, 0, -1, (first + 1) // bs, 2, 10 ** 6, -1], [1, (first // bs), nblk + 3, -1, -1, -1, -1]]
        out, lse = attend.window_reference(q, k, v, "bf16", tables[0], first, 2, 16, 0.25, blocks=lists, block_size=bs)
        for c in range(2):
            own = first + c
            index = sorted({n for b in lists[c] if b >= 0 for n in range(b * bs, (b + 1) * bs) if n <= own and n < 200})
            assert attend.listed(lists[c], bs, 200).nonzero().flatten().tolist() == \
                sorted({n for b in lists[c] if b >= 0 for n in range(b * bs, (b + 1) * bs) if n < 200})
            want, want_lse = attend.reference(q[c].bfloat16().double(), keys[index], values[index],
                                              torch.ones(len(index), dtype=torch.bool), 0.25)
            assert torch.allclose(out[c], want, atol=1e-12, rtol=1e-12), (bs, c)
            assert torch.allclose(lse[c], want_lse, atol=1e-12, rtol=1e-12), (bs, c)
        every = [list(range(nblk)), list(range(nblk))[::-1]]
        full, _ = attend.window_reference(q, k, v, "bf16", tables[0], first, 2, 16, 0.25, blocks=every, block_size=bs)
        plain, _ = attend.window_reference(q, k, v, "bf16", tables[0], first, 2, 16, 0.25)
        assert torch.equal(full, plain)
    none, none_lse = attend.window_reference(q, k, v, "bf16", tables[0], first, 2, 16, 0.25, blocks=[[-1], [-1]], block_size=16)
    assert bool((none == 0).all()) and bool(torch.isinf(none_lse).all())


def test_fresh_rows_replace_the_positions_from_their_first_on_unscaled():
    # Pins with_fresh() and its use in window_reference(): a chunk that reads its positions from `first` on from fresh
    # 16-bit rows attends as a plain chunk would over a 16-bit pool whose pages hold, at those positions, the fresh rows
    # (written by hand below, not through with_fresh) and elsewhere the pages' decoded values; the page scales do not
    # touch a fresh position (FP8 pages with multipliers 0.5 / 0.25: a fresh row counts as given); fresh rows that
    # equal the stored ones, and a first past the chunk, change nothing; the worked case of one key: a token that sees
    # only a fresh position returns that row's value whatever the pages hold.
    gen = torch.Generator().manual_seed(11)
    k, v, ks, vs, tables, _ = _pool("fp8", 1, 16, 16, 16, [100])
    position, T = 60, 40
    q = torch.randn(T, 2, 16, generator=gen)
    fk = torch.randn(T, 1, 16, generator=gen).bfloat16()
    fv = torch.randn(T, 1, 16, generator=gen).bfloat16()
    mult = (0.5, 0.25)
    keys, values = attend.stored_rows(k, v, tables[0], 100, 16, "fp8", multipliers=mult)
    for first in (position, position + 13, 0, 10 ** 6):
        out, lse = attend.window_reference(q, k, v, "fp8", tables[0], position, T, 16, 0.25, multipliers=mult,
                                           fresh=(fk, fv, position, max(first, position)))
        kk, vv = keys.clone(), values.clone()
        for n in range(max(first, position), 100):
            kk[n], vv[n] = fk[n - position].double(), fv[n - position].double()
        for c in (0, 12, 13, 39):
            seen = torch.arange(100) <= position + c
            want, want_lse = attend.reference(q[c].bfloat16().double(), kk, vv, seen, 0.25)
            assert torch.allclose(out[c], want, atol=1e-12, rtol=1e-12), (first, c)
            assert torch.allclose(lse[c], want_lse, atol=1e-12, rtol=1e-12), (first, c)
    plain, plain_lse = attend.window_reference(q, k, v, "fp8", tables[0], position, T, 16, 0.25, multipliers=mult)
    none, none_lse = attend.window_reference(q, k, v, "fp8", tables[0], position, T, 16, 0.25, multipliers=mult,
                                             fresh=(fk, fv, position, 10 ** 6))
    assert torch.equal(plain, none) and torch.equal(plain_lse, none_lse)
    k16, v16, _, _, t16, _ = _pool("bf16", 1, 16, 16, 16, [100])
    own_k, own_v = attend.stored_rows(k16, v16, t16[0], 100, 16, "bf16")
    same, _ = attend.window_reference(q, k16, v16, "bf16", t16[0], position, T, 16, 0.25,
                                      fresh=(own_k[position:].bfloat16(), own_v[position:].bfloat16(), position, position))
    assert torch.equal(same, attend.window_reference(q, k16, v16, "bf16", t16[0], position, T, 16, 0.25)[0])
    one, one_lse = attend.window_reference(q[:1], k, v, "fp8", tables[0], 0, 1, 16, 0.25, multipliers=mult,
                                           fresh=(fk, fv, 0, 0))
    assert torch.allclose(one[0], fv[0, 0].double().expand(2, 16), atol=1e-12)
    assert torch.allclose(one_lse[0], (q[0].bfloat16().double() @ fk[0, 0].double()) * 0.25, atol=1e-12)


def test_int8_query_rows_are_their_codes_times_their_scale():
    # Pins int8_rows(): known answers (amax maps to +-127; halves round away from zero; a zero row stays zero at the
    # floor scale), the closed form codes = round_half_away(q * 127 / amax) on random rows, |codes| <= 127, an error of
    # at most half a step, and its use in window_reference(): the same as attending with the rounded queries.
    q = torch.tensor([[127.0, -127.0, 63.5, -63.5, 0.4, -0.6, 0.0, 1.0], [0.0] * 8, [2.0, 1.0, 0.5, 0.25, -2.0, 0.0, 0.0, 0.0]])
    got = attend.int8_rows(q)
    assert got[0].tolist() == [127.0, -127.0, 64.0, -64.0, 0.0, -1.0, 0.0, 1.0]
    assert got[1].tolist() == [0.0] * 8
    step = 2.0 / 127.0
    assert torch.allclose(got[2], torch.tensor([127, 64, 32, 16, -127, 0, 0, 0], dtype=torch.float64) * float(torch.tensor(step)), atol=1e-12)
    x = torch.randn(64, 128, generator=torch.Generator().manual_seed(3)).bfloat16().float()
    amax = x.abs().amax(-1, keepdim=True)
    scale = (amax / 127.0).double()
    codes = attend.int8_rows(x) / scale
    assert bool((codes == codes.round()).all()) and float(codes.abs().max()) <= 127
    assert float((attend.int8_rows(x) - x.double()).abs().max() / scale.max()) <= 0.5 + 1e-6
    k, v, ks, vs, tables, _ = _pool("int8", 1, 16, 16, 16, [60])
    q = torch.randn(3, 2, 16, generator=torch.Generator().manual_seed(4))
    out, lse = attend.window_reference(q, k, v, "int8", tables[0], 57, 3, 16, 0.25, ks, vs, int8_qk=True)
    keys, values = attend.stored_rows(k, v, tables[0], 60, 16, "int8", ks, vs)
    for c in range(3):
        want, want_lse = attend.reference(attend.int8_rows(q[c].bfloat16()), keys, values, torch.arange(60) <= 57 + c, 0.25)
        assert torch.allclose(out[c], want, atol=1e-12) and torch.allclose(lse[c], want_lse, atol=1e-12)


def test_an_int8_chunks_fresh_rows_meet_the_queries_as_they_are():
    # Pins window_reference(int8_qk=True, fresh=...) and reference(late=): the pages' positions are scored with the
    # queries' INT8 codes times their scale, the fresh ones (from `first` on) with the 16-bit queries themselves
    # (_kernels.py:668-671 against 708-709). Checked against a softmax written out position by position in plain Python.
    k, v, ks, vs, tables, _ = _pool("int8", 2, 16, 16, 16, [40])
    g = torch.Generator().manual_seed(9)
    q = torch.randn(3, 4, 16, generator=g)
    fk, fv = torch.randn(3, 2, 16, generator=g).bfloat16(), torch.randn(3, 2, 16, generator=g).bfloat16()
    first = 38                                           # the chunk is positions 37..39; 38 and 39 are fresh
    out, lse = attend.window_reference(q, k, v, "int8", tables[0], 37, 3, 16, 0.25, ks, vs, int8_qk=True,
                                       fresh=(fk, fv, 37, first))
    keys, values = attend.stored_rows(k, v, tables[0], 40, 16, "int8", ks, vs)
    coded, given = attend.int8_rows(q.bfloat16()), q.bfloat16().double()
    for c in range(3):
        for h in range(4):
            scores, rows = [], []
            for n in range(37 + c + 1):
                if n >= first:
                    key, value, query = fk[n - 37, h // 2].double(), fv[n - 37, h // 2].double(), given[c, h]
                else:
                    key, value, query = keys[n, h // 2], values[n, h // 2], coded[c, h]
                scores.append(float(key @ query) * 0.25)
                rows.append(value)
            top = max(scores)
            weights = [math.exp(x - top) for x in scores]
            total = sum(weights)
            want = sum(w / total * r for w, r in zip(weights, rows))
            assert torch.allclose(out[c, h], want, atol=1e-12), (c, h)
            assert abs(float(lse[c, h]) - (top + math.log(total))) < 1e-12
    # the difference is there to see: scoring the fresh rows with the codes too gives another answer
    other, _ = attend.window_reference(q, k, v, "int8", tables[0], 37, 3, 16, 0.25, ks, vs, int8_qk=True)
    assert not torch.allclose(out, other, atol=1e-4)


# -- the pool's device-side bookkeeping ------------------------------------------------------------------------------------
def _round_pool(page=4, table_pages=6, lengths=((0, 17), (1, 9), (3, 24)), round_slots=4, seed=0):
    """Round tables of a few bound sequences over shuffled pages; unbound slots and the entries past a sequence's pages
    at the dump page (test_rounds.py:52-54)."""
    g = torch.Generator().manual_seed(seed)
    pages = round_slots * table_pages
    order = torch.randperm(pages, generator=g).tolist()
    tables = torch.full((round_slots, table_pages), pages, dtype=torch.int32)
    capacity = torch.zeros(round_slots, dtype=torch.int64)
    for s, n in lengths:
        held = -(-n // page)
        tables[s, :held] = torch.tensor([order.pop() for _ in range(held)], dtype=torch.int32)
        capacity[s] = n
    return tables, capacity, pages


def test_slots_at_is_the_closed_form_inside_a_slots_capacity_and_the_dump_page_outside():
    from oracle import pool
    page = 4
    tables, capacity, dump = _round_pool(page)
    slot = torch.tensor([[0, 0, 0, 0], [1, 1, 1, 1], [2, 2, 3, 3]])
    where = torch.tensor([[0, 5, 16, 17], [8, 9, -1, 400], [0, 3, 23, 24]])
    got = pool.slots_at(tables, capacity, slot, where, page, dump)
    for s, p, found in zip(slot.reshape(-1).tolist(), where.reshape(-1).tolist(), got.reshape(-1).tolist()):
        if 0 <= p < int(capacity[s]):
            assert found == int(tables[s, p // page]) * page + p % page      # test_rounds.py:34-36
        else:
            assert found == dump * page      # past capacity, before 0, an unbound slot: test_rounds.py:58-60, 289
    inside = got[(where >= 0) & (where < capacity[slot])]
    assert len(set(inside.tolist())) == inside.numel() and int(inside.max()) < dump * page
    # a round's reserve: each token's row's slot first (pages.py:652-653)
    slots_t, rows_t = torch.tensor([3, 0]), torch.tensor([0, 0, 1, 1, 1])
    positions = torch.tensor([22, 23, 15, 16, 17])
    got = pool.reserve_round(tables, capacity, slots_t, rows_t, positions, page, dump).tolist()
    want = [int(tables[3, 5]) * 4 + 2, int(tables[3, 5]) * 4 + 3, int(tables[0, 3]) * 4 + 3, int(tables[0, 4]) * 4, dump * 4]
    assert got == want


def _sequence_rows(store, table, positions, page):
    at = torch.tensor([int(table[p // page]) * page + p % page for p in positions])
    return store[:, at]


def test_compact_moves_an_accepted_path_to_consecutive_positions_once():
    from oracle import pool
    page, layers = 4, 2
    # one sequence of 30 tokens bound with room for 80 (test_rounds.py:190-215): a window of 6 at 30, the nodes 0, 2
    # and 5 accepted
    tables, capacity, dump = _round_pool(page, table_pages=20, lengths=((0, 80),), round_slots=2)
    slots = (dump + 1) * page
    g = torch.Generator().manual_seed(1)
    keys = torch.randn(layers, slots, 2, 16, generator=g).bfloat16()
    scales = torch.rand(layers, slots, 2, generator=g)
    before_k, before_s = keys.clone(), scales.clone()
    start, emitted, moved = torch.tensor([30, 0]), torch.tensor([3, 0]), torch.zeros(2, dtype=torch.int64)
    path = torch.tensor([[0, 2, 5, -1, -1, -1]])
    pool.compact([keys, None, scales], slots, tables, capacity, start, emitted, path, moved, page, dump)
    for now, was in ((keys, before_k), (scales, before_s)):
        got, old = _sequence_rows(now, tables[0], range(36), page), _sequence_rows(was, tables[0], range(36), page)
        assert torch.equal(got[:, :30], old[:, :30])
        assert torch.equal(got[:, 30:33], old[:, [30, 32, 35]])
        assert torch.equal(got[:, 33:], old[:, 33:])      # what lies past the new frontier is left as it was
    assert moved.tolist() == [1, 0]
    again = keys.clone()
    pool.compact([keys, None, scales], slots, tables, capacity, start, emitted, path, moved, page, dump)
    assert torch.equal(keys, again)      # a second commit finds the path moved (test_rounds.py:211)
    # a held row (nothing emitted) moves nothing
    moved.zero_()
    pool.compact([keys], slots, tables, capacity, start, torch.tensor([0, 0]), path, moved, page, dump)
    assert torch.equal(keys, again)


def test_compact_reads_every_source_before_it_writes_a_target():
    from oracle import pool
    # path [0, 1, 3, 2 ...] would be no tree, but the rule is index_copy_(index_select()): position 2 is column 2's
    # target and column 3's source, and column 3 must still deliver position 2's old row. A model that moves one row
    # after the other in column order delivers the new one and must differ.
    page = 4
    tables, capacity, dump = _round_pool(page, table_pages=8, lengths=((0, 30), (1, 30)), round_slots=2)
    slots = (dump + 1) * page
    values = torch.arange(slots, dtype=torch.float32).view(1, slots, 1).repeat(1, 1, 3).contiguous()
    before = values.clone()
    start, emitted, moved = torch.tensor([8, 5]), torch.tensor([4, 3]), torch.zeros(2, dtype=torch.int64)
    path = torch.tensor([[0, 1, 3, 2, 4], [0, 4, 1, 3, -1]])
    pool.compact([values], slots, tables, capacity, start, emitted, path, moved, page, dump)
    old0 = _sequence_rows(before, tables[0], range(14), page)
    got0 = _sequence_rows(values, tables[0], range(14), page)
    assert torch.equal(got0[:, 8:12], old0[:, [8, 9, 11, 10]])
    assert torch.equal(got0[:, 12:], old0[:, 12:])
    old1 = _sequence_rows(before, tables[1], range(10), page)
    got1 = _sequence_rows(values, tables[1], range(10), page)
    assert torch.equal(got1[:, 5:8], old1[:, [5, 9, 6]])      # column 3 lies at emitted: not moved
    assert torch.equal(got1[:, 8:], old1[:, 8:])
    one_by_one = before.clone()
    for j, node in ((1, 1), (2, 3), (3, 2)):
        src, dst = int(tables[0, (8 + node) // 4]) * 4 + (8 + node) % 4, int(tables[0, (8 + j) // 4]) * 4 + (8 + j) % 4
        one_by_one[:, dst] = one_by_one[:, src]
    assert not torch.equal(_sequence_rows(one_by_one, tables[0], range(14), page), got0)


def test_copy_pages_copies_whole_pages_in_every_layer_and_store():
    from oracle import pool
    page, pages, layers = 4, 10, 3
    g = torch.Generator().manual_seed(2)
    keys = torch.randn(layers, pages * page, 2, 8, generator=g)
    codes = torch.randint(0, 255, (layers, pages * page, 2, 8), generator=g, dtype=torch.uint8).view(torch.float8_e4m3fn)
    before_k, before_c = keys.clone(), codes.clone()
    pool.copy_pages([keys, codes], pages * page, torch.tensor([3, -1, 7]), torch.tensor([0, 5, 9]), page)
    for now, was in ((keys, before_k), (codes.view(torch.uint8), before_c.view(torch.uint8))):
        paged, old = now.view(layers, pages, -1), was.view(layers, pages, -1)
        assert torch.equal(paged[:, 0], old[:, 3]) and torch.equal(paged[:, 9], old[:, 7])
        rest = [1, 2, 3, 4, 5, 6, 7, 8]
        assert torch.equal(paged[:, rest], old[:, rest])


def test_a_rounds_lengths_follow_the_references_known_answers():
    from oracle import pool
    # tests/test_rounds.py:66-72: bound at 20, a round emits 3 up to frontier 23
    lengths, start, moved = torch.tensor([20, 0]), torch.tensor([20, 0]), torch.tensor([1, 1])
    pool.commit_round(lengths, start, torch.tensor([3]), torch.tensor([23]))
    assert lengths.tolist() == [23, 0]
    # tests/test_rounds.py:113-133: b held (it emitted nothing) keeps what the round found, its frontier stale or not; a
    # truncation commits again from the round's start; a keep between rounds stands
    lengths, start, moved = torch.tensor([20, 30, 7]), torch.tensor([-1, -1, -1]), torch.tensor([1, 1, 1])
    pool.start_round(lengths, start, moved, 2)
    assert start.tolist() == [20, 30, -1] and moved.tolist() == [0, 0, 1]
    pool.commit_round(lengths, start, torch.tensor([3, 0]), torch.tensor([23, 30]))
    assert lengths.tolist() == [23, 30, 7]
    pool.commit_round(lengths, start, torch.tensor([2, 0]), torch.tensor([22, 30]))
    assert lengths.tolist() == [22, 30, 7]
    lengths[1] = 27                                            # keep("b", 27) on the host
    pool.start_round(lengths, start, moved, 2)
    pool.commit_round(lengths, start, torch.tensor([2, 0]), torch.tensor([24, 31]))
    assert lengths.tolist() == [24, 27, 7]


def test_a_steps_buffers_are_the_ones_worked_out_by_hand():
    from oracle import pool
    page, dump, window, table_pages = 4, 9, 3, 5
    tables = {"a": [6, 2, 5], "b": [1], "c": [7, 0, 3, 8]}
    rows = [("a", 9, 2), ("c", 3, 5), ("b", 2, 1), ("a", 4, 3)]      # (sequence, first position, count); c is a prompt row
    starts, positions, row_of = pool.step_batch(rows)
    assert starts == [0, 2, 7, 8, 11]
    assert positions == [9, 10, 3, 4, 5, 6, 7, 2, 4, 5, 6]
    assert row_of == [0, 0, 1, 1, 1, 1, 1, 2, 3, 3, 3]
    slots, d_starts, d_counts, d_firsts, d_offsets, d_tables = pool.step_buffers(tables, rows, page, dump, window, table_pages)
    #            a@9  a@10  c@3   c@4  c@5  c@6  c@7  b@2  a@4  a@5  a@6
    assert slots == [21, 22, 31, 0, 1, 2, 3, 6, 8, 9, 10]
    assert (d_starts, d_counts, d_firsts, d_offsets) == ([0, 7, 8], [2, 1, 3], [9, 2, 4], [0, 2, 3])
    assert d_tables == [[6, 2, 5, 9, 9], [1, 9, 9, 9, 9], [6, 2, 5, 9, 9]]
    # the same slots through the round tables' closed form, where the sequences are bound to round slots
    round_tables = torch.tensor([t + [dump] * (table_pages - len(t)) for t in tables.values()], dtype=torch.int32)
    capacity = torch.tensor([len(t) * page for t in tables.values()])
    slot_of = {"a": 0, "b": 1, "c": 2}
    at = pool.slots_at(round_tables, capacity, torch.tensor([slot_of[rows[r][0]] for r in row_of]), torch.tensor(positions), page, dump)
    assert at.tolist() == slots
    # offsets are the window rows' running token count, starts every row's
    assert d_offsets == [sum(d_counts[:i]) for i in range(len(d_counts))]


# -- rows read back ------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("kind", ["bf16", "fp16", "fp8", "fp8:row", "int8"])
def test_rows_read_back_are_the_codes_times_their_scale_one_fp32_product(kind):
    # Pins rows_at() and gather(): each element against the closed-form decoder (e4m3.decode: every code's value from
    # its bit fields) or the integer code, times the scale as one IEEE FP32 product (numpy float32, no torch); gather of
    # a sequence's first positions is rows_at of the slots its table gives (the slot closed form), in the compute dtype.
    g = torch.Generator().manual_seed(21)
    pages, page, hkv, d = 9, 4, 2, 8
    slots_n = pages * page
    ks = vs = None
    if kind in ("bf16", "fp16"):
        k = torch.randn(pages, page, hkv, d, generator=g).to(append.STORAGE[kind])
        v = torch.randn(pages, page, hkv, d, generator=g).to(append.STORAGE[kind])
    else:
        raw = lambda: torch.randint(0, 256, (pages, page, hkv, d), generator=g, dtype=torch.uint8)
        k, v = raw(), raw()
        k[k == 0x7f], k[k == 0xff], v[v == 0x7f], v[v == 0xff] = 0, 0, 0, 0      # (E4M3's NaN codes aside)
        k, v = k.view(append.STORAGE[kind]), v.view(append.STORAGE[kind])
    if kind in append.ROW_SCALED:
        ks, vs = torch.rand(pages, page, hkv, generator=g) + 0.01, torch.rand(pages, page, hkv, generator=g) + 0.01
    mult = (0.37, 1.9)
    slots = torch.tensor([[5, 0, 35], [17, 17, 8]])
    got_k, got_v = attend.rows_at(k, v, slots, kind, ks, vs, mult)
    assert got_k.shape == (2, 3, hkv, d) and got_k.dtype == torch.float32
    for store, scales, m, got in ((k, ks, mult[0], got_k), (v, vs, mult[1], got_v)):
        flat = store.reshape(slots_n, hkv, d)
        for a, row in enumerate(slots.tolist()):
            for b, s in enumerate(row):
                for h in range(hkv):
                    if kind in ("bf16", "fp16"):
                        want = flat[s, h].float().numpy()
                    else:
                        codes = flat[s, h].view(torch.uint8).numpy()
                        real = e4m3.decode(codes).astype(np.float32) if kind != "int8" else codes.view(np.int8).astype(np.float32)
                        scale = np.float32(m) if kind == "fp8" else scales.reshape(slots_n, hkv)[s, h].numpy()
                        want = real * scale
                    assert np.array_equal(got[a, b, h].numpy(), want), (kind, s, h)
    table = torch.tensor([7, 2, 8, 0])
    for compute in (torch.bfloat16, torch.float32):
        gk, gv = attend.gather(k, v, table, 13, page, kind, compute, ks, vs, mult)
        rk, rv = attend.rows_at(k, v, append.slots(table, torch.arange(13), page), kind, ks, vs, mult)
        assert gk.dtype == compute and torch.equal(gk, rk.to(compute)) and torch.equal(gv, rv.to(compute))


# -- rotary embedding before the append -----------------------------------------------------------------------------------
@pytest.mark.parametrize("style", ["half", "interleaved"])
def test_rope_turns_each_pair_by_its_positions_angle(style):
    # Pins append.rope(): against the rotation as complex numbers in float64 ((a + ib) e^{i theta}, to FP32 rounding),
    # against a scalar loop in numpy float32 with the same separate roundings (bit for bit), by what a rotation
    # preserves (each pair's norm), by the angle sum (turning by p then by r equals turning by p + r, to rounding), and
    # at position 0 (the identity); positions outside the table read its first and last rows.
    g = torch.Generator().manual_seed(41)
    T, H, D, P = 7, 3, 16, 50
    half = D // 2
    freqs = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))
    angle = torch.arange(P, dtype=torch.float64)[:, None] * freqs[None, :]
    table = torch.cat([angle.cos(), angle.sin()], 1).float()
    x = torch.randn(T, H, D, generator=g)
    positions = torch.tensor([0, 3, 49, 17, 5, 60, -2])
    got = append.rope(x, positions, table, style)
    at = positions.clamp(0, P - 1)
    pair = (lambda t: (t[..., :half], t[..., half:])) if style == "half" else (lambda t: (t[..., 0::2], t[..., 1::2]))
    a, b = pair(x.double())
    turned = torch.complex(a, b) * torch.polar(torch.ones(T, 1, half, dtype=torch.float64), angle[at][:, None, :])
    ga, gb = pair(got.double())
    torch.testing.assert_close(ga, turned.real, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(gb, turned.imag, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(ga ** 2 + gb ** 2, a ** 2 + b ** 2, atol=1e-5, rtol=1e-5)
    assert torch.equal(got[0], x[0]) and torch.equal(got[6], x[6])      # position 0 (and -2, clamped to it)
    xn, tn = x.numpy(), table.numpy()
    for t in range(T):
        for h in range(H):
            for j in range(half):
                ia, ib = (j, j + half) if style == "half" else (2 * j, 2 * j + 1)
                c, s = tn[int(at[t]), j], tn[int(at[t]), half + j]
                wa = np.float32(np.float32(xn[t, h, ia] * c) - np.float32(xn[t, h, ib] * s))
                wb = np.float32(np.float32(xn[t, h, ib] * c) + np.float32(xn[t, h, ia] * s))
                assert got[t, h, ia].item() == wa and got[t, h, ib].item() == wb
    twice = append.rope(append.rope(x, torch.full((T,), 11), table, style), torch.full((T,), 6), table, style)
    torch.testing.assert_close(twice, append.rope(x, torch.full((T,), 17), table, style), atol=2e-6, rtol=1e-5)
    # scale multiplies cos and sin first; 16-bit inputs come back in their dtype, rounded once
    scaled = append.rope(x, positions, table, style, scale=0.5)
    torch.testing.assert_close(scaled, got * 0.5, atol=1e-6, rtol=1e-6)
    low = append.rope(x.bfloat16(), positions, table, style)
    assert low.dtype == torch.bfloat16 and torch.equal(low, append.rope(x.bfloat16().float(), positions, table, style).bfloat16())


@pytest.mark.parametrize("style", ["half", "interleaved"])
def test_rms_norm_rope_normalises_weighs_and_turns(style):
    # Pins append.rms_norm_rope(): against the closed form in float64 (x / sqrt(mean(x^2) + eps) * (w + offset), then
    # the rotation as complex numbers) to FP32 rounding; against a scalar loop in numpy float32 taking the sum of
    # squares in the stated order (bit for bit); against torch's own rms_norm followed by the rotation (the reference's
    # text, torch_norms.py:60-68, 149-176: its summation order is the library's, so a few outputs may round the other
    # way); by what the norm fixes (mean square 1 before the weight when eps = 0; c x normalises to what x does for a
    # power of two c, bit for bit); and at position 0 with weight 1 it is the plain norm.
    g = torch.Generator().manual_seed(43)
    T, H, D, P = 6, 3, 64, 40
    half = D // 2
    freqs = 1.0 / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))
    angle = torch.arange(P, dtype=torch.float64)[:, None] * freqs[None, :]
    table = torch.cat([angle.cos(), angle.sin()], 1).float()
    x = torch.randn(T, H, D, generator=g) * 3
    weight = torch.randn(D, generator=g) * 0.2 + 1
    positions = torch.tensor([0, 3, 39, 17, 5, 44])
    eps, offset = 1e-6, 0.5
    got = append.rms_norm_rope(x, weight, eps, positions, table, offset, style)
    at = positions.clamp(0, P - 1)
    xd = x.double()
    normed = xd / (xd.pow(2).mean(-1, keepdim=True) + eps).sqrt() * (weight.double() + offset)
    pair = (lambda t: (t[..., :half], t[..., half:])) if style == "half" else (lambda t: (t[..., 0::2], t[..., 1::2]))
    a, b = pair(normed)
    turned = torch.complex(a, b) * torch.polar(torch.ones(T, 1, half, dtype=torch.float64), angle[at][:, None, :])
    ga, gb = pair(got.double())
    torch.testing.assert_close(ga, turned.real, atol=5e-6, rtol=5e-6)
    torch.testing.assert_close(gb, turned.imag, atol=5e-6, rtol=5e-6)
    # the scalar loop, the same order of every operation
    xn, wn, tn = x.numpy(), weight.numpy(), table.numpy()
    for t in range(T):
        for h in range(H):
            groups = []
            for g8 in range(D // 8):
                s8 = np.float32(xn[t, h, 8 * g8] * xn[t, h, 8 * g8])
                for j in range(1, 8):
                    s8 = np.float32(s8 + np.float32(xn[t, h, 8 * g8 + j] * xn[t, h, 8 * g8 + j]))
                groups.append(s8)
            while len(groups) > 1:
                groups = [np.float32(groups[i] + groups[i + 1]) for i in range(0, len(groups), 2)]
            r = np.float32(np.float32(1.0) / np.sqrt(np.float32(np.float32(groups[0] / np.float32(D)) + np.float32(eps))))
            n = [np.float32(np.float32(xn[t, h, i] * r) * np.float32(wn[i] + np.float32(offset))) for i in range(D)]
            for j in range(half):
                ia, ib = (j, j + half) if style == "half" else (2 * j, 2 * j + 1)
                c, s = tn[int(at[t]), j], tn[int(at[t]), half + j]
                assert np.float32(np.float32(n[ia] * c) - np.float32(n[ib] * s)) == got[t, h, ia].item(), (t, h, j)
                assert np.float32(np.float32(n[ib] * c) + np.float32(n[ia] * s)) == got[t, h, ib].item(), (t, h, j)
    # torch's own norm (another summation order) then the oracle's rotation: equal but for the last place of a few
    theirs = torch.nn.functional.rms_norm(x.float(), (D,), eps=eps) * (weight.float() + offset)
    theirs = append.rope(theirs, positions, table, style)
    torch.testing.assert_close(got, theirs, atol=1e-6, rtol=1e-6)
    # invariants
    plain = append.rms_norm_rope(x, torch.ones(D), 0.0, torch.zeros(T, dtype=torch.int64), table, 0.0, style)
    torch.testing.assert_close(plain.double().pow(2).mean(-1), torch.ones(T, H, dtype=torch.float64), atol=1e-6, rtol=1e-6)
    assert torch.equal(append.rms_norm_rope(4 * x, weight, 0.0, positions, table, offset, style),
                       append.rms_norm_rope(x, weight, 0.0, positions, table, offset, style))
    # 16-bit inputs come back in their dtype, rounded once
    xb = x.bfloat16()
    gb16 = append.rms_norm_rope(xb, weight, eps, positions, table, offset, style)
    assert gb16.dtype == torch.bfloat16
    assert torch.equal(gb16, append.rms_norm_rope(xb.float(), weight, eps, positions, table, offset, style).bfloat16())


# -- sparse index selection ---------------------------------------------------------------------------------------------
def test_sparse_scores_are_the_sum_written_out_term_by_term():
    from oracle import indexer
    rng = np.random.default_rng(5)
    t, h, d, n = 3, 4, 5, 7
    q, keys, w = rng.standard_normal((t, h, d)), rng.standard_normal((n, d)), rng.standard_normal((t, h))
    ends = np.array([7, 3, 0])
    got = indexer.sparse_scores(q, keys, w, ends, 0.37)
    for i in range(t):
        for s in range(n):
            if s >= ends[i]:
                assert got[i, s] == -math.inf
                continue
            total = 0.0
            for j in range(h):
                dot = sum(float(q[i, j, c]) * float(keys[s, c]) for c in range(d))
                total += float(w[i, j]) * 0.37 * max(0.0, dot)
            assert abs(got[i, s] - total) <= 1e-12 * max(1.0, abs(total))


def test_sparse_scores_closed_forms_one_hot_queries_relus_sign_and_linear_weights():
    from oracle import indexer
    rng = np.random.default_rng(6)
    keys = rng.standard_normal((9, 4))
    q = np.zeros((1, 2, 4))
    q[0, 0, 1], q[0, 1, 3] = 1.0, -1.0      # head 0 reads component 1, head 1 minus component 3
    w = np.array([[2.0, 3.0]])
    got = indexer.sparse_scores(q, keys, w, [9], 0.5)[0]
    want = 2.0 * 0.5 * np.maximum(keys[:, 1], 0.0) + 3.0 * 0.5 * np.maximum(-keys[:, 3], 0.0)
    assert np.allclose(got, want, rtol=0, atol=1e-15)
    # a transposed operand or a ReLU after the head sum would fail these: heads that cancel before the ReLU do not after
    q2 = np.stack([np.ones((1, 4)), -np.ones((1, 4))], 1)      # two opposite heads
    both = indexer.sparse_scores(q2, keys, np.ones((1, 2)), [9], 1.0)[0]
    assert np.allclose(both, np.abs(keys.sum(1)), atol=1e-14)
    a, b = rng.standard_normal((1, 2)), rng.standard_normal((1, 2))
    qq = rng.standard_normal((1, 2, 4))
    lin = indexer.sparse_scores(qq, keys, 2 * a - 3 * b, [9], 0.25)
    assert np.allclose(lin, 2 * indexer.sparse_scores(qq, keys, a, [9], 0.25) - 3 * indexer.sparse_scores(qq, keys, b, [9], 0.25))


def _select_by_taking_the_best(row, end, k):
    """The rule without a sort: k times, the best remaining score (a number beats a NaN, the larger number wins, the
    lower position on a tie)."""
    left = list(range(end))
    if end <= k:
        return left
    taken = []
    for _ in range(k):
        best = None
        for at in left:
            x = row[at]
            if best is None:
                best = at
                continue
            y = row[best]
            if (y != y and x == x) or (x == x and y == y and x > y):
                best = at
        taken.append(best)
        left.remove(best)
    return sorted(taken)


def test_sparse_index_takes_the_best_remaining_score_k_times_and_holds_the_references_known_answers():
    from oracle import indexer
    nan, inf = float("nan"), float("inf")
    s = np.array([[1.0, nan, -inf, 2.0, nan]])
    assert indexer.sparse_index(s, [5], 4).tolist() == [[0, 1, 2, 3]]      # 2, 1, -inf, then the first NaN
    assert indexer.sparse_index(s, [5], 3).tolist() == [[0, 2, 3]]
    assert indexer.sparse_index(s, [2], 4).tolist() == [[0, 1, -1, -1]]    # fewer valid keys than k: all of them
    assert indexer.sparse_index(s, [0], 2).tolist() == [[-1, -1]]
    assert indexer.sparse_index(np.array([[0.0, -0.0, 0.0, -0.0]]), [4], 2).tolist() == [[0, 1]]      # the zeros tie
    rng = np.random.default_rng(8)
    for case in range(40):
        n, k = int(rng.integers(1, 40)), int(rng.integers(1, 12))
        row = np.round(rng.standard_normal(n) * 2) / 2      # many ties
        row[rng.integers(0, n, n // 5)] = nan
        row[rng.integers(0, n, n // 7)] = -inf
        row[rng.integers(0, n, n // 9)] = -0.0
        end = int(rng.integers(0, n + 1))
        got = indexer.sparse_index(row[None], [end], k)[0]
        want = _select_by_taking_the_best(row, end, k)
        assert got[:len(want)].tolist() == want and (got[len(want):] == -1).all(), case
