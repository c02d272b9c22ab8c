"""Rows read back on the GPU (a sequence's first positions, rows at arbitrary slots) against the CPU oracle's restatement
of KVPool.gather and KVPool.rows_at (inference/attention-state/code/pages.py:455-493), bit for bit. Mirrors the
reference's inference/attention-state/tests/test_rounds.py:262-273 (rows_at in FP32, gather in the compute dtype)."""
import pytest
import torch

from oracle import append as oracle_append
from oracle import attend as oracle_attend
from tests.support import KINDS, STORE, bits, kernels

pytestmark = pytest.mark.gpu
dev = "cuda"


def _pool(kind, pages, page, hkv, d, dv, seed):
    g = torch.Generator().manual_seed(seed)
    ks = vs = None
    if kind in ("bf16", "fp16"):
        k = (torch.randn(pages, page, hkv, d, generator=g) * 3).to(STORE[kind])
        v = (torch.randn(pages, page, hkv, dv, generator=g) * 3).to(STORE[kind])
    else:
        k = torch.randint(0, 256, (pages, page, hkv, d), generator=g, dtype=torch.uint8).view(STORE[kind])
        v = torch.randint(0, 256, (pages, page, hkv, dv), generator=g, dtype=torch.uint8).view(STORE[kind])
    if kind in ("fp8:row", "int8"):
        ks, vs = torch.rand(pages, page, hkv, generator=g) * 2, torch.rand(pages, page, hkv, generator=g) * 2
    return k, v, ks, vs


def _equal(got, want, what):
    got, want = got.cpu(), want
    assert got.dtype == want.dtype and got.shape == want.shape, what
    nan = torch.isnan(want.float())
    assert torch.equal(torch.isnan(got.float()), nan), what       # (E4M3's NaN codes read back as NaN)
    assert torch.equal(bits(got)[~nan], bits(want)[~nan]), what


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hkv,d,dv", [(2, 128, 128), (8, 64, 128), (3, 24, 8)])
def test_rows_at_slots_and_a_sequences_first_positions_read_back_as_torch_does(kind, hkv, d, dv):
    pk = kernels()
    pages, page = 40, 16
    k, v, ks, vs = _pool(kind, pages, page, hkv, d, dv, 31)
    mult = (0.043, 1.7)
    on = lambda t: None if t is None else t.to(dev)
    g = torch.Generator().manual_seed(32)
    slots = torch.randint(0, pages * page, (7, 33), generator=g)
    want_k, want_v = oracle_attend.rows_at(k, v, slots, kind, ks, vs, mult)
    got_k, got_v = pk.rows_at(on(k), on(v), kind, slots.to(dev), key_scales=on(ks), value_scales=on(vs), multipliers=mult)
    _equal(got_k, want_k, "keys at slots")
    _equal(got_v, want_v, "values at slots")
    table = torch.randperm(pages, generator=g)[:20]
    for compute in (torch.bfloat16, torch.float16, torch.float32):
        for count, tab in ((307, table.to(torch.int32)), (1, table), (320, table)):
            want_k, want_v = oracle_attend.gather(k, v, table, count, page, kind, compute, ks, vs, mult)
            got_k, got_v = pk.gather(on(k), on(v), kind, tab.to(dev), count, page, key_scales=on(ks), value_scales=on(vs),
                                     multipliers=mult, dtype=compute)
            _equal(got_k, want_k, f"gathered keys {compute} {count}")
            _equal(got_v, want_v, f"gathered values {compute} {count}")
    # keys only (a pool without values), into a buffer given, a negative slot and one past the pages as zeros
    out = (torch.full((5, hkv, d), 9.0, device=dev), None)
    some = torch.tensor([3, -1, 0, 639, 640])      # (640: the first slot past the pages)
    pk.rows_at(on(k), None, kind, some.to(dev), key_scales=on(ks), multipliers=mult, out=out)
    want_k, _ = oracle_attend.rows_at(k, v, some.clamp(0, 639), kind, ks, vs, mult)
    want_k[1], want_k[4] = 0, 0
    _equal(out[0], want_k, "keys only")


@pytest.mark.parametrize("kind,dtype", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_sixteen_bit_pages_read_back_in_their_own_type_keep_every_bit(kind, dtype):
    # KVPool.gather's rows.to(compute) of the pages' own dtype is the tensor itself (pages.py:455-477): every one of
    # the 65,536 bit patterns comes back as it is stored, a NaN with its payload and sign; read back as FP32 (rows_at)
    # every number is exact and a NaN is a NaN.
    pk = kernels()
    patterns = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    k = patterns.reshape(16, 16, 2, 128)
    v = patterns.flip(0).reshape(16, 16, 2, 128)
    table = torch.randperm(16, generator=torch.Generator().manual_seed(2)).to(torch.int32)
    gk, gv = pk.gather(k.to(dev), v.to(dev), kind, table.to(dev), 250, 16, dtype=dtype)
    want_k, want_v = oracle_attend.gather(k, v, table, 250, 16, kind, dtype)
    assert torch.equal(gk.cpu().view(torch.int16), want_k.view(torch.int16))
    assert torch.equal(gv.cpu().view(torch.int16), want_v.view(torch.int16))
    slots = torch.arange(256)
    rk, _ = pk.rows_at(k.to(dev), v.to(dev), kind, slots.to(dev))
    want = k.reshape(256, 2, 128).float()
    numbers = ~torch.isnan(want)
    assert torch.equal(torch.isnan(rk.cpu()), ~numbers) and torch.equal(rk.cpu()[numbers], want[numbers])


def test_per_head_multipliers_and_what_is_refused():
    pk = kernels()
    k, v, _, _ = _pool("fp8", 8, 16, 4, 128, 128, 33)
    heads = torch.tensor([[0.5, 0.25, 2.0, 1.5], [1.0, 3.0, 0.125, 0.7]])
    slots = torch.arange(0, 128, 3)
    got_k, got_v = pk.rows_at(k.to(dev), v.to(dev), "fp8", slots.to(dev), multipliers=heads.to(dev))
    for h in range(4):
        want_k, want_v = oracle_attend.rows_at(k, v, slots, "fp8", multipliers=(float(heads[0, h]), float(heads[1, h])))
        _equal(got_k[:, h], want_k[:, h].contiguous(), f"head {h}")
        _equal(got_v[:, h], want_v[:, h].contiguous(), f"head {h}")
    with pytest.raises(ValueError):
        pk.rows_at(k.to(dev), v.to(dev), "fp8", slots.to(torch.int32).to(dev))
    with pytest.raises(ValueError):
        pk.gather(k.to(dev), v.to(dev), "fp8", torch.arange(2, dtype=torch.int32, device=dev), 33, 16)
    with pytest.raises(ValueError):
        pk.rows_at(k.to(dev), v.to(dev), "fp8", slots.to(dev), dtype=torch.float64)
    with pytest.raises(ValueError):
        pk.rows_at(k.to(dev), v.to(dev), "int8", slots.to(dev))
