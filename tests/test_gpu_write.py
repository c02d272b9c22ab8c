"""KV append on the GPU against the CPU oracle: every stored byte (and row scale) equal, skipped slots untouched.
Mirrors the reference's kernels/techniques/attention/paged-kv-attention/tests/test_paged_kv_attention.py:88-126,
482-498. Calls go through the kernels module, which reaches the HIP kernels through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import append as oracle_append
from oracle import e4m3
from tests.support import KINDS, STORE, bits, expected_pages, kernels

pytestmark = pytest.mark.gpu
dev = "cuda"


def _check(kind, got, want):
    for name, g, w in zip(("keys", "values", "key scales", "value scales"), got, want):
        if w is None:
            continue
        assert torch.equal(bits(g.cpu()).reshape(-1), bits(w).reshape(-1)), (kind, name)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("d,dv", [(128, 128), (64, 128), (256, 256)])
@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
def test_writes_encode_as_torch_does_and_skip_negative_slots(kind, d, dv, in_dtype):
    pk = kernels()
    g = torch.Generator().manual_seed(1)
    keys = (torch.randn(40, 3, d, generator=g) * 3).to(in_dtype)
    values = torch.randn(40, 3, dv, generator=g).to(in_dtype)
    keys[5] = 0.0
    k = torch.zeros(64, 3, d, dtype=STORE[kind], device=dev)
    v = torch.zeros(64, 3, dv, dtype=STORE[kind], device=dev)
    ks = vs = None
    if kind in ("fp8:row", "int8"):
        ks, vs = torch.zeros(64, 3, device=dev), torch.zeros(64, 3, device=dev)
    slots = torch.randperm(64, generator=g)[:40]
    slots[7] = -1
    mult = (0.05, 0.07)
    pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs, multipliers=mult)
    _check(kind, (k, v, ks, vs), expected_pages(kind, keys, values, slots, 64, mult))


@pytest.mark.parametrize("kind,dtype", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
@pytest.mark.parametrize("d", [128, 20])
def test_sixteen_bit_rows_into_pages_of_their_own_type_keep_every_bit(kind, dtype, d):
    # The reference's write() stores keys.to(the pages' dtype) (pages.py:439-453): for inputs of the pages' own type that
    # is the tensor itself, so every bit pattern arrives as it is, a NaN with its payload and sign (a cast from FP32
    # stores the canonical NaN instead: the oracle's rule, checked beside it). d = 20: the scalar kernel.
    pk = kernels()
    patterns = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    rows = 65536 // (4 * d) * 4
    x = patterns[:rows * d].reshape(rows // 4, 4, d)
    k = torch.zeros(rows // 4, 4, d, dtype=dtype, device=dev)
    v = torch.zeros_like(k)
    slots = torch.randperm(rows // 4, generator=torch.Generator().manual_seed(3))
    pk.write(x.to(dev), x.flip(0).to(dev), slots.to(dev), k, v, kind)
    assert torch.equal(k.cpu().view(torch.int16)[slots], x.view(torch.int16))
    assert torch.equal(v.cpu().view(torch.int16)[slots], x.flip(0).view(torch.int16))
    # The same values as FP32 inputs go through torch's cast. What it stores for a NaN follows the host (its vectorised
    # BF16 conversion stores 0xFFFF, its scalar one 0x7FC0; FP16 keeps the payload): every other value bit for bit, a
    # NaN as a NaN, and as the oracle's where this host casts the way the kernels do.
    wide = x.float()
    pk.write(wide.to(dev), wide.to(dev), slots.to(dev), k, v, kind)
    want = expected_pages(kind, wide, wide, slots, rows // 4, (1.0, 1.0))[0]
    got = k.cpu()
    numbers = ~torch.isnan(want.float())
    assert torch.equal(torch.isnan(got.float()), ~numbers)
    assert torch.equal(got.view(torch.int16)[numbers], want.view(torch.int16)[numbers])
    host_nan = torch.tensor([float("nan")] * 16).to(dtype).view(torch.int16)[0].item() & 0xffff
    if dtype == torch.float16 or host_nan == 0xffff:
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("d", [128, 24])
def test_every_sixteen_bit_pattern_is_encoded_as_the_oracle_encodes_it(kind, in_dtype, d):
    # Every BF16 / FP16 bit pattern as an input (FP32 inputs: every BF16 pattern widened, and with low bits set on either
    # side of the rounding ties), into every page kind, vector kernel (d = 128) and scalar one (d = 24): every number's
    # stored bits and every row scale equal the oracle's; a NaN is stored as a NaN (whose bits, where a cast makes them,
    # are its conversion instruction's: the test of the pages' own type above has the cases that are pinned).
    pk = kernels()
    patterns = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    if in_dtype == torch.float32:
        wide = patterns.view(torch.bfloat16).float().view(torch.int32)
        x = torch.cat([wide, wide | 0x8000, wide | 0x7fff, wide | 0x8001, wide | 0x0001]).view(torch.float32)
    else:
        x = patterns.view(in_dtype)
    x = x[:x.numel() // (4 * d) * 4 * d].reshape(-1, 4, d)
    T = x.shape[0]
    k = torch.zeros(T, 4, d, dtype=STORE[kind], device=dev)
    v = torch.zeros_like(k)
    ks = vs = None
    if kind in ("fp8:row", "int8"):
        ks, vs = torch.zeros(T, 4, device=dev), torch.zeros(T, 4, device=dev)
    slots = torch.randperm(T, generator=torch.Generator().manual_seed(3))
    mult = (0.05, 0.07)
    pk.write(x.to(dev), x.flip(0).to(dev), slots.to(dev), k, v, kind, ks, vs, multipliers=mult)
    want = expected_pages(kind, x, x.flip(0), slots, T, mult)
    for name, got, exact in zip(("keys", "values", "key scales", "value scales"), (k, v, ks, vs), want):
        if exact is None:
            continue
        got = got.cpu()
        nan = torch.isnan(exact.float())
        assert torch.equal(torch.isnan(got.float()), nan), (name, "which are NaN")
        assert torch.equal(bits(got)[~nan], bits(exact)[~nan]), (name, "the numbers' bits")


@pytest.mark.parametrize("T", [4152, 33001])
@pytest.mark.parametrize("kind", ["bf16", "fp8", "fp8:row", "int8"])
def test_a_large_append_with_edge_values_is_bit_exact(kind, T):
    # 4,152 tokens (the mixed prefill + decode batch's append) and 33,001 (an odd count, so the last workgroup is
    # ragged, over thousands of workgroups), 8 KV heads, with the values that break sloppy encoders: signed zeros, the
    # subnormal ties, saturation, infinities, 1% outliers x20.
    pk = kernels()
    g = torch.Generator().manual_seed(2)
    hkv, d = 8, 128
    keys, values = torch.randn(T, hkv, d, generator=g), torch.randn(T, hkv, d, generator=g)
    hot = torch.rand(T, hkv, d, generator=g) < 0.01
    keys = torch.where(hot, keys * 20, keys)
    mult = (0.04, 0.06)
    edge = torch.tensor([0.0, -0.0, 2.0 ** -10, -(2.0 ** -10), 2.0 ** -9, 448.0, -448.0, 449.0, 1e30, -1e30,
                         float("inf"), float("-inf"), 1e-30, 0.0146484375, 432.0, 248.0])
    keys[0, 0, :16] = edge * mult[0]
    values[1, 2, :16] = edge * mult[1]
    n_slots = 8192 if T < 8192 else 40000
    slots = torch.randperm(n_slots, generator=g)[:T]
    slots[100] = -1
    slots[4000] = -5
    k = torch.zeros(n_slots, hkv, d, dtype=STORE[kind], device=dev)
    v = torch.zeros(n_slots, hkv, d, dtype=STORE[kind], device=dev)
    ks = vs = None
    if kind in ("fp8:row", "int8"):
        ks, vs = torch.zeros(n_slots, hkv, device=dev), torch.zeros(n_slots, hkv, device=dev)
    if kind in ("fp8:row", "int8"):      # an infinite row maximum makes every quotient NaN: keep the rows finite there
        keys = torch.nan_to_num(keys, posinf=3e4, neginf=-3e4)
        values = torch.nan_to_num(values, posinf=3e4, neginf=-3e4)
    pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs, multipliers=mult)
    _check(kind, (k, v, ks, vs), expected_pages(kind, keys, values, slots, n_slots, mult))


def test_fp8_codes_on_every_97th_bit_pattern_equal_torchs_cast_and_the_reference_vectors():
    # The reference's own check of its encoder (kernels/core/tests/test_core_triton.py:68-77), through write().
    pk = kernels()
    top = int(np.float32(448.0).view(np.uint32))
    pos = np.arange(0, top + 1, 97, dtype=np.uint32)
    allbits = np.concatenate([pos, pos | np.uint32(0x80000000)])
    allbits = np.concatenate([allbits, np.zeros((-len(allbits)) % 128, dtype=np.uint32)])
    x = torch.from_numpy(allbits.view(np.float32).copy()).view(-1, 1, 128)
    T = x.shape[0]
    k = torch.zeros(T, 1, 128, dtype=torch.float8_e4m3fn, device=dev)
    pk.write(x.to(dev), None, torch.arange(T, device=dev), k, None, "fp8", multipliers=(1.0, 1.0))
    want = x.clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(k.cpu().view(torch.uint8), want)
    assert np.array_equal(e4m3.encode(x.numpy().reshape(-1)), want.numpy().reshape(-1))


@pytest.mark.parametrize("kind", ["bf16", "fp8:row", "int8"])
def test_key_only_writes_leave_no_values(kind):
    pk = kernels()
    g = torch.Generator().manual_seed(3)
    keys = torch.randn(20, 1, 64, generator=g).to(dev)
    k = torch.zeros(32, 1, 64, dtype=STORE[kind], device=dev)
    ks = torch.zeros(32, 1, device=dev) if kind != "bf16" else None
    slots = torch.arange(20, device=dev) + 5
    pk.write(keys, None, slots, k, None, kind, ks, None)
    both = torch.zeros_like(k)
    other = torch.zeros(32, 1, 64, dtype=STORE[kind], device=dev)
    both_s = torch.zeros(32, 1, device=dev) if ks is not None else None
    pk.write(keys, keys, slots, both, other, kind, both_s, torch.zeros_like(both_s) if ks is not None else None)
    assert torch.equal(bits(k), bits(both))
    if ks is not None:
        assert torch.equal(ks, both_s)
    want = expected_pages(kind, keys.cpu(), keys.cpu(), slots.cpu(), 32, (1.0, 1.0))
    assert torch.equal(bits(k.cpu()), bits(want[0]))


def test_values_only_writes_use_the_value_multiplier():
    pk = kernels()
    g = torch.Generator().manual_seed(4)
    values = torch.randn(9, 2, 128, generator=g)
    v = torch.zeros(16, 2, 128, dtype=torch.float8_e4m3fn, device=dev)
    slots = torch.arange(9)
    pk.write(None, values.to(dev), slots.to(dev), None, v, "fp8", multipliers=(0.5, 0.03))
    want = oracle_append.encode(values, "fp8", 0.03)[0]
    assert torch.equal(v.cpu().view(torch.uint8)[:9], want.view(torch.uint8))


def test_one_multiplier_per_kv_head():
    pk = kernels()
    g = torch.Generator().manual_seed(5)
    keys, values = torch.randn(33, 8, 128, generator=g), torch.randn(33, 8, 128, generator=g)
    mults = torch.rand(2, 8, generator=g) * 0.1 + 0.01
    k = torch.zeros(64, 8, 128, dtype=torch.float8_e4m3fn, device=dev)
    v = torch.zeros_like(k)
    slots = torch.randperm(64, generator=g)[:33]
    pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, "fp8", multipliers=mults.to(dev))
    want = expected_pages("fp8", keys, values, slots, 64, (mults[0], mults[1]))
    _check("fp8", (k, v, None, None), want)


def _codes_between(kind, n, g):
    """n values halfway between two neighbouring codes of the kind (in the codes' own units)."""
    if kind == "int8":
        return torch.randint(-127, 127, (n,), generator=g).double() + 0.5
    c = torch.randint(0, 126, (n,), generator=g).to(torch.uint8)          # 0 .. 448's code - 1
    lo, hi = c.view(torch.float8_e4m3fn).double(), (c + 1).view(torch.float8_e4m3fn).double()
    sign = torch.randint(0, 2, (n,), generator=g).double() * 2 - 1
    return sign * (lo + hi) / 2


def test_fp8_quotients_at_rounding_boundaries_under_awkward_multipliers():
    # Inputs within a few FP32 steps of (a tie between two codes) x (the head's multiplier): any division that is not the
    # correctly rounded one lands on the wrong side of some of them. Multipliers that are no powers of two, negative,
    # and far enough out that the reciprocal is subnormal or the quotient overflows.
    pk = kernels()
    g = torch.Generator().manual_seed(11)
    T, hkv, d = 257, 8, 128
    mults = torch.tensor([[0.03, 1.0 / 3.0, 3.7e-5, -0.7, 1e-35, 1e35, 0.999999, 1234.567],
                          [7e-3, -1.1e-4, 2.5, 1e-37, 0.1, 5e30, 3.0, 0.06]], dtype=torch.float32)
    rows = []
    for which in range(2):
        mid = _codes_between("fp8", T * hkv * d, g).view(T, hkv, d)
        steps = torch.randint(-6, 7, (T, hkv, d), generator=g).double() * 2.0 ** -24
        rows.append((mid * mults[which].double()[None, :, None] * (1 + steps)).float())
    keys, values = rows
    k = torch.zeros(512, hkv, d, dtype=torch.float8_e4m3fn, device=dev)
    v = torch.zeros_like(k)
    slots = torch.randperm(512, generator=g)[:T]
    pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, "fp8", multipliers=mults.to(dev))
    _check("fp8", (k, v, None, None), expected_pages("fp8", keys, values, slots, 512, (mults[0], mults[1])))


@pytest.mark.parametrize("kind", ["fp8:row", "int8"])
def test_row_scaled_quotients_at_rounding_boundaries(kind):
    # Each row holds its maximum once and otherwise values within a few FP32 steps of (a tie between two codes) x (the
    # scale that maximum gives the row).
    pk = kernels()
    g = torch.Generator().manual_seed(12)
    T, hkv, d = 300, 4, 128
    top = 448.0 if kind == "fp8:row" else 127.0
    amax = (torch.rand(T, hkv, generator=g) * 40 + 0.01).float()
    scale = (amax / torch.full_like(amax, top)).clamp(min=1e-30)
    mid = _codes_between("fp8" if kind == "fp8:row" else "int8", T * hkv * d, g).view(T, hkv, d)
    steps = torch.randint(-6, 7, (T, hkv, d), generator=g).double() * 2.0 ** -24
    keys = (mid * scale.double()[..., None] * (1 + steps)).float()
    keys = torch.where(keys.abs() >= amax[..., None], keys * 0.5, keys)
    keys[:, :, 5] = amax * (torch.randint(0, 2, (T, hkv), generator=g).float() * 2 - 1)
    values = keys.flip(0).contiguous()
    k = torch.zeros(512, hkv, d, dtype=STORE[kind], device=dev)
    v = torch.zeros_like(k)
    ks, vs = torch.zeros(512, hkv, device=dev), torch.zeros(512, hkv, device=dev)
    slots = torch.randperm(512, generator=g)[:T]
    pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs)
    _check(kind, (k, v, ks, vs), expected_pages(kind, keys, values, slots, 512, (1.0, 1.0)))


def test_odd_widths_and_strided_inputs_take_the_scalar_path():
    pk = kernels()
    g = torch.Generator().manual_seed(6)
    big = torch.randn(12, 2, 3, 80, generator=g)
    keys, values = big[:, :, 0], big[:, :, 2, :40]            # head stride 240, token stride 480; widths 80 and 40
    for kind in ("bf16", "fp8", "int8"):
        k = torch.zeros(16, 2, 80, dtype=STORE[kind], device=dev)
        v = torch.zeros(16, 2, 40, dtype=STORE[kind], device=dev)
        ks = vs = None
        if kind == "int8":
            ks, vs = torch.zeros(16, 2, device=dev), torch.zeros(16, 2, device=dev)
        slots = torch.randperm(16, generator=g)[:12]
        bigd = big.to(dev)
        pk.write(bigd[:, :, 0], bigd[:, :, 2, :40], slots.to(dev), k, v, kind, ks, vs, multipliers=(0.1, 0.2))
        _check(kind, (k, v, ks, vs), expected_pages(kind, keys, values, slots, 16, (0.1, 0.2)))


def test_bad_arguments_are_refused():
    pk = kernels()
    k = torch.zeros(4, 1, 64, dtype=torch.bfloat16, device=dev)
    x = torch.zeros(2, 1, 64, device=dev)
    with pytest.raises(ValueError):
        pk.write(None, None, torch.zeros(2, dtype=torch.int64, device=dev), None, None, "bf16")
    with pytest.raises(ValueError, match="page kind"):
        pk.write(x, None, torch.zeros(2, dtype=torch.int64, device=dev), k, None, "fp4")
    with pytest.raises(ValueError, match="scales"):
        pk.write(x, None, torch.zeros(2, dtype=torch.int64, device=dev), k, None, "int8")
    pk.write(x[:0], None, torch.zeros(0, dtype=torch.int64, device=dev), k, None, "bf16")     # no tokens: nothing


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("d,dv,in_dtype", [(128, 128, torch.bfloat16), (64, 64, torch.float32), (256, 128, torch.bfloat16),
                                           (128, 64, torch.float16), (64, 128, torch.bfloat16)])      # (values wider than keys: two launches)
@pytest.mark.parametrize("style", ["half", "interleaved"])
def test_keys_rotated_on_their_way_in_are_the_bytes_of_rope_then_write(kind, d, dv, in_dtype, style):
    # write(rope=(table, positions, style, scale)): the reference's rope() on the keys (inference/fused-norms/code/
    # torch_norms.py:89-147, what its model plugins run just before the append) fused into the launch: every stored byte
    # and row scale equals the oracle's rope() followed by its write(), the values untouched by the rotation; positions
    # past the table read its last row; a skipped slot stays zero.
    pk = kernels()
    g = torch.Generator().manual_seed(51)
    T, hkv, P = 70, 3, 200
    keys = (torch.randn(T, hkv, d, generator=g) * 2).to(in_dtype)
    values = torch.randn(T, hkv, dv, generator=g).to(in_dtype)
    half = d // 2
    angle = torch.arange(P, dtype=torch.float64)[:, None] / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))[None, :]
    table = torch.cat([angle.cos(), angle.sin()], 1).float()
    positions = torch.randint(0, P, (T,), generator=g)
    positions[:3] = torch.tensor([0, P + 5, -1])
    slots = torch.randperm(96, generator=g)[:T]
    slots[9] = -1
    mult = (0.05, 0.07)
    for scale in (1.0, 0.75):
        k = torch.zeros(96, hkv, d, dtype=STORE[kind], device=dev)
        v = torch.zeros(96, hkv, dv, dtype=STORE[kind], device=dev)
        ks = vs = None
        if kind in ("fp8:row", "int8"):
            ks, vs = torch.zeros(96, hkv, device=dev), torch.zeros(96, hkv, device=dev)
        pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs, multipliers=mult,
                 rope=(table.to(dev), positions.to(dev), style, scale))
        turned = oracle_append.rope(keys, positions, table, style, scale)
        want = expected_pages(kind, turned, values, slots, 96, mult)
        _check(kind, (k, v, ks, vs), want)
    if kind == "bf16":      # keys only; a table or positions that do not fit are refused
        k = torch.zeros(96, hkv, d, dtype=STORE[kind], device=dev)
        pk.write(keys.to(dev), None, slots.to(dev), k, None, kind, rope=(table.to(dev), positions.to(dev), style))
        want = expected_pages(kind, oracle_append.rope(keys, positions, table, style), values, slots, 96, mult)
        assert torch.equal(bits(k.cpu()).reshape(-1), bits(want[0]).reshape(-1))
        with pytest.raises(ValueError):
            pk.write(keys.to(dev), None, slots.to(dev), k, None, kind, rope=(table[:, :half].contiguous().to(dev), positions.to(dev)))
        with pytest.raises(ValueError):
            pk.write(keys.to(dev), None, slots.to(dev), k, None, kind, rope=(table.to(dev), positions[:5].to(dev)))
        with pytest.raises(ValueError):
            pk.write(keys.to(dev), None, slots.to(dev), k, None, kind, rope=(table.to(dev), positions.to(dev), "pairs"))


@pytest.mark.parametrize("kind,d,dv,in_dtype", [("bf16", 128, 128, torch.bfloat16), ("fp8", 128, 128, torch.bfloat16),
                                           ("fp8:row", 128, 128, torch.float32), ("int8", 64, 64, torch.bfloat16),
                                           ("fp16", 256, 256, torch.float16), ("fp8", 256, 128, torch.float32),
                                           ("bf16", 64, 64, torch.float32), ("fp8:row", 64, 256, torch.bfloat16)])
@pytest.mark.parametrize("style", ["half", "interleaved"])
def test_keys_normed_and_rotated_on_their_way_in_are_the_bytes_of_rms_norm_rope_then_write(kind, d, dv, in_dtype, style):
    # write(rope=..., norm=(weight, eps, offset)): the reference's rms_norm_rope() on the keys (inference/fused-norms/
    # code/torch_norms.py:149-176; the keys' half of rms_norm_rope_pair, what model-template runs before the append,
    # blocks.py:160-170) fused into the launch: every stored byte and row scale equals the oracle's rms_norm_rope()
    # followed by its write(); the values are neither normed nor rotated. With and without an offset, with a scale on
    # the rotation, a weight in the keys' dtype.
    pk = kernels()
    g = torch.Generator().manual_seed(53)
    T, hkv, P = 70, 3, 200
    keys = (torch.randn(T, hkv, d, generator=g) * 3).to(in_dtype)
    keys[5] = 0                       # a row of zeros: eps alone under the root
    values = torch.randn(T, hkv, dv, generator=g).to(in_dtype)
    half = d // 2
    angle = torch.arange(P, dtype=torch.float64)[:, None] / (10000.0 ** (torch.arange(half, dtype=torch.float64) / half))[None, :]
    table = torch.cat([angle.cos(), angle.sin()], 1).float()
    positions = torch.randint(0, P, (T,), generator=g)
    slots = torch.randperm(96, generator=g)[:T]
    slots[11] = -1
    mult = (0.05, 0.07)
    weight = torch.randn(d, generator=g) * 0.3 + 1
    for eps, offset, scale, w in ((1e-6, 0.0, 1.0, weight), (1e-5, 1.0, 0.75, (weight - 1).to(in_dtype))):
        k = torch.zeros(96, hkv, d, dtype=STORE[kind], device=dev)
        v = torch.zeros(96, hkv, dv, dtype=STORE[kind], device=dev)
        ks = vs = None
        if kind in ("fp8:row", "int8"):
            ks, vs = torch.zeros(96, hkv, device=dev), torch.zeros(96, hkv, device=dev)
        pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs, multipliers=mult,
                 rope=(table.to(dev), positions.to(dev), style, scale), norm=(w.to(dev), eps, offset))
        turned = oracle_append.rms_norm_rope(keys, w, eps, positions, table, offset, style, scale)
        want = expected_pages(kind, turned, values, slots, 96, mult)
        _check(kind, (k, v, ks, vs), want)
    with pytest.raises(ValueError, match="rope"):
        pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs, norm=(weight.to(dev), 1e-6))
    with pytest.raises(ValueError):
        pk.write(keys.to(dev), values.to(dev), slots.to(dev), k, v, kind, ks, vs,
                 rope=(table.to(dev), positions.to(dev), style), norm=(weight[:8].to(dev), 1e-6))
