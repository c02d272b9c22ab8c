"""crit_pkv_attend_static, the entry point that allocates nothing (its partials and launch counters live in a static
device array of the library): the same bits as crit_pkv_attend on two calls in a row, the second on a smaller input,
for a split launch, a fused one and 8-bit pages; a launch whose partials exceed the array is refused with a clear
error. Collected last: it runs alone in a fresh process and after every other test alike."""
import ctypes

import pytest
import torch

from crit_amd.paged_kv_attention import _abi
from tests.support import Cache, kernels, rand_q

pytestmark = pytest.mark.gpu
dev = "cuda"


def _both(cache, q, rows, firsts, columns, counts=None, **kw):
    """(crit_pkv_attend's out and lse, crit_pkv_attend_static's) for one launch, outputs preallocated."""
    T, hq = q.shape[0], q.shape[1]
    r = torch.tensor(rows, dtype=torch.int32, device=dev)
    starts = torch.arange(0, columns * len(rows), columns, dtype=torch.int32, device=dev)
    f = torch.tensor(firsts, dtype=torch.int64, device=dev)
    c = None if counts is None else torch.tensor(counts, dtype=torch.int32, device=dev)
    found = []
    for static in (False, True):
        out = torch.full((T, hq, cache.dv), 3.0, dtype=torch.bfloat16, device=dev)
        lse = torch.full((T, hq), 5.0, device=dev)
        cache.attend(q, r, starts, f, columns, counts=c, out=out, lse=lse, static=static, **kw)
        found.append((out, lse))
    torch.cuda.synchronize()
    return found


@pytest.mark.parametrize("kind", ["bf16", "fp8:row"])
def test_two_calls_in_a_row_the_second_smaller_give_the_allocating_entry_points_bits(kind):
    lengths = [3000, 1700, 129, 2500, 4097, 64]
    cache = Cache(kind, 4, 128, 128, 16, lengths, seed=61)
    q = rand_q(12, 16, 128, 62)
    # first call: six rows of two columns; second call: two rows of one column (fewer partials, fewer units)
    for rows, cols, tokens in (([0, 1, 2, 3, 4, 5], 2, 12), ([4, 2], 1, 2)):
        firsts = [lengths[s] - cols for s in rows]
        (out, lse), (out_s, lse_s) = _both(cache, q[:tokens], rows, firsts, cols)
        assert torch.equal(out_s, out) and torch.equal(lse_s, lse), (kind, rows)
        want, want_lse = cache.want(q[:cols], rows[0], firsts[0], cols)
        torch.testing.assert_close(out_s[:cols].double().cpu(), want, atol=8e-3, rtol=2e-2)
        torch.testing.assert_close(lse_s[:cols].double().cpu(), want_lse, atol=1e-3, rtol=1e-4)
    # a fused launch (the counters only), then a ragged one with counts
    (out, lse), (out_s, lse_s) = _both(cache, q[:6], [0, 3, 4], [2990, 2490, 4090], 2, fused=True)
    assert torch.equal(out_s, out) and torch.equal(lse_s, lse)
    (out, lse), (out_s, lse_s) = _both(cache, q[:8], [5, 1], [60, 1690], 4, counts=[3, 4])
    assert torch.equal(out_s, out) and torch.equal(lse_s, lse)


def test_the_generic_kernel_and_other_widths_through_the_static_scratch():
    cache = Cache("int8", 2, 64, 128, 16, [700, 90], seed=63)
    q = rand_q(4, 8, 64, 64)
    (out, lse), (out_s, lse_s) = _both(cache, q, [0, 1], [698, 88], 2)
    assert torch.equal(out_s, out) and torch.equal(lse_s, lse)
    (out, lse), (out_s, lse_s) = _both(cache, q[:1], [1], [89], 1)
    assert torch.equal(out_s, out) and torch.equal(lse_s, lse)


def test_a_launch_past_the_static_scratch_is_refused_and_nothing_runs():
    pk = kernels()
    cache = Cache("bf16", 8, 128, 128, 16, [300] * 40, seed=65)
    q = rand_q(40, 32, 128, 66)
    rows = torch.arange(40, dtype=torch.int32, device=dev)
    firsts = torch.full((40,), 299, dtype=torch.int64, device=dev)
    parts = pk.partitions(dev, 8, "bf16")
    assert 256 + 40 * 32 * parts * 130 * 4 > _abi.STATIC_SCRATCH_BYTES
    out = torch.full((40, 32, 128), 3.0, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError, match="static scratch"):
        cache.attend(q, rows, rows, firsts, 1, out=out, static=True)
    torch.cuda.synchronize()
    assert bool((out == 3.0).all())
    # the same rows fused need the counters only
    got = cache.attend(q, rows, rows, firsts, 1, out=out, static=True, fused=True)
    assert torch.equal(got, cache.attend(q, rows, rows, firsts, 1, fused=True))
    assert _abi.load().crit_pkv_attend_static(ctypes.byref(_abi.AttendParams()), None) == -1
