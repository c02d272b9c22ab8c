"""Slot math and the append encodings of crit's paged KV pool, on torch-CPU. Test infrastructure only.

A layer's pages are [pages + 1][page][kv_heads][dim]; the last page is the dump page. Position p of a sequence with page
table `table` lives at slot table[p // page] * page + p % page (reference inference/attention-state/code/pages.py:721-722).
"""
import torch

from . import e4m3

STORAGE = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32, "fp8": torch.float8_e4m3fn,
           "fp8:row": torch.float8_e4m3fn, "int8": torch.int8}
ROW_SCALED = ("fp8:row", "int8")


def slot(table, position, page):
    """The slot of one position (pages.py:721-722)."""
    return int(table[position // page]) * page + position % page


def slots(table, positions, page):
    """Slots of many positions: table [pages] integer tensor, positions integer tensor -> int64."""
    positions = torch.as_tensor(positions, dtype=torch.int64)
    return torch.as_tensor(table, dtype=torch.int64)[positions // page] * page + positions % page


def row_scales(x, top):
    """Each row's FP32 scale: its absolute maximum over `top` as an IEEE division (tensor / tensor), at least 1e-30
    (pages.py:872-876)."""
    amax = x.abs().amax(dim=-1)
    return (amax / amax.new_full(amax.shape, top)).clamp(min=1e-30)


def fp8_rows(rows):
    """[tokens][kv_heads][dim] -> (E4M3 codes, FP32 scale per token and head) (pages.py:888-895)."""
    x = rows.float()
    scale = row_scales(x, 448.0)
    return (x / scale[..., None]).clamp(-448, 448).to(torch.float8_e4m3fn), scale


def int8_rows(rows):
    """[tokens][kv_heads][dim] -> (INT8 codes, FP32 scale per token and head), ties to even (pages.py:879-885)."""
    x = rows.float()
    scale = row_scales(x, 127.0)
    return torch.round(x / scale[..., None]).clamp(-127, 127).to(torch.int8), scale


def encode(rows, kind, multiplier=1.0):
    """One tensor of rows [tokens][kv_heads][dim] encoded for a page kind -> (stored tensor, scales or None).

    fp8: (x.float() / multiplier).clamp(-448, 448) cast to E4M3 (pages.py:444). `multiplier` is a float, a 0-d tensor
    (the reference's per-layer scale) or a [kv_heads] tensor (one scale per KV head, broadcast over tokens and dims: a
    superset of the reference rule with the same expression). The division is tensor / tensor, which is IEEE on
    every torch backend."""
    if kind in ("bf16", "fp16", "fp32"):
        # rows.to(storage), the reference's own expression (pages.py:453): rows of the pages' type are stored as they
        # are, every bit (a NaN with its payload); what a cast stores for a NaN is torch's and follows the host (FP32 to
        # BF16: 0xFFFF by its vectorised conversion, 0x7FC0 by its scalar one; to FP16 the payload's top bits)
        return rows.to(STORAGE[kind]), None
    x = rows.float()
    if kind == "fp8":
        m = torch.as_tensor(multiplier, dtype=torch.float32)
        if m.dim() == 1:
            m = m[None, :, None]
        return (x / m.expand_as(x)).clamp(-448, 448).to(torch.float8_e4m3fn), None
    if kind == "fp8:row":
        return fp8_rows(rows)
    if kind == "int8":
        return int8_rows(rows)
    raise ValueError(kind)


def encode_fp8_integer(rows, multiplier=1.0):
    """The fp8 rule with the integer encoder instead of torch's cast: an independent path to the same bytes."""
    x = rows.float()
    m = torch.as_tensor(multiplier, dtype=torch.float32)
    if m.dim() == 1:
        m = m[None, :, None]
    quotient = (x / m.expand_as(x)).numpy()
    return torch.from_numpy(e4m3.encode(quotient))


def _bytes(t):
    return t.view(torch.uint8) if t.dtype == torch.float8_e4m3fn else t


def write(keys, values, slot_ids, key_pages, value_pages, kind, key_scales=None, value_scales=None,
          multipliers=(1.0, 1.0), dump_slot=None):
    """Store keys [T][HKV][D] and values [T][HKV][DV] at slot_ids [T] of one layer's pages (any view of
    [slots][HKV][dim] storage), in place (pages.py:439-453). A slot below 0 goes to `dump_slot` when given (the torch
    path, pages.py:439) and is skipped otherwise (the kernel path, _kernels.py:121). values / value_pages None: keys
    only."""
    slot_ids = torch.as_tensor(slot_ids, dtype=torch.int64)
    if dump_slot is not None:
        slot_ids = torch.where(slot_ids >= 0, slot_ids, torch.full_like(slot_ids, dump_slot))
        keep = torch.ones_like(slot_ids, dtype=torch.bool)
    else:
        keep = slot_ids >= 0
    parts = [(keys, key_pages, key_scales, multipliers[0])]
    if values is not None:
        parts.append((values, value_pages, value_scales, multipliers[1]))
    for rows, store, scales, mult in parts:
        hkv, dim = rows.shape[1], rows.shape[2]
        codes, scale = encode(rows[keep], kind, mult)
        target = _bytes(store).view(-1, hkv, dim)
        target.index_copy_(0, slot_ids[keep], _bytes(codes))
        if scale is not None:
            scales.view(-1, hkv).index_copy_(0, slot_ids[keep], scale)


def decode_rows(store, scales, kind, multiplier=1.0, dtype=torch.float64):
    """Stored rows [..., HKV, dim] (and their scales [..., HKV] for row kinds) as real values: code * multiplier or
    code * scale (test_paged_kv_attention.py:50-60)."""
    x = store.to(dtype)
    if kind == "fp8":
        m = torch.as_tensor(multiplier, dtype=dtype)
        if m.dim() == 1:
            m = m[:, None]
        x = x * m
    if kind in ROW_SCALED:
        x = x * scales.to(dtype)[..., None]
    return x


def rope(x, positions, table, style="half", scale=1.0):
    """Each token's heads [tokens][heads][dim] rotated at its position over the whole head width, as the reference's
    rope() with a [positions][dim] table (cos of every pair, then sin; inference/fused-norms/code/torch_norms.py:89-147):
    FP32 inside (a cos - b sin, b cos + a sin as separate products and a sum), positions clamped to the table's rows,
    scale on cos and sin, one rounding to x's dtype. Pairs (j, j + dim / 2) for style half, (2j, 2j + 1) interleaved."""
    dim = x.shape[-1]
    half = dim // 2
    rows = table.float().index_select(0, torch.as_tensor(positions, dtype=torch.int64).clamp(0, table.shape[0] - 1))
    cos, sin = rows[:, :half], rows[:, half:]
    if scale != 1.0:
        cos, sin = cos * scale, sin * scale
    cos, sin = cos[:, None, :], sin[:, None, :]
    x32 = x.float()
    if style == "half":
        a, b = x32[..., :half], x32[..., half:]
        turned = torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
    elif style == "interleaved":
        a, b = x32[..., 0::2], x32[..., 1::2]
        turned = torch.stack([a * cos - b * sin, b * cos + a * sin], -1).flatten(-2)
    else:
        raise ValueError(style)
    return turned.to(x.dtype)


def sum_of_squares(x32):
    """The FP32 sum of squares of each last-dimension row (a multiple of 8 wide, that many groups a power of two) in
    the fixed order the fused append takes it in: every square rounded to FP32, groups of 8 consecutive elements summed
    in order, the groups by a balanced tree of adjacent pairs. Plain FP32 additions, no fused multiply-add."""
    import numpy as np
    sq = x32.numpy().astype(np.float32)
    sq = sq * sq
    groups = sq.reshape(*sq.shape[:-1], sq.shape[-1] // 8, 8)
    s = groups[..., 0].copy()
    for j in range(1, 8):
        s = s + groups[..., j]
    while s.shape[-1] > 1:
        s = s[..., 0::2] + s[..., 1::2]
    return torch.from_numpy(s[..., 0].astype(np.float32))


def rms_norm_rope(x, weight, eps, positions, table, offset=0.0, style="half", scale=1.0):
    """Each token's heads [tokens][heads][dim] RMS-normalised, weighted and rotated at its position, as the reference's
    rms_norm_rope() (inference/fused-norms/code/torch_norms.py:149-176: rms_norm of each head in FP32, times weight (+
    offset), then rope, FP32 between them, one rounding to x's dtype) over the whole head width with a
    [positions][dim] table. The reference's mean of squares is torch's (its order of summation is the library's own);
    here it is sum_of_squares() / dim, so that a kernel can reproduce the bytes; 1 / sqrt(mean + eps) by an IEEE square
    root and an IEEE division (what torch's CPU rsqrt does), (x * r) * (weight + offset) as two FP32 products."""
    import numpy as np
    x32 = x.float()
    dim = x.shape[-1]
    mean = (sum_of_squares(x32).numpy() / np.float32(dim)).astype(np.float32)
    with np.errstate(divide="ignore"):      # (a row of zeros under eps 0: 1 / 0 is the infinity torch's rsqrt gives)
        r = (np.float32(1.0) / np.sqrt(mean + np.float32(eps), dtype=np.float32)).astype(np.float32)
    factor = weight.float()
    if offset:
        factor = factor + offset
    normed = (x32 * torch.from_numpy(r)[..., None]) * factor
    return rope(normed, positions, table, style, scale).to(x.dtype)
