"""Latent attention (multi-head latent attention, absorbed) on MI355X: the host side of crit's latent-attention kernels
module (reference kernels/techniques/attention/latent-attention/torch-ext/latent_attention/__init__.py), same names,
arguments and errors, over the gfx950 kernels of libcrit_pkv.so (crit_pkv_latent_attend). crit's attention plugin calls
it for pools of keys only with one KV head (inference/attention-state/code/device_attention.py:444-519).

    write(latent, rope, slots, cache)                  # rows into their page slots: cache [pages][page][R + P]
    out = attend(q, cache, tables, rows, starts, firsts, columns, page, rank=R)
    # q [tokens][heads][R + P]: the query's latent part (the key up-projection absorbed) then its rotary part;
    # out [tokens][heads][R]: the attention output in the latent space

Row b of a launch is table row rows[b]'s sequence; its columns are tokens starts[b] .. starts[b] + counts[b] - 1 at
positions firsts[b] + column, each seeing the positions up to its own. A row's positions are cut into pieces of PIECE
positions, piece i to partition i mod partitions(); the partitions' states are merged in partition order. A token's bits
depend on its own query and positions, the piece and the partition count, never on the rows or columns beside it.
fused=True gives the same bits (here: the same launches over the module's bounded partials, a few rows at a time);
prefill() reads a prompt chunk as windows of MAX_COLUMNS columns, so a prompt token has the bits of the same position
decoded (what the reference's plugin does with prompt_reader "decode"). There is no other implementation behind this
module: without the library every call fails.
"""
from typing import Optional

import torch

from ..paged_kv_attention import _abi
from ..paged_kv_attention import _launch, _ptr, _require_device

try:        # crit's kernel build writes the engine's tuned knobs beside the module (kernels/crit_kernels/build.py:255-313)
    from . import _crit_tuning
except ImportError:
    _crit_tuning = None

__all__ = ["MAX_COLUMNS", "PARTIAL_BYTES", "PIECE", "SHAPES", "attend", "partitions", "prefill", "write"]

MAX_COLUMNS = 64
PARTIAL_BYTES = 512 << 20   # a launch's partials: rows whose partials would take more are launched a few at a time
PIECE = 256                 # positions a piece (an order knob: one value for every launch)
MAX_PARTS = 64
SHAPES = ((512, 64), (256, 64), (128, 64), (128, 32), (64, 64), (64, 32))   # (rank, rotary width) the kernels are built for
FP8 = torch.float8_e4m3fn
_DTYPE = {torch.float32: _abi.F32, torch.bfloat16: _abi.BF16, torch.float16: _abi.F16}
_CUS = {}
_partials = {}      # device index -> the module's partials (FP32), grown outside a capture


def _cus(device):
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _CUS:
        _CUS[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _CUS[index]


def _knob(name, heads, rank, rope, page, kind):
    """The engine's tuned value of a knob of the "window" structure for this geometry, 0 where it has none (the
    reference's _knobs(), __init__.py:44-50)."""
    if _crit_tuning is None:
        return 0
    key = {"R": int(rank), "P": int(rope), "H": int(heads), "PAGE": int(page), "KIND": int(kind)}
    return int(_crit_tuning.knobs("window", key, 1).get(name, 0) or 0)


def partitions(device, heads, rank, rope, page, kind=0):
    """The partitions a launch over this geometry splits a row's positions into: the tuning's PARTS, else the rule:
    the CUs over twice the heads' 16-row tiles, 1 to MAX_PARTS, from the heads and the device only (the reference's:
    2 x SMs over the tiles, __init__.py:65-71). Every partition's state is a partial the merge reads again, and a
    row's tiles all write theirs: measured on MI355X (64 rows of 1,024 to 8,192 positions, R 512, P 64) 128 heads
    take 356 / 294 / 261 us with 32 / 16 / 8 partitions and a lone row of 8,192 positions 34 / 42 / 67 us; 16 heads
    102 / 97 / 89 us with 64 / 16 / 8 and a lone row 28 / 36 / 57 us. The rule gives 64, 64, 32, 16 for 16, 32, 64
    and 128 heads; an engine that serves batches only sets PARTS lower."""
    tuned = _knob("PARTS", heads, rank, rope, page, kind)
    if tuned:
        return max(1, min(MAX_PARTS, tuned))
    return max(1, min(MAX_PARTS, _cus(device) // (2 * max(1, -(-int(heads) // 16)))))


def write(latent, rope, slots, cache, scales=None):
    """latent [N][R] and rope [N][P] into their slots (int64 [N], page * page_size + offset) of cache
    [pages][page][R + P], in the cache's dtype (device work only; capture-safe). An E4M3 cache takes scales FP32
    [pages][page][2]: each position's latent and rotary key coded at their own scale, max |x| / 448 (at least 1e-30),
    the codes the nearest E4M3 values of x / scale (IEEE divisions). Plain torch indexing, as the reference's."""
    rank = latent.shape[-1]
    if cache.shape[-1] != rank + rope.shape[-1] or latent.shape[0] != rope.shape[0] or slots.shape[0] != latent.shape[0]:
        raise ValueError("a cache row is the latent then the rotary key, one row a slot")
    slots = slots.long()
    if cache.dtype == FP8:
        if scales is None or tuple(scales.shape) != (*cache.shape[:2], 2) or scales.dtype != torch.float32:
            raise ValueError("an E4M3 cache takes scales FP32 [pages][page][2] (the latent's, the rotary key's)")
        codes, found = [], []
        for x in (latent.float(), rope.float()):
            amax = x.abs().amax(-1)
            s = (amax / torch.full_like(amax, 448.0)).clamp(min=1e-30)
            codes.append((x / s[:, None]).clamp(-448.0, 448.0).to(FP8).view(torch.uint8))
            found.append(s)
        cache.view(torch.uint8).view(-1, cache.shape[-1]).index_copy_(0, slots, torch.cat(codes, dim=-1))
        scales.view(-1, 2).index_copy_(0, slots, torch.stack(found, dim=-1))
        return
    cache.view(-1, cache.shape[-1]).index_copy_(0, slots, torch.cat([latent.to(cache.dtype), rope.to(cache.dtype)], dim=-1))


def _check(q, cache, page, rank, sinks, scales):
    """(R, P, fp8) of a call, its inputs checked (the reference's checks and messages, __init__.py:96-117)."""
    _require_device(q, "latent attention's q")
    T, H, width = q.shape
    R, P = int(rank), width - int(rank)
    if cache.dim() != 3 or cache.shape[-1] != width or cache.shape[1] != page or not cache.is_contiguous():
        raise ValueError(f"the cache is contiguous [pages][{page}][{width}]: the latent then the rotary key")
    fp8 = cache.dtype == FP8
    if (q.dtype != cache.dtype and not fp8) or q.dtype not in (torch.bfloat16, torch.float16) or q.stride(-1) != 1:
        raise ValueError("q is BF16 or FP16 in the cache's dtype (either over an E4M3 cache), its last dimension "
                         "contiguous")
    if fp8 and (scales is None or tuple(scales.shape) not in ((*cache.shape[:2], 2), (*cache.shape[:2], 1)) or
                scales.dtype != torch.float32 or not scales.is_contiguous()):
        raise ValueError("an E4M3 cache takes its scales FP32 [pages][page][2] (or [pages][page][1]: one a row)")
    if R < 16 or P < 16 or R & (R - 1) or P & (P - 1) or R > 1024 or P > 256:
        raise ValueError("the rank and the rotary width are powers of two (16 to 1024 and 16 to 256)")
    if sinks is not None and (sinks.dtype != torch.float32 or tuple(sinks.shape) != (H,) or not sinks.is_contiguous()
                              or sinks.device != q.device):
        raise ValueError(f"sinks are contiguous FP32 [{H}] on q's device")
    if (R, P) not in SHAPES:
        raise NotImplementedError(f"latent_attention (gfx950): rank {R} with a rotary width of {P} is not built; "
                                  f"(rank, rotary width) is one of {SHAPES}")
    if cache.device != q.device:
        raise ValueError("q and the cache live on one device")
    return R, P, fp8


def _workspace(device, floats):
    index = device.index if device.index is not None else torch.cuda.current_device()
    held = _partials.get(index)
    if held is None or held.numel() < floats:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("latent_attention: the partials grow outside a capture: run the launch's shape eagerly first")
        held = _partials[index] = torch.empty(floats, dtype=torch.float32, device=device)
    return held


def attend(q, cache, tables, rows, starts, firsts, columns, page, *, rank, counts=None, scale=None,
           out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
           sinks: Optional[torch.Tensor] = None, scales: Optional[torch.Tensor] = None,
           fused: Optional[bool] = None, piece=None, partitions=None, phases=0) -> torch.Tensor:
    """Decode tokens and verify windows over the latent cache (see the module's description). q [tokens][heads][R + P]
    BF16 or FP16 in the cache's dtype, the last dimension contiguous; cache [pages][page][R + P] contiguous; tables
    [S][width] int32; rows, starts [B] int32 (rows int64 too: a round's slots as they are); firsts [B] int64; counts [B]
    int32 (None: `columns` each); columns the widest row (a Python int, 1 to MAX_COLUMNS). Returns out
    [tokens][heads][R] in q's dtype (written at the rows' tokens); lse [tokens][heads] FP32 when given; sinks FP32
    [heads]. scale defaults to (R + P) ** -0.5 (pass the model's). An E4M3 cache takes its scales, with BF16 or FP16
    queries: write()'s two a position, or one a position for the whole row ([pages][page][1], a KV pool's fp8:row pages
    of one head). fused: the same bits whatever it says; the rows are launched a few at a time where their partials
    would take more than PARTIAL_BYTES. piece: positions a piece (a multiple of 32; default the tuning's PIECE, else
    PIECE), partitions: 1 to MAX_PARTS (default partitions()); a token's bits depend on both, so a caller keeps one
    value of each for a geometry. phases (a measurement's): 1 the partitions' launch only, 2 the merge only."""
    R, P, fp8 = _check(q, cache, page, rank, sinks, scales)
    T, H, width = q.shape
    B = int(starts.shape[0])
    if not 1 <= columns <= MAX_COLUMNS or B == 0:
        raise ValueError(f"1..{MAX_COLUMNS} columns a row, one row or more")
    if tables.dtype != torch.int32 or tables.stride(-1) != 1 or rows.dtype not in (torch.int32, torch.int64) or \
            starts.dtype != torch.int32 or firsts.dtype != torch.int64 or (counts is not None and counts.dtype != torch.int32):
        raise ValueError("tables, starts and counts are int32, rows int32 or int64 and firsts int64")
    device = q.device
    piece = int(piece or _knob("PIECE", H, R, P, page, int(fp8)) or PIECE)
    if piece < 32 or piece % 32:
        raise ValueError(f"a piece is a multiple of 32 positions, not {piece}")
    parts = globals()["partitions"](device, H, R, P, page, int(fp8)) if partitions is None else int(partitions)
    if not 1 <= parts <= MAX_PARTS:
        raise ValueError(f"1..{MAX_PARTS} partitions, not {parts}")
    if out is None:
        out = torch.empty(T, H, R, dtype=q.dtype, device=device)
    if out.dtype not in _DTYPE or out.stride(-1) != 1 or out.shape[-1] != R:
        raise ValueError("out is [tokens][heads][rank] BF16, FP16 or FP32, its last dimension contiguous")
    if lse is not None and (lse.dtype != torch.float32 or not lse.is_contiguous()):
        raise ValueError("lse is contiguous FP32 [tokens][heads]")
    per_row = int(columns) * H * parts                    # partial states a batch row takes
    rows_a_launch = max(1, min(B, (PARTIAL_BYTES // 4) // (per_row * (R + 2))))
    work = _workspace(device, rows_a_launch * per_row * (R + 2))
    p = _abi.LatentParams()
    p.q, p.cache, p.scales, p.tables = q.data_ptr(), cache.data_ptr(), _ptr(scales) if fp8 else None, tables.data_ptr()
    p.out, p.lse, p.sinks = out.data_ptr(), _ptr(lse), _ptr(sinks)
    p.q_stride_t, p.q_stride_h, p.out_stride_t, p.out_stride_h = q.stride(0), q.stride(1), out.stride(0), out.stride(1)
    p.table_stride, p.table_width = tables.stride(0), tables.shape[1]
    p.columns, p.heads, p.rank, p.rope, p.page = int(columns), H, R, P, int(page)
    p.cache_dtype = 2 if fp8 else (1 if cache.dtype == torch.float16 else 0)
    p.q_dtype, p.out_dtype = _DTYPE[q.dtype], _DTYPE[out.dtype]
    p.scales_per_row = int(scales.shape[-1]) if fp8 else 0
    p.partitions, p.piece, p.rows_are_64, p.phases = parts, piece, int(rows.dtype == torch.int64), int(phases)
    p.scale = float(scale if scale is not None else width ** -0.5)
    for at in range(0, B, rows_a_launch):
        n = min(rows_a_launch, B - at)
        states = n * per_row
        p.partial_out = work.data_ptr()
        p.partial_max = work.data_ptr() + states * R * 4
        p.partial_sum = work.data_ptr() + states * (R + 1) * 4
        p.n_rows = n
        p.rows = rows.data_ptr() + at * rows.element_size()
        p.starts, p.firsts = starts.data_ptr() + at * 4, firsts.data_ptr() + at * 8
        p.counts = None if counts is None else counts.data_ptr() + at * 4
        _launch(device, "crit_pkv_latent_attend", "latent_attention.attend", p)
    return out


def prefill(q, cache, table, position, page, *, rank, scale=None, out: Optional[torch.Tensor] = None,
            lse: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None,
            scales: Optional[torch.Tensor] = None) -> torch.Tensor:
    """A prompt chunk of one sequence over the latent cache: q [T][heads][R + P] at positions position .. position +
    T - 1 (their rows written), table [pages] int32 its page table, position an int or a one-element int64 device
    tensor read on the device (one graph for every position) -> out [T][heads][R] in q's dtype (and lse [T][heads] when
    given), causal. Read as windows of MAX_COLUMNS columns through attend(): a token's bits do not depend on the
    chunk's length and are those of the same position decoded. Sinks, lse, scale and an E4M3 cache's scales as
    attend()."""
    T = q.shape[0]
    _check(q, cache, page, rank, sinks, scales)
    if T < 1 or table.dim() != 1:
        raise ValueError("a prompt chunk is one token or more over one page table [pages]")
    device = q.device
    if torch.is_tensor(position):
        first = position.reshape(1)
        if first.dtype != torch.int64 or first.device != device:
            raise ValueError("a device position is a one-element int64 tensor on q's device")
    else:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("latent_attention.prefill: a captured chunk takes its position as a device tensor")
        first = torch.tensor([int(position)], dtype=torch.int64, device=device)
    n = -(-T // MAX_COLUMNS)
    step = torch.arange(n, dtype=torch.int64, device=device) * MAX_COLUMNS
    counts = (T - step).clamp(max=MAX_COLUMNS).to(torch.int32)
    tables = table.reshape(1, -1)
    if tables.dtype != torch.int32:
        tables = tables.to(torch.int32)
    return attend(q, cache, tables, torch.zeros(n, dtype=torch.int32, device=device), step.to(torch.int32), first + step,
                  min(MAX_COLUMNS, T), page, rank=rank, counts=counts, scale=scale, out=out, lse=lse, sinks=sinks,
                  scales=scales, fused=True)
