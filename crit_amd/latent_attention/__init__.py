"""Latent attention (multi-head latent attention with the key up-projection absorbed) on MI355X: the host side of crit's
latent-attention kernels module (reference kernels/techniques/attention/latent-attention/torch-ext/latent_attention/
__init__.py: `write` :74-97, `prefill` :121-152, `attend` :155-229, `partitions` :65-71), with the same calls, keyword
arguments and error types, over the gfx950 kernels of libcrit_pkv.so (crit_pkv_latent_attend, crit_pkv_latent_write).
crit's attention plugin calls it for keys-only pools of one KV head (inference/attention-state/code/
device_attention.py:444-519). There is no other implementation behind this module: without the library every call fails.

The cache is [pages][page][R + P]: position n of a sequence keeps its latent (R values) and then its rotary key (P
values) in one row at slot table[n // page] * page + n % page. A query is [R + P] too, its latent part already
multiplied through the key up-projection, so for every head

    score[n] = scale * (q[:R] . row[n][:R] + q[R:] . row[n][R:])      out = sum_n softmax(score)[n] * row[n][:R]

write()    puts rows into their slots (one launch, any float input type).
attend()   decode tokens and verify windows: batch row b is the sequence of table row rows[b]; its counts[b] columns are
           tokens starts[b].. of q at positions firsts[b] + column, each seeing positions up to its own.
prefill()  a prompt chunk of one sequence, causal.

Order of the sums. A row's positions are cut into pieces of `piece` positions, piece i going to partition i mod
partitions; each partition's running state is folded into the result in partition order, the sink last. A token's bits
depend on its own query and positions, `piece` and the partition count only, never on the batch it rode in, so
fused=True / False and any row batching give equal bits, and prefill() (which reads a chunk as windows of MAX_COLUMNS
columns) gives each prompt token the bits it would have decoded.
"""
from typing import Optional

import torch

from ..paged_kv_attention import _abi
from ..paged_kv_attention import _grown, _holding, _launch, _ptr, _require_device

try:        # crit's kernel build writes the engine's tuned knobs beside the module (kernels/crit_kernels/build.py:255-313)
    from . import _crit_tuning
except ImportError:
    _crit_tuning = None

__all__ = ["MAX_COLUMNS", "PARTIAL_BYTES", "PIECE", "PIECE_MANY_HEADS", "SHAPES", "attend", "partitions", "prefill",
           "tile_rows", "write"]

MAX_COLUMNS = 64
PARTIAL_BYTES = 512 << 20   # the most partials one launch may take; a larger batch goes in several launches of rows
PIECE = 256                 # default positions a piece
PIECE_MANY_HEADS = 512      # ... where the many-heads kernel reads (TILE_ROWS 128)
MAX_PARTS = 64
SHAPES = tuple((r, p) for r in (1024, 512, 256, 128, 64) for p in (256, 128, 64, 32))   # (R, P) the matrix-core kernels read;
# ranks 16 and 32 and a rotary width of 16 are served by a kernel of plain vector arithmetic
FP8 = torch.float8_e4m3fn
_DTYPE = {torch.float32: _abi.F32, torch.bfloat16: _abi.BF16, torch.float16: _abi.F16}
_CACHE_DTYPE = {torch.bfloat16: 0, torch.float16: 1, FP8: 2}
_CUS = {}


def _cus(device):
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _CUS:
        _CUS[index] = torch.cuda.get_device_properties(index).multi_processor_count
    return _CUS[index]


def _knob(name, heads, rank, rope, page, kind):
    """The engine's tuned value of knob `name` for this geometry (structure "window", keyed as the reference keys it,
    __init__.py:44-50), or 0."""
    if _crit_tuning is None:
        return 0
    key = {"R": int(rank), "P": int(rope), "H": int(heads), "PAGE": int(page), "KIND": int(kind)}
    return int(_crit_tuning.knobs("window", key, 1).get(name, 0) or 0)


def partitions(device, heads, rank, rope, page, kind=0, tile_rows=None):
    """How many partitions a row's pieces are dealt to for this geometry on `device`: the tuned PARTS if the engine has
    one, else one workgroup's worth of work for every second compute unit per 16 heads, between 1 and MAX_PARTS (64 for
    16 and 32 heads, 32 for 64, 16 for 128 on 256 compute units); where the many-heads kernel reads (tile_rows(...) ==
    128), whose workgroups take a compute unit each and 128 query rows, one for every 32 compute units (8). It depends
    on the geometry and the device only, because a token's bits depend on it. (The reference's rule is the same idea
    for its tiles: __init__.py:65-71.)"""
    tuned = _knob("PARTS", heads, rank, rope, page, kind)
    if tuned:
        return min(MAX_PARTS, max(1, tuned))
    if globals()["tile_rows"](heads, rank, rope, page, kind, tile_rows) == 128:
        return min(MAX_PARTS, max(1, _cus(device) // 32))
    return min(MAX_PARTS, max(1, _cus(device) // (2 * max(1, -(-int(heads) // 16)))))


def tile_rows(heads, rank, rope, page, kind=0, asked=None):
    """The query rows a workgroup holds for this geometry, 16 or 128, which names the kernel that reads it (and a token's
    bits follow the kernel). 128, the many-heads kernel (32 x 32 matrix tiles, the cache rows by DMA into LDS, one
    workgroup a compute unit), takes caches of DeepSeek's shape (512, 64), 16-bit or E4M3, with pages of a multiple of 16
    positions. Heads in 128s get it unless `asked` (attend's tile_rows=) or the engine's tuned TILE_ROWS says 16: it
    reads a batch of 64 rows about twice as fast as the small tiles, and a single row twice slower (one workgroup a
    partition instead of four). With fewer heads it is there for the asking (a tile is then 128 / heads columns of a
    window: prompt chunks, prefill's packed=True); left alone they get 16, as does everything else."""
    able = (int(rank), int(rope)) == (512, 64) and int(page) % 16 == 0
    want = int(asked or _knob("TILE_ROWS", heads, rank, rope, page, kind) or 0)
    if want not in (0, 16, 128):
        raise ValueError(f"tile_rows: {want}; 16 or 128 (or 0: by the geometry)")
    if want == 128 and not able:
        raise ValueError("tile_rows 128 reads caches of (512, 64) with pages of a multiple of 16 positions")
    return 128 if able and (want == 128 or (want == 0 and int(heads) % 128 == 0)) else 16


def write(latent, rope, slots, cache, scales=None):
    """Append rows: token t's latent[t] ([N][R]) and rope[t] ([N][P]) side by side into row slots[t] (int64 [N]) of
    cache [pages][page][R + P], converted to the cache's dtype. A float8_e4m3fn cache also takes scales FP32
    [pages][page][2]: each part is coded at its own scale max|x| / 448 (not below 1e-30) and the two scales are stored
    at the row's place. One kernel launch, nothing allocated when the inputs are contiguous rows of one float type."""
    if latent.dim() != 2 or rope.dim() != 2 or cache.dim() != 3:
        raise ValueError("write: latent [N][R], rope [N][P] and cache [pages][page][R + P]")
    n, rank = latent.shape
    width = rope.shape[1]
    if rope.shape[0] != n or slots.shape != (n,) or cache.shape[2] != rank + width:
        raise ValueError(f"write: {n} latents of {rank} need {n} rotary keys, {n} slots and cache rows of "
                         f"{rank} + {width}, not {tuple(rope.shape)}, {tuple(slots.shape)}, {cache.shape[2]}")
    _require_device(cache, "the latent cache")
    if cache.dtype not in _CACHE_DTYPE or not cache.is_contiguous():
        raise ValueError("write: the cache is contiguous BF16, FP16 or float8_e4m3fn")
    coded = cache.dtype == FP8
    if coded and (scales is None or scales.dtype != torch.float32 or tuple(scales.shape) != (*cache.shape[:2], 2)
                  or not scales.is_contiguous()):
        raise ValueError(f"write: an E4M3 cache keeps two FP32 scales a row, [{cache.shape[0]}][{cache.shape[1]}][2]")
    if n == 0:
        return
    if latent.dtype not in _DTYPE:
        latent = latent.float()
    if rope.dtype != latent.dtype:
        rope = rope.to(latent.dtype)
    if latent.stride(1) != 1:
        latent = latent.contiguous()
    if rope.stride(1) != 1:
        rope = rope.contiguous()
    if slots.dtype != torch.int64 or not slots.is_contiguous():
        slots = slots.long().contiguous()
    p = _abi.LatentWriteParams()
    p.latent, p.rope, p.slots, p.cache, p.scales = latent.data_ptr(), rope.data_ptr(), slots.data_ptr(), cache.data_ptr(), \
        _ptr(scales) if coded else None
    p.tokens, p.latent_stride, p.rope_stride = n, latent.stride(0), rope.stride(0)
    p.rank, p.rope_width, p.in_dtype, p.cache_dtype = rank, width, _DTYPE[latent.dtype], _CACHE_DTYPE[cache.dtype]
    _launch(cache.device, "crit_pkv_latent_write", "latent_attention.write", p)


class _Call:
    """The operands every reading call shares, validated once: q, the cache, its scales and the sinks."""
    __slots__ = ("tokens", "heads", "rank", "rope", "coded")

    def __init__(self, q, cache, page, rank, sinks, scales):
        if q.dim() != 3:
            raise ValueError("q: [tokens][heads][R + P]")
        _require_device(q, "latent attention's q")
        self.tokens, self.heads, width = q.shape
        self.rank, self.rope = int(rank), width - int(rank)
        self.coded = cache.dtype == FP8
        if cache.dim() != 3 or tuple(cache.shape[1:]) != (page, width) or not cache.is_contiguous():
            raise ValueError(f"cache: contiguous [pages][{page}][{width}] (a row is R latent values, then P rotary), "
                             f"not {tuple(cache.shape)}")
        if q.dtype not in (torch.bfloat16, torch.float16) or q.stride(-1) != 1 or not (self.coded or q.dtype == cache.dtype):
            raise ValueError("q: BF16 or FP16 in the cache's dtype (either of the two over an E4M3 cache), unit stride "
                             "along its last dimension")
        if self.coded:
            ok = scales is not None and scales.dtype == torch.float32 and scales.is_contiguous() and \
                scales.dim() == 3 and tuple(scales.shape[:2]) == tuple(cache.shape[:2]) and scales.shape[2] in (1, 2)
            if not ok:
                raise ValueError("scales: an E4M3 cache takes its scales, contiguous FP32 [pages][page][2] (latent, rotary "
                                 "key) or [pages][page][1] (one for the row)")

        def power_of_two(n, low, high):
            return low <= n <= high and n & (n - 1) == 0

        if not power_of_two(self.rank, 16, 1024) or not power_of_two(self.rope, 16, 256):
            raise ValueError(f"rank {self.rank} / rotary width {self.rope}: both are powers of two, 16..1024 and 16..256")
        if sinks is not None:
            if sinks.dtype != torch.float32 or tuple(sinks.shape) != (self.heads,) or not sinks.is_contiguous() or \
                    sinks.device != q.device:
                raise ValueError(f"sinks: one FP32 logit a head, contiguous [{self.heads}] on q's device")
        if cache.device != q.device:
            raise ValueError(f"cache is on {cache.device}, q on {q.device}")


def _partials(device, floats):
    """The current owner's partials buffer on `device` (paged_kv_attention.owner()), at least `floats` long. It grows
    outside a capture only, and a buffer it outgrew is kept alive, because a captured graph may still replay into it."""
    return _grown(_holding(device), "latent", floats, device, 1 << 16,
                  "latent attend: run a launch of this shape once before capturing it")


def attend(q, cache, tables, rows, starts, firsts, columns, page, *, rank, counts=None, scale=None,
           out: Optional[torch.Tensor] = None, lse: Optional[torch.Tensor] = None,
           sinks: Optional[torch.Tensor] = None, scales: Optional[torch.Tensor] = None,
           fused: Optional[bool] = None, piece=None, partitions=None, workspace: Optional[torch.Tensor] = None,
           phases=0, tile_rows=None) -> torch.Tensor:
    """Decode tokens and verify windows (see the module text). q [tokens][heads][R + P]; tables [S][width] int32; rows
    and starts [B] int32 (rows may be int64); firsts [B] int64; counts [B] int32 or None (every row has `columns`);
    columns: the widest row, a Python int within 1..MAX_COLUMNS. Returns out [tokens][heads][R] (q's dtype unless `out`
    is given as BF16, FP16 or FP32), written at the rows' tokens only. lse: FP32 [tokens][heads], the natural
    log-sum-exp of a token's scaled scores, its sink included. sinks: FP32 [heads] logits of one extra position that has
    no value. scale: default (R + P) ** -0.5. scales: an E4M3 cache's, as write() stores them, or one a row.

    fused is accepted for the reference's signature and changes nothing: the bits are the same either way and the
    partials stay bounded (PARTIAL_BYTES; a larger batch is launched a few rows at a time). piece (a multiple of 32)
    and partitions (1..MAX_PARTS) default to the tuned values or PIECE and partitions(); keep one value of each per
    geometry, since a token's bits depend on them. workspace: FP32 scratch for the partials; without it the module uses
    a buffer held per owner (paged_kv_attention.owner) and device, so launches of two owners on two streams never share
    partials. phases is for timing: 1 runs the partitions' launch alone, 2 the merge alone. tile_rows: 16 or 128, the
    kernel that reads (see tile_rows()); default: the tuned TILE_ROWS, else by the geometry."""
    call = _Call(q, cache, page, rank, sinks, scales)
    heads, R, P = call.heads, call.rank, call.rope
    batch = int(starts.shape[0])
    if batch < 1 or not 1 <= int(columns) <= MAX_COLUMNS:
        raise ValueError(f"a launch has at least one row and 1..{MAX_COLUMNS} columns a row, not {batch} x {columns}")
    columns = int(columns)
    if tables.dtype != torch.int32 or tables.dim() != 2 or tables.stride(1) != 1:
        raise ValueError("tables: int32 [sequences][pages], unit stride along pages")
    if rows.dtype not in (torch.int32, torch.int64) or starts.dtype != torch.int32 or firsts.dtype != torch.int64 or \
            (counts is not None and counts.dtype != torch.int32):
        raise ValueError("rows: int32 or int64; starts and counts: int32; firsts: int64")
    device = q.device
    coded = int(call.coded)
    tiles = globals()["tile_rows"](heads, R, P, page, coded, tile_rows)
    piece = int(piece or _knob("PIECE", heads, R, P, page, coded) or (PIECE_MANY_HEADS if tiles == 128 else PIECE))
    if piece < 32 or piece % 32:
        raise ValueError(f"piece: {piece}; a multiple of 32 positions")
    parts = int(partitions) if partitions is not None else globals()["partitions"](device, heads, R, P, page, coded, tiles)
    if not 1 <= parts <= MAX_PARTS:
        raise ValueError(f"partitions: {parts}; within 1..{MAX_PARTS}")
    if out is None:
        out = torch.empty(call.tokens, heads, R, dtype=q.dtype, device=device)
    elif out.dtype not in _DTYPE or out.dim() != 3 or out.shape[2] != R or out.stride(2) != 1:
        raise ValueError(f"out: BF16, FP16 or FP32 [tokens][heads][{R}], unit stride along its last dimension")
    if lse is not None and (lse.dtype != torch.float32 or not lse.is_contiguous()):
        raise ValueError("lse: contiguous FP32 [tokens][heads]")
    # (the many-heads kernel stores whole tiles of 128 rows)
    states_a_row = (-(-columns * heads // 128) * 128 if tiles == 128 else columns * heads) * parts
    floats_a_row = states_a_row * (R + 2)
    if workspace is None:
        rows_a_launch = max(1, min(batch, (PARTIAL_BYTES // 4) // floats_a_row))
        work = _partials(device, rows_a_launch * floats_a_row)
    else:
        if workspace.dtype != torch.float32 or not workspace.is_contiguous() or workspace.numel() < floats_a_row:
            raise ValueError(f"workspace: contiguous FP32 with room for one row's partials at least ({floats_a_row})")
        rows_a_launch = min(batch, workspace.numel() // floats_a_row)
        work = workspace
    p = _abi.LatentParams()
    p.q, p.cache, p.tables = q.data_ptr(), cache.data_ptr(), tables.data_ptr()
    p.scales = _ptr(scales) if coded else None
    p.out, p.lse, p.sinks = out.data_ptr(), _ptr(lse), _ptr(sinks)
    p.q_stride_t, p.q_stride_h, p.out_stride_t, p.out_stride_h = q.stride(0), q.stride(1), out.stride(0), out.stride(1)
    p.table_stride, p.table_width = tables.stride(0), tables.shape[1]
    p.columns, p.heads, p.rank, p.rope, p.page = columns, heads, R, P, int(page)
    p.cache_dtype = _CACHE_DTYPE[cache.dtype]
    p.q_dtype, p.out_dtype = _DTYPE[q.dtype], _DTYPE[out.dtype]
    p.scales_per_row = int(scales.shape[2]) if coded else 0
    p.partitions, p.piece, p.rows_are_64, p.phases = parts, piece, int(rows.dtype == torch.int64), int(phases)
    p.tile_rows = tiles
    p.scale = float((R + P) ** -0.5 if scale is None else scale)
    base = work.data_ptr()
    for first in range(0, batch, rows_a_launch):
        n = min(rows_a_launch, batch - first)
        states = n * states_a_row
        p.partial_out, p.partial_max, p.partial_sum = base, base + 4 * states * R, base + 4 * states * (R + 1)
        p.n_rows = n
        p.rows = rows.data_ptr() + first * rows.element_size()
        p.starts, p.firsts = starts.data_ptr() + 4 * first, firsts.data_ptr() + 8 * first
        p.counts = None if counts is None else counts.data_ptr() + 4 * first
        _launch(device, "crit_pkv_latent_attend", "latent_attention.attend", p)
    return out


def prefill(q, cache, table, position, page, *, rank, scale=None, out: Optional[torch.Tensor] = None,
            lse: Optional[torch.Tensor] = None, sinks: Optional[torch.Tensor] = None,
            scales: Optional[torch.Tensor] = None, tile_rows=None, packed=False) -> torch.Tensor:
    """A prompt chunk of one sequence, causal: q [T][heads][R + P] are the tokens at positions position .. position +
    T - 1 (their rows already written), table [pages] int32 the sequence's page table; position is an int, or a
    one-element int64 device tensor that is read on the device so that one captured graph serves every position.
    Returns out [T][heads][R] (and fills lse [T][heads] when given). The chunk is read as windows of MAX_COLUMNS
    columns through attend(), so a token's bits are those of the same position decoded and do not depend on T. scale,
    sinks, lse and an E4M3 cache's scales as attend() takes them.

    packed=True reads the chunk with the many-heads kernel whatever the heads (tile_rows 128: a tile of 128 query rows
    is 128 / heads tokens, the cache rows staged once for all of them), which a chunk of some hundred tokens fills where
    a decode step of few heads does not: several times the small tiles' speed at 16 heads. A token's bits are then the
    many-heads kernel's, not those of the same position decoded with the small tiles (the same attention, other sums:
    within the tolerance either has against the exact result); they still do not depend on T or on its neighbours."""
    _Call(q, cache, page, rank, sinks, scales)
    if packed:
        tile_rows = 128
    count = q.shape[0]
    if count < 1 or table.dim() != 1:
        raise ValueError("prefill: at least one token, over one page table [pages]")
    device = q.device
    if torch.is_tensor(position):
        if position.numel() != 1 or position.dtype != torch.int64 or position.device != device:
            raise ValueError("position: an int, or a one-element int64 tensor on q's device")
        origin = position.reshape(1)
    elif torch.cuda.is_current_stream_capturing():
        raise RuntimeError("latent_attention.prefill: under capture pass `position` as a device tensor")
    else:
        origin = torch.tensor([int(position)], dtype=torch.int64, device=device)
    windows = -(-count // MAX_COLUMNS)
    offsets = torch.arange(0, windows * MAX_COLUMNS, MAX_COLUMNS, dtype=torch.int64, device=device)
    widths = torch.clamp(count - offsets, max=MAX_COLUMNS).to(torch.int32)
    one_table = table.reshape(1, -1) if table.dtype == torch.int32 else table.reshape(1, -1).to(torch.int32)
    return attend(q, cache, one_table, torch.zeros(windows, dtype=torch.int32, device=device), offsets.to(torch.int32),
                  origin + offsets, min(MAX_COLUMNS, count), page, rank=rank, counts=widths, scale=scale, out=out, lse=lse,
                  sinks=sinks, scales=scales, fused=True, tile_rows=tile_rows)
