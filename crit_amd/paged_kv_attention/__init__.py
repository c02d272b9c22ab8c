"""Attention over paged KV caches on one MI355X (gfx950): the kernels module crit's KVPool and DeviceAttention call.

The same module interface as crit's `paged_kv_attention` package (reference kernels/techniques/attention/
paged-kv-attention/torch-ext/paged_kv_attention/__init__.py): write(), attend(), prefill(), partitions(), piece_size(),
tile_for(), workspace_floats(), the flash_* and cuda_* rules, owner()/release(), KINDS and MAX_COLUMNS, with the same
argument names, meaning and errors, so `KVPool(kernels=this_module)` and `DeviceAttention(kernels=this_module)` work
unchanged. Behind it are hand-written HIP kernels in libcrit_pkv.so, reached through a C ABI with ctypes (_abi.py);
torch is used for device memory and streams only. There is no fallback: a missing library is an error.

Pages. A cache layer is keys [pages][page][kv_heads][dim] and values [pages][page][kv_heads][value_dim]; position p of
a sequence lives at slot table[p // page] * page + p % page. Page kinds: "bf16", "fp16"; "fp8" (E4M3 codes, value =
code * multiplier, one multiplier per layer for keys and one for values, or with a [2][kv_heads] FP32 tensor one per
KV head); "fp8:row" and "int8" (codes with an FP32 scale per position and KV head).

Windows (attend). Row r is counts[r] <= columns tokens of one sequence: tokens starts[r].. of q, column c at position
firsts[r] + c (its keys and values written already), page table tables[rows[r]]. Column c sees positions up to its own.
Keys are read in pieces of `piece` positions; piece i belongs to partition i mod P. Each partition's unnormalised
output, running maximum and sum go to the partials and a merge folds a column's partitions in order. A column's bits
depend on its own query and keys, P, the piece and the page kind only: not on the rows beside it nor on the launch's
width. With flash=True (or "cuda") the pieces are contiguous splits of `chunk` positions, one per partition, so the
bits depend on the chunk only.

Everything a launch reads about lengths (firsts, counts, position) is read on the device; after the first call of a
shape nothing is allocated when `out` and `workspace` are given, so launches can be captured in a HIP graph.
"""
import contextlib
import math
import threading
from typing import NamedTuple

import torch

from . import _abi

try:        # crit's kernel build writes the engine's tuned knobs beside the module (kernels/crit_kernels/build.py:255-313)
    from . import _crit_tuning
except ImportError:
    _crit_tuning = None

__all__ = ["KINDS", "PIECE", "MAX_COLUMNS", "Derive", "attend", "derive", "cuda_block", "cuda_chunk", "cuda_parts",
           "cuda_prompt", "cuda_ramp", "cuda_splits", "flash_block", "flash_chunk", "flash_parts", "flash_tile",
           "merge_shards", "owner", "partitions", "piece_size", "prefill", "prefill_rows", "prefill_state_floats", "release",
           "stream_read", "slots_at", "compact", "copy_pages", "rows_at", "gather",
           "tile_for", "workspace_floats", "write"]

KINDS = {"bf16": 0, "fp16": 0, "fp8": 1, "fp8:row": 2, "int8": 3}
PIECE = 1536         # positions per piece of FP8 or INT8 pages at a 128-wide head (piece_size)
MAX_COLUMNS = 64     # columns of one row a launch reads
MAX_LISTED_BLOCKS = 1024      # block ids a token's list holds at most (attend's blocks=)
MAX_QUERY_ROWS = 8   # query rows (columns x group heads) one workgroup holds; wider windows take more tiles
HEAD_WIDTHS = (16, 32, 64, 128, 256)      # key and value head widths attend() reads, in any pairing

_DTYPE = {torch.float32: _abi.F32, torch.bfloat16: _abi.BF16, torch.float16: _abi.F16}


class Derive(NamedTuple):
    """Keys derived from the value rows on read (attend's and prefill's derive=, reference __init__.py:82-121): weight
    FP32 [dim] (or None: all ones), eps, freqs FP32 [rotary_dim / 2] inverse frequencies, rotary_dim. One made by
    derive() holds its table (the freqs, then the weight) packed on the device, so a call allocates nothing; a plain
    tuple of the four is packed at each call."""
    weight: object
    eps: float
    freqs: object
    rotary_dim: int
    table: object = None


def derive(weight, eps, freqs, rotary_dim):
    """A Derive with its table packed once, for every call over the layer."""
    return _derived(Derive(weight, eps, freqs, rotary_dim), None, None)[0]


def _derived(given, d, device):
    """`given` (a Derive or a tuple of its four fields) checked for heads of width d (None: not known yet) on `device`:
    (the Derive with its packed table, whether it has a weight). The checks and their messages are the reference's
    (__init__.py:99-121): any even rotary width from 2 up to the head width, at every head width."""
    found = given if isinstance(given, Derive) else Derive(*given)
    weight, eps, freqs, rot = found.weight, float(found.eps), found.freqs, int(found.rotary_dim)
    if rot < 2 or rot % 2 or (d is not None and rot > d):
        raise ValueError(f"derive's rotary_dim is even, 2 up to the head width {d}, not {rot}")
    device = device if device is not None else (freqs.device if torch.is_tensor(freqs) else None)
    if not torch.is_tensor(freqs) or freqs.dtype != torch.float32 or tuple(freqs.shape) != (rot // 2,) or freqs.device != device:
        raise ValueError(f"derive's freqs are FP32 [{rot // 2}] (rotary_dim / 2 inverse frequencies) on q's device")
    if weight is not None and (not torch.is_tensor(weight) or weight.dtype != torch.float32 or weight.dim() != 1 or
                               (d is not None and weight.shape[0] != d) or weight.device != device):
        raise ValueError(f"derive's weight is FP32 [{d}] (the head width) on q's device, or None")
    if not eps >= 0:
        raise ValueError("derive's eps is 0 or more")
    table = found.table
    if table is None:
        if device is not None and device.type == "cuda" and torch.cuda.is_current_stream_capturing():
            raise RuntimeError("paged_kv_attention: a captured call takes a Derive made by derive() (its table packed)")
        table = freqs.contiguous() if weight is None else torch.cat([freqs, weight.contiguous()])
    elif table.numel() != rot // 2 + (0 if weight is None else weight.shape[0]):
        raise ValueError("a Derive's packed table does not fit its freqs and weight")
    return found._replace(eps=eps, rotary_dim=rot, table=table), weight is not None


# -- owners: what the module itself keeps on a device (reference __init__.py:129-171 keeps its workspaces the same way) --
class _Holding:
    """One owner's memory on one device: the partials of its split launches (`latent`: those of its latent-attention
    launches), the row states of its prompt chunks with fresh rows, and the counters its unit-pulling launches draw from. Buffers a launch outgrew stay in `kept`: a
    captured graph may still replay into them."""
    __slots__ = ("partials", "states", "latent", "counters", "pairs_used", "pair_of", "kept")

    def __init__(self):
        self.partials = self.states = self.latent = self.counters = None
        self.pairs_used, self.pair_of, self.kept = 0, {}, []


COUNTER_PAIRS = 512      # counter pairs an owner's block holds (one a stream that launches, one a capture)
COUNTER_HEADROOM = 384   # pairs an eager launch leaves free for captures: it starts a new block when fewer are left
_holdings = {}           # (device index, owner key) -> _Holding
_local = threading.local()


class owner:
    """`with owner(key):` — the launches inside take module memory of their own (partials, prompt-row states, launch
    counters), apart from every other owner's and from launches outside any block; a graph captured inside replays
    into its owner's memory. Nests; per thread. release(key) drops the memory."""

    def __init__(self, key):
        self.key = key

    def __enter__(self):
        stack = _local.__dict__.setdefault("owners", [])
        stack.append(self.key)
        return self

    def __exit__(self, *exc):
        _local.owners.pop()
        return False


def _owner_key():
    stack = getattr(_local, "owners", None)
    return stack[-1] if stack else None


def release(key):
    """Forget everything the module holds for owner `key`, on every device (its captured graphs must be gone first:
    they replay into that memory)."""
    for at in [at for at in _holdings if at[1] == key]:
        _holdings.pop(at)


def _holding(device):
    index = device.index if device.index is not None else torch.cuda.current_device()
    at = (index, _owner_key())
    found = _holdings.get(at)
    if found is None:
        found = _holdings[at] = _Holding()
    return found


def _grown(holding, name, floats, device, floor, what):
    """The holding's FP32 buffer `name`, at least `floats` long; grown (never under a capture) by replacing it."""
    found = getattr(holding, name)
    if found is None or found.numel() < floats:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError(f"paged_kv_attention.{what} (the module allocates outside a capture only)")
        if found is not None:
            holding.kept.append(found)
        found = torch.empty(max(floats, floor), dtype=torch.float32, device=device)
        setattr(holding, name, found)
    return found


def _launch_state(device, stream):
    """The address of the two counters a unit-pulling launch on `stream` draws from: one pair per (owner, device,
    stream) for eager launches, which run one after another there, and one per (capture, stream) for captured ones, so
    a replaying graph never meets an eager launch or another graph in its counters, whatever streams they run on.
    The pairs come from a zeroed block the owner holds; a launch leaves its pair zero."""
    holding = _holding(device)
    capture = _abi.capture_id(stream)
    if not capture and (holding.counters is None or holding.pairs_used > COUNTER_PAIRS - COUNTER_HEADROOM):
        # An eager launch tops the block up while there is still room for the captures that may follow it: a block is
        # zeroed memory, which a capture cannot allocate. The pairs handed out stay where they are (`kept`).
        if holding.counters is not None:
            holding.kept.append(holding.counters)
        holding.counters, holding.pairs_used = torch.zeros(2 * COUNTER_PAIRS, dtype=torch.int32, device=device), 0
    at = holding.pair_of.get((stream, capture))
    if at is None:
        if holding.counters is None:
            raise RuntimeError("paged_kv_attention.attend: run a launch once on this device before capturing one "
                               "(its launch counters are allocated, zeroed, outside a capture)")
        if holding.pairs_used == COUNTER_PAIRS:
            raise RuntimeError(f"paged_kv_attention.attend: {COUNTER_HEADROOM} captures in a row have used up this "
                               "owner's launch counters; run one launch outside a capture (it allocates the next "
                               "block) and capture again")
        at = holding.pair_of[(stream, capture)] = holding.counters.data_ptr() + 8 * holding.pairs_used
        holding.pairs_used += 1
    return at


def _ptr(t):
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)      # (the stream's handle without a Stream object)


def _stream_of(device):
    """The handle of the caller's current stream on `device`."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    return _raw_stream(index) if _raw_stream is not None else torch.cuda.current_stream(device).cuda_stream


def _launch(device, name, what, *args, stream=None):
    """Calls entry point `name` with args and the caller's current stream of `device` (or `stream`, its handle) as its
    last argument, with `device` current (a decode step calls this about a hundred times: the device is switched only
    where it is not the current one already); raises what _abi.check raises."""
    entry = getattr(_abi.load(), name)
    if stream is None:
        stream = _stream_of(device)
    if device.index is None or device.index == torch.cuda.current_device():
        code = entry(*args, stream)
    else:
        with torch.cuda.device(device):
            code = entry(*args, stream)
    if code:
        _abi.check(code, what)


def _require_device(t, what):
    if not t.is_cuda:
        raise ValueError(f"{what} lives on the GPU (these are HIP kernels; there is no CPU path)")


def _check_kind(kind, key_scales):
    """The kind's number; row-scaled kinds come with their scales, the others without."""
    number = KINDS.get(kind)
    if number is None:
        raise ValueError(f"{kind!r} is no page kind ({', '.join(KINDS)})")
    row_scaled, given = number >= 2, key_scales is not None
    if row_scaled and not given:
        raise ValueError(f"{kind} pages are read with their scales (one per position and KV head)")
    if given and not row_scaled:
        raise ValueError(f"{kind} pages carry no scales per position")
    return number


def _check_sliding(sliding, blocks):
    width = int(sliding) if sliding else 0
    if width < 0:
        raise ValueError(f"sliding={sliding}: a window's width in positions, or 0 for none")
    if width > 0 and blocks is not None:
        raise ValueError("sliding windows and block lists do not combine")
    return width


def _check_sinks(sinks, q):
    if sinks is None:
        return
    heads = q.shape[1]
    ok = (sinks.dtype == torch.float32 and tuple(sinks.shape) == (heads,) and sinks.is_contiguous()
          and sinks.device == q.device)
    if not ok:
        raise ValueError(f"sinks: one FP32 logit per query head ([{heads}], contiguous, on q's device)")


def _multipliers(multipliers, kv_heads, device):
    """(key multiplier, value multiplier, per-head tensor or None): a pair of numbers, or a [2][kv_heads] FP32 tensor
    on the device (one multiplier per KV head: keys' row then values')."""
    if torch.is_tensor(multipliers):
        if multipliers.dtype != torch.float32 or tuple(multipliers.shape) != (2, kv_heads) or \
                not multipliers.is_contiguous() or multipliers.device != device:
            raise ValueError(f"per-head multipliers are a contiguous FP32 [2][{kv_heads}] tensor on the pages' device")
        return 1.0, 1.0, multipliers
    return float(multipliers[0]), float(multipliers[1]), None


def _page_dtype(pages, kind):
    if KINDS[kind] == 0:
        want = torch.float16 if kind == "fp16" else torch.bfloat16
        if pages.dtype != want:
            raise ValueError(f"{kind} pages are {want}, not {pages.dtype}")
        return _abi.F16 if kind == "fp16" else _abi.BF16
    return _abi.BF16


_cu_count = {}


def _cus(device):
    found = _cu_count.get(device)
    if found is None:
        found = _cu_count[device] = torch.cuda.get_device_properties(device).multi_processor_count
    return found


# -- the split's order knobs -----------------------------------------------------------------------------------------------
def _tuned(name, head_dim, value_dim, kv_heads, kind):
    """The engine's tuned value of an order knob of the split launch (the "split" structure, keyed by the cache's
    geometry as the reference keys it, __init__.py:262-286), 0 where it has none."""
    if _crit_tuning is None or head_dim is None or kv_heads is None:
        return 0
    # (a cache described by its key width alone has values of that width: the reference's _split_key, __init__.py:255-257)
    key = {"D": int(head_dim), "DV": int(value_dim or head_dim), "HKV": int(kv_heads), "KIND": KINDS[kind]}
    return int(_crit_tuning.knobs("split", key, 1).get(name, 0) or 0)


def partitions(device, kv_heads, kind, head_dim=None, value_dim=None):
    """The partition count for a cache of `kv_heads` heads on `device`: the tuning's PARTS, else about two workgroups
    per compute unit for one long row, a workgroup serving two KV heads (a power of two within 8..64; partitions past
    a launch's page tables are never launched, so a large count costs short rows nothing). A column's bits depend on
    it: one count per cache."""
    if kind not in KINDS:
        raise ValueError(f"{kind!r} is no page kind ({', '.join(KINDS)})")
    tuned = _tuned("PARTS", head_dim, value_dim, kv_heads, kind)
    if tuned:
        return tuned
    programs = 2 * _cus(torch.device(device))
    wanted = max(1, programs // max(1, int(kv_heads) // 2))
    return max(8, min(64, 1 << (wanted - 1).bit_length()))


def piece_size(head_dim, value_dim, kind="bf16", kv_heads=None):
    """Positions per piece: 64 Ki head values for 16-bit pages (512 positions at 128-wide heads, and at 64-wide ones,
    which are read in pairs), 192 Ki for 8-bit ones (1,536), within 256..2048, a multiple of 16. Measured on MI355X: the smallest pieces large batches still stream at
    their best rate with (a unit's fixed costs are hidden behind the next unit's rows), so a batch that does not fill
    the chip is cut into as many units as that allows; the tuning's PIECE where the engine has one for the cache's
    geometry (an engine of small batches gains from shorter pieces: 4 rows of 2,000 positions over FP8 pages take 36 us
    a layer at 1,536 and 19 us at 256). A column's bits depend on it; it follows the cache's geometry
    and page kind only."""
    if kind not in KINDS:
        raise ValueError(f"{kind!r} is no page kind ({', '.join(KINDS)})")
    tuned = _tuned("PIECE", head_dim, value_dim, kv_heads, kind)
    if tuned:
        return tuned
    values = 65536 if KINDS[kind] == 0 else 196608
    width = max(int(head_dim), int(value_dim))
    if width == 64:
        width = 128      # (64-wide heads are read in pairs, as 128-wide ones: measured 66 % of the HBM peak at 512 positions, 62 % at 1,024)
    return max(256, min(2048, values // width // 16 * 16))


def tile_for(columns, group, capability, fused=False):
    """(rows, waves, stages) of a window launch's query tile: up to MAX_QUERY_ROWS rows of the flattened (column, group
    head) list in a workgroup of four wavefronts, two steps in flight. rows // group never exceeds `columns`, so a
    launch keeps the width its rows have."""
    rows = max(1, min(int(columns) * int(group), MAX_QUERY_ROWS))
    return rows, 4, 2


def workspace_floats(tokens, heads, partitions, value_dim):
    """FP32 floats of the partials a launch needs for `tokens` partial rows."""
    return tokens * heads * partitions * (value_dim + 2)


def _workspace(device, tokens, heads, parts, dv, given=None):
    """(partial outputs, maxima, sums) of a split launch: three views of the caller's FP32 workspace, or of the one the
    current owner holds on the device."""
    states = tokens * heads * parts
    floats = states * (dv + 2)
    if given is None:
        given = _grown(_holding(device), "partials", floats, device, 4096 * (dv + 2),
                       "attend: run a launch of this size once before capturing it")
    elif given.dtype != torch.float32 or not given.is_contiguous() or given.numel() < floats:
        raise ValueError(f"workspace: {floats} contiguous FP32 floats for this launch (workspace_floats()), "
                         f"{given.numel()} given")
    outs, rest = given[:states * dv], given[states * dv:]
    return outs, rest[:states], rest[states:2 * states]


# -- writes ----------------------------------------------------------------------------------------------------------------
def write(keys, values, slots, key_pages, value_pages, kind, key_scales=None, value_scales=None,
          multipliers=(1.0, 1.0), *, rope=None, norm=None):
    """A step's keys [tokens][kv_heads][dim] and values [tokens][kv_heads][value_dim] (FP32, BF16 or FP16) into their
    slots ([tokens] int64; a slot below 0 is skipped) of one layer's pages (any view whose storage is
    [slots][kv_heads][dim]), encoded for the page kind, in one launch; the bytes torch's own casts would store
    (x.float() / multiplier clamped to +-448 then E4M3 for "fp8"; the row rules for "fp8:row" and "int8", their scales
    written beside the codes). values and value_pages None: keys only. keys and key_pages None: values only.
    rope (no counterpart in the reference's write: the rope() its model plugins call on the keys just before,
    inference/fused-norms/code/torch_norms.py:89-147, fused into this launch): (table, positions) or (table, positions,
    style, scale): table FP32 [rows][dim] (cos of every pair, then sin), positions [tokens] int64 (clamped to the table's
    rows), style "half" (pairs j, j + dim / 2) or "interleaved" (2j, 2j + 1), scale on cos and sin; the keys go in as
    rope() would have returned them in their own dtype. Head widths 64, 128, 256 (values wider than the keys go in a
    second launch).
    norm, with rope: (weight, eps) or (weight, eps, offset): each key head's RMS norm in front of the rotation, the
    reference's rms_norm_rope() (torch_norms.py:149-176; what rms_norm_rope_pair does to the keys, blocks.py:160-170)
    fused in as well: x / sqrt(mean(x^2) + eps) * (weight + offset) in FP32, rotated in FP32, rounded once to the keys'
    dtype. weight: [dim], any float dtype (read as FP32)."""
    if keys is None:
        if rope is not None:
            raise ValueError("rope rotates keys")
        if values is None:
            raise ValueError("write takes keys, values or both")
        if torch.is_tensor(multipliers):
            multipliers = torch.stack([multipliers[1], multipliers[1]])
        else:
            multipliers = (multipliers[1], multipliers[1])
        return write(values, None, slots, value_pages, None, kind, value_scales, None, multipliers=multipliers)
    k_kind = _check_kind(kind, key_scales)
    _require_device(keys, "write's keys")
    T, hkv, d = keys.shape
    if T == 0:
        return
    if rope is not None and values is not None and values.shape[-1] > d:
        # (the rotating launch lays a row over the lanes of the wider of the two widths, and a key's partner lanes are
        # counted in its own: values wider than the keys go in a launch of their own, the same bytes)
        write(keys, None, slots, key_pages, None, kind, key_scales, None, multipliers=multipliers, rope=rope, norm=norm)
        return write(None, values, slots, None, value_pages, kind, None, value_scales, multipliers=multipliers)
    if keys.dtype not in _DTYPE:
        keys = keys.float()
    if keys.stride(-1) != 1:
        keys = keys.contiguous()
    if values is not None:
        if values.dtype != keys.dtype:
            values = values.to(keys.dtype)
        if values.stride(-1) != 1:
            values = values.contiguous()
        if value_pages is None or (k_kind >= 2 and value_scales is None):
            raise ValueError("values come with their pages (and their scales for fp8:row and int8)")
    if slots.dtype != torch.int64 or not slots.is_contiguous():
        slots = slots.to(torch.int64).contiguous()
    if not key_pages.is_contiguous() or (value_pages is not None and not value_pages.is_contiguous()):
        raise ValueError("a layer's pages are contiguous ([slots][kv_heads][dim] storage)")
    km, vm, per_head = _multipliers(multipliers, hkv, keys.device)
    p = _abi.WriteParams()
    p.keys, p.values, p.slots = keys.data_ptr(), _ptr(values), slots.data_ptr()
    p.key_pages, p.value_pages = key_pages.data_ptr(), _ptr(value_pages)
    p.key_scales, p.value_scales = _ptr(key_scales), _ptr(value_scales)
    p.head_multipliers = _ptr(per_head)
    p.tokens = T
    p.key_stride_t, p.key_stride_h = keys.stride(0), keys.stride(1)
    if values is not None:
        p.value_stride_t, p.value_stride_h = values.stride(0), values.stride(1)
    p.kv_heads, p.head_dim = hkv, d
    p.value_dim = values.shape[-1] if values is not None else 0
    p.kind, p.page_dtype, p.in_dtype = k_kind, _page_dtype(key_pages, kind), _DTYPE[keys.dtype]
    p.key_multiplier, p.value_multiplier = km, vm
    if rope is not None:
        if not 2 <= len(rope) <= 4:
            raise ValueError("rope is (table, positions), with a style and a scale if not half and 1")
        table, positions, style, scale = tuple(rope) + ("half", 1.0)[len(rope) - 2:]
        if style not in ("half", "interleaved"):
            raise ValueError(f"rope's style is half or interleaved, not {style!r}")
        if not torch.is_tensor(table) or table.dtype != torch.float32 or table.dim() != 2 or table.shape[1] != d or \
                table.shape[0] < 1 or not table.is_contiguous() or table.device != keys.device:
            raise ValueError(f"rope's table is a contiguous FP32 [rows][{d}] tensor (cos, then sin) on the keys' device")
        if not torch.is_tensor(positions) or positions.dtype != torch.int64 or tuple(positions.shape) != (T,) or \
                not positions.is_contiguous() or positions.device != keys.device:
            raise ValueError(f"rope's positions are a contiguous int64 [{T}] tensor on the keys' device")
        if d not in (64, 128, 256):
            raise ValueError("rope in the append takes head widths 64, 128 and 256")
        p.rope_table, p.rope_positions, p.rope_rows = table.data_ptr(), positions.data_ptr(), table.shape[0]
        p.rope_interleaved, p.rope_scale = int(style == "interleaved"), float(scale)
    if norm is not None:
        if rope is None:
            raise ValueError("norm is the RMS norm in front of the keys' rotation: it comes with rope")
        if not 2 <= len(norm) <= 3:
            raise ValueError("norm is (weight, eps) or (weight, eps, offset)")
        weight, eps, offset = tuple(norm) + (0.0,)[len(norm) - 2:]
        if not torch.is_tensor(weight) or tuple(weight.shape) != (d,) or weight.device != keys.device or \
                not weight.is_floating_point():
            raise ValueError(f"norm's weight is a float [{d}] tensor on the keys' device")
        if weight.dtype != torch.float32 or not weight.is_contiguous() or weight.data_ptr() % 16:
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("paged_kv_attention.write: a captured append takes norm's weight as contiguous FP32")
            weight = weight.float().contiguous().clone()
        p.norm_weight, p.norm_eps, p.norm_offset = weight.data_ptr(), float(eps), float(offset)
    _launch(keys.device, "crit_pkv_write", "paged_kv_attention.write", p)


# -- windows ---------------------------------------------------------------------------------------------------------------
FLASH_CHUNK = 1024        # positions a split of a contiguous-split launch over a cache (flash_chunk's rule)


def flash_block(head_dim, value_dim, heads, kv_heads, page, kind="bf16"):
    """Positions a wavefront's step covers (the granule a chunk is a multiple of): four loads of 64 / (dim / 8) rows."""
    return 4 * (64 // max(1, max(int(head_dim), int(value_dim)) // 8)) if max(head_dim, value_dim) <= 512 else 4


def flash_chunk(head_dim, value_dim, heads, kv_heads, page, kind="bf16"):
    """Positions a split of every contiguous-split launch over a cache of this geometry: FLASH_CHUNK, a multiple of
    the block. A column's bits depend on it: one per cache."""
    block = flash_block(head_dim, value_dim, heads, kv_heads, page, kind)
    return max(block, FLASH_CHUNK // block * block)


def flash_parts(positions, chunk):
    """Splits a contiguous-split launch's partial row takes over page tables holding `positions` positions a row."""
    return max(1, -(-int(positions) // int(chunk)))


def flash_tile(head_dim, value_dim, heads, kv_heads, page, kind, capability):
    return MAX_QUERY_ROWS, 4


# The reference's hand-written CUDA tile has no counterpart of its own here: reader "cuda" runs the same contiguous-split
# kernels as reader "flash".
cuda_block, cuda_chunk = flash_block, flash_chunk


def cuda_ramp(*args, **kwargs):
    return (1, 0)


def cuda_splits(*args, **kwargs):
    return 1


def cuda_parts(head_dim, value_dim, heads, kv_heads, page, kind, positions, chunk=None, ramp=None):
    chunk = chunk or cuda_chunk(head_dim, value_dim, heads, kv_heads, page, kind)
    return flash_parts(positions, chunk)


def cuda_prompt(head_dim, value_dim, dtype, kind, device):
    """Whether the CUDA flash prompt chunk serves a pool: never (prompt chunks go through prefill())."""
    return False


def attend(q, key_pages, value_pages, kind, tables, rows, starts, firsts, columns, page, *, counts=None,
           offsets=None, tokens=None, key_scales=None, value_scales=None, multipliers=(1.0, 1.0), scale=None,
           partitions=None, parents=None, blocks=None, block_size=None, out=None, lse=None, workspace=None, piece=None,
           fused=False, fresh=None, vsplit=None, tile=None, num_warps=None, num_stages=None, maxnreg=None,
           flash=False, chunk=None, ramp=None, sinks=None, sliding=0, derive=None, phases=0, static=False,
           int8_qk=False):
    """Decode and verify windows over paged KV (see the module's description).

    q [tokens][heads][dim] BF16 or FP16 (FP16 for "fp16" pages); key_pages/value_pages one layer's pages, key_scales/
    value_scales their scales for "fp8:row" and "int8"; tables [S][width] int32 page tables; rows [R] int32 (or int64: a round's slots as they are) the table
    row of each batch row; starts [R] int32 its first token in q; firsts [R] int64 its column 0's position; counts [R]
    int32 its columns (None: `columns` each; more than `columns` read as `columns`); columns the widest row
    (<= MAX_COLUMNS), a Python int. offsets [R] int32 and tokens: each row's first partial row and the partial rows
    the launch takes from offsets[0] on. Writes out [tokens][heads][value_dim] (BF16, FP16 or FP32; q's dtype when
    not given) at the rows' tokens, and lse [tokens][heads] FP32 when given; returns out. workspace: an FP32 tensor of
    workspace_floats(partial rows, heads, partitions, value_dim) or more (default: one the module keeps per device and
    owner, grown outside a capture). fused: one launch folds every partition itself, the same bits, no workspace.
    flash (True or "cuda"): contiguous splits of `chunk` positions (default flash_chunk()), one per partition.
    sinks: FP32 [heads] sink logits folded into each row's final state; sliding: a sliding window in positions.
    multipliers: an "fp8" layer's (key, value) multipliers, or a [2][kv_heads] FP32 tensor (one per KV head).
    parents: draft trees, one int32 or int64 per token of q: its parent's column in its row's window, -1 for none,
    parents before children; a column then sees every position below its row's first and, of the window, its ancestors'
    positions and its own (a chain -1, 0, 1, ... is the plain causal window, bit for bit).
    blocks [tokens][k] int32 and block_size: each token's list of KV block ids (block_size positions each, -1 for none,
    no id twice): the token sees, of its positions, only those of its listed blocks, and only they are read (a list is
    one run of k x block_size positions cut into pieces and partitions; up to MAX_LISTED_BLOCKS ids; not with fused,
    flash or sliding). fresh: (keys [N][kv_heads][dim], values [N][kv_heads][value_dim] in q's dtype, shift, first):
    each row's positions from `first` on are read from those rows instead of the pages (row = position - shift; a
    prompt chunk's own keys and values as the projections gave them, unscaled), shift and first int64 device tensors
    of one element a row, or of one element for every row; not with block lists; such launches take the generic
    kernel, split or fused, the same bits either way. derive: a Derive (or the tuple (weight, eps, freqs, rotary_dim)):
    the keys derived from the value pages on read (key_pages None: the layer keeps value rows only), k = rope(rms_norm(r)
    * weight, position) in FP32 from the row as stored; any head width and any even rotary width up to it; not
    with block lists, fresh keys or flash. int8_qk (INT8 pages, fused launches; what prefill passes for the chunks it
    reads as window rows): the queries as INT8 codes at each row's own scale, a page position's score the exact
    product of the codes times both scales. phases (a measurement's): 1 runs the split
    launch only, 2 the merge only. static: the launch takes its partials and counters from the library's static device
    array (crit_pkv_attend_static: for callers that cannot allocate; the same bits; launches that overlap on one GPU
    race there; refused past _abi.STATIC_SCRATCH_BYTES of partials); no workspace is read."""
    if derive is not None:
        if flash:
            raise ValueError("derive= reads keys from the value rows on the split and fused launches and prefill's "
                             "default one: the flash structures (flash=True, flash='cuda') take key pages")
        if blocks is not None:
            raise ValueError("derive= reads windows without block lists")
        if key_pages is not None:
            raise ValueError("derive= reads the value pages as keys too: key_pages None")
        if fresh is not None and fresh[0] is not None:
            raise ValueError("derive= derives the fresh rows' keys from their values too: fresh keys None")
        key_pages = value_pages
    if parents is not None:
        _require_device(parents, "attend's parents")
        parents = parents.reshape(-1)
        if parents.dtype not in (torch.int32, torch.int64) or parents.stride(0) != 1 or parents.numel() < q.shape[0]:
            raise ValueError("parents holds one int32 or int64 parent column per token of q, contiguous")
        if int(columns) > 64:
            raise ValueError("a draft tree's row has at most 64 columns (a column's ancestors are a 64-bit set)")
    if blocks is not None:
        _require_device(blocks, "attend's blocks")
        if fused:
            raise ValueError("a fused launch reads windows without block lists")
        if not block_size or int(block_size) < 1:
            raise ValueError("block-sparse attention takes the blocks' size in positions")
        if blocks.dtype != torch.int32 or blocks.dim() != 2 or blocks.shape[0] < q.shape[0]:
            raise ValueError("blocks holds one list of int32 KV block ids per token of q: [tokens][k]")
        if not 1 <= blocks.shape[1] <= MAX_LISTED_BLOCKS:
            raise ValueError(f"a token lists 1 .. {MAX_LISTED_BLOCKS} blocks, not {blocks.shape[1]}")
        if blocks.stride(-1) != 1:
            blocks = blocks.contiguous()
        flash = False      # (block lists: the split launch, as in the reference)
    if fresh is not None and blocks is not None:
        raise ValueError("fresh rows are not read through block lists")
    k_kind = _check_kind(kind, value_scales if derive is not None else key_scales)
    if int8_qk:
        if k_kind != 3:
            raise ValueError("int8_qk multiplies INT8 queries with INT8 keys: int8 pages only")
        if derive is not None or blocks is not None or flash or not fused:
            raise ValueError("int8_qk reads windows in the fused launch, without block lists, derived keys or flash")
    _require_device(q, "attend's q")
    T, hq, d = q.shape
    derived, has_weight = (None, False) if derive is None else _derived(derive, d, q.device)
    if derived is not None and d != value_pages.shape[-1]:
        raise ValueError("derive= reads one row as key and value: one head width")
    _check_sinks(sinks, q)
    sliding = _check_sliding(sliding, blocks)
    hkv, dv = key_pages.shape[-2], value_pages.shape[-1]
    R = int(starts.shape[0])
    if hq % hkv or not 1 <= columns <= MAX_COLUMNS or R == 0:
        raise ValueError("query heads a multiple of the KV heads, 1..64 columns a row, one row or more")
    if q.stride(-1) != 1:
        raise ValueError("q's last dimension is contiguous")
    if d not in HEAD_WIDTHS or dv not in HEAD_WIDTHS or key_pages.shape[-1] != d:
        raise ValueError(f"head widths are powers of two from 16 to 256 (q's, keys' and values'), not {d} and {dv}")
    want_q = torch.float16 if kind == "fp16" else torch.bfloat16
    if q.dtype != want_q:
        raise ValueError(f"q is {want_q} over {kind} pages, not {q.dtype}")
    if (offsets is None) != (tokens is None):
        raise ValueError("offsets come with the partial rows they take (tokens)")
    if tables.dtype != torch.int32 or tables.stride(-1) != 1 or rows.dtype not in (torch.int32, torch.int64) or \
            starts.dtype != torch.int32 or firsts.dtype != torch.int64:
        raise ValueError("tables and starts are int32, rows int32 or int64 and firsts int64")
    if counts is not None and counts.dtype != torch.int32 or offsets is not None and offsets.dtype != torch.int32:
        raise ValueError("counts and offsets are int32")
    partial_rows = R * columns if offsets is None else int(tokens)
    device = q.device
    if key_pages.device != device or value_pages.device != device or tables.device != device:
        raise ValueError("q, the pages and the page tables live on one device")
    block = flash_block(d, dv, hq, hkv, page, kind)
    if flash:
        piece = int(chunk or flash_chunk(d, dv, hq, hkv, page, kind))
        if piece % block:
            raise ValueError(f"a contiguous split ({piece} positions) is a multiple of the block ({block})")
        parts = flash_parts(tables.shape[1] * page, piece)
    else:
        parts = int(partitions or globals()["partitions"](device, hkv, kind, d, dv))
        piece = int(piece or piece_size(d, dv, kind, hkv))
        if piece < 1:
            raise ValueError(f"a piece is a number of positions, not {piece}")
        # A piece is a whole number of the wavefronts' steps: one that is not (crit's piece option admits 16 to 128,
        # a step at narrow heads is up to 128 positions) is read as the next multiple. Still one piece per cache.
        piece = -(-piece // block) * block
    scale = float(scale if scale is not None else d ** -0.5)
    if fused or static:
        po = pm = pl = None
    else:
        po, pm, pl = _workspace(device, partial_rows, hq, parts, dv, workspace)
    if out is None:
        out = torch.empty(T, hq, dv, dtype=q.dtype, device=device)
    if out.dtype not in _DTYPE or out.stride(-1) != 1 or out.shape[-1] != dv:
        raise ValueError("out is [tokens][heads][value_dim] BF16, FP16 or FP32, its last dimension contiguous")
    if lse is not None and (lse.dtype != torch.float32 or not lse.is_contiguous()):
        raise ValueError("lse is contiguous FP32 [tokens][heads]")
    km, vm, per_head = _multipliers(multipliers, hkv, device)
    p = _abi.AttendParams()
    p.q, p.key_pages, p.value_pages = q.data_ptr(), key_pages.data_ptr(), value_pages.data_ptr()
    p.key_scales, p.value_scales, p.head_multipliers = _ptr(key_scales), _ptr(value_scales), _ptr(per_head)
    if derived is not None:
        p.key_pages = p.key_scales = None
        p.derive_table, p.derive_eps = derived.table.data_ptr(), derived.eps
        p.derive_rot, p.derive_weighted = derived.rotary_dim, int(has_weight)
    p.tables, p.rows, p.starts, p.counts = tables.data_ptr(), rows.data_ptr(), starts.data_ptr(), _ptr(counts)
    p.rows_are_64 = int(rows.dtype == torch.int64)
    p.firsts, p.offsets = firsts.data_ptr(), _ptr(offsets)
    p.partial_out, p.partial_max, p.partial_sum = _ptr(po), _ptr(pm), _ptr(pl)
    p.out, p.lse, p.sinks = out.data_ptr(), _ptr(lse), _ptr(sinks)
    if parents is not None:
        p.parents, p.parents64 = (parents.data_ptr(), None) if parents.dtype == torch.int32 else (None, parents.data_ptr())
    if blocks is not None:
        p.blocks, p.blocks_stride = blocks.data_ptr(), blocks.stride(0)
        p.blocks_k, p.block_size = int(blocks.shape[1]), int(block_size)
    p.q_stride_t, p.q_stride_h, p.out_stride_t, p.out_stride_h = q.stride(0), q.stride(1), out.stride(0), out.stride(1)
    p.table_stride, p.table_width = tables.stride(0), tables.shape[1]
    p.n_rows, p.columns, p.heads, p.kv_heads, p.head_dim, p.value_dim, p.page = R, int(columns), hq, hkv, d, dv, int(page)
    p.kind, p.page_dtype, p.out_dtype = k_kind, _page_dtype(key_pages, kind), _DTYPE[out.dtype]
    p.partitions, p.piece, p.fused, p.sliding, p.phases = parts, piece, int(bool(fused)), sliding, int(phases)
    p.scale, p.key_multiplier, p.value_multiplier = scale, km, vm
    p.int8_qk = int(bool(int8_qk))
    if fresh is not None:
        fk, fv, fshift, ffirst = fresh
        if derive is not None:      # (checked as the keys the values stand for: one width)
            fk = fv
        if not (torch.is_tensor(fk) and torch.is_tensor(fv)) or fk.dim() != 3 or fk.shape[1:] != (hkv, d) or \
                fv.shape[1:] != (hkv, dv) or fk.shape[0] != fv.shape[0] or fk.shape[0] < 1 or fk.stride(-1) != 1 or \
                fv.stride(-1) != 1 or fk.stride(1) != d or fv.stride(1) != dv or not torch.is_tensor(fshift) or \
                not torch.is_tensor(ffirst) or fshift.numel() != ffirst.numel() or fshift.numel() not in (1, R):
            raise ValueError(f"fresh rows are [N][{hkv}][dim] each, head rows contiguous, with one shift and first "
                             "a row or one for every row")
        if fk.dtype != q.dtype or fv.dtype != q.dtype or fk.device != device or fv.device != device:
            raise ValueError("fresh rows in q's dtype on q's device")
        if fshift.dtype != torch.int64 or ffirst.dtype != torch.int64 or fshift.device != device or \
                ffirst.device != device or not fshift.is_contiguous() or not ffirst.is_contiguous():
            raise ValueError("a fresh row's shift and first are contiguous int64 tensors on q's device")
        if fk.stride(0) % 8 or fv.stride(0) % 8 or fk.data_ptr() % 16 or fv.data_ptr() % 16:
            raise ValueError("fresh rows 16-byte aligned, their token stride a multiple of 8 elements")
        p.fresh_keys, p.fresh_values = None if derive is not None else fk.data_ptr(), fv.data_ptr()
        p.fresh_shifts, p.fresh_firsts = fshift.data_ptr(), ffirst.data_ptr()
        p.fresh_stride_k, p.fresh_stride_v, p.fresh_rows = fk.stride(0), fv.stride(0), int(fk.shape[0])
        p.fresh_per_row = int(fshift.numel() != 1)
    if static:
        _launch(device, "crit_pkv_attend_static", "paged_kv_attention.attend", p)
        return out
    stream = _stream_of(device)
    p.launch_state = _launch_state(device, stream)
    _launch(device, "crit_pkv_attend", "paged_kv_attention.attend", p, stream=stream)
    return out


def merge_shards(outs, lses):
    """Partials of the same queries over disjoint keys (outs [parts][tokens][heads][dim], lses [parts][tokens][heads]
    FP32, -inf for a part with no key) -> (out FP32, lse FP32), the parts weighted by exp(lse - max): the device twin
    of the partitioned-attention plugin's merge() (reference inference/partitioned-attention/plugin.py:52-64). A token
    no part saw gets zeros and -inf. Not part of the reference module's interface."""
    outs = outs if torch.is_tensor(outs) else torch.stack(list(outs))
    lses = lses if torch.is_tensor(lses) else torch.stack(list(lses))
    _require_device(outs, "merge_shards' outs")
    if outs.dtype not in _DTYPE:
        outs = outs.float()
    outs, lses = outs.contiguous(), lses.float().contiguous()
    parts, tokens, heads, dim = outs.shape
    out = torch.empty(tokens, heads, dim, dtype=torch.float32, device=outs.device)
    lse = torch.empty(tokens, heads, dtype=torch.float32, device=outs.device)
    p = _abi.MergeParams()
    p.outs, p.lses, p.out, p.lse = outs.data_ptr(), lses.data_ptr(), out.data_ptr(), lse.data_ptr()
    p.rows, p.parts, p.value_dim, p.in_dtype = tokens * heads, parts, dim, _DTYPE[outs.dtype]
    _launch(outs.device, "crit_pkv_merge", "paged_kv_attention.merge_shards", p)
    return out, lse


# -- prompt chunks -----------------------------------------------------------------------------------------------------------
def prefill_state_floats(tokens, heads, dim):
    """FP32 floats of the scratch a prompt launch with fresh rows hands its rows' states through (prefill's and
    prefill_rows' workspace=), for q of `tokens` rows."""
    return tokens * heads * (dim + 4)


def _prefill_state(device, tokens, heads, dim, given):
    need = prefill_state_floats(tokens, heads, dim)
    if given is None:
        return _grown(_holding(device), "states", need, device, 1 << 16,
                      "prefill: run a chunk of this size with fresh rows once before capturing it, or pass workspace=")
    if given.dtype != torch.float32 or given.numel() < need or not given.is_contiguous() or given.device != device \
            or given.data_ptr() % 16:
        raise ValueError(f"a prompt chunk with fresh rows needs {need} contiguous FP32 floats of workspace on its "
                         "device, 16-byte aligned (prefill_state_floats)")
    return given


def _check_fresh(fresh, q, hkv, d, chunks, derived=False):
    """(keys, values, firsts or None) of a prompt launch's fresh rows, checked as the reference checks them
    (__init__.py:1301-1308): [tokens][kv_heads][dim] each in q's dtype, head rows contiguous. derived: the keys are
    derived from the values (keys None)."""
    fk, fv, firsts = fresh
    T = q.shape[0]
    if derived and fk is not None:
        raise ValueError("derive= derives the fresh rows' keys from their values too: fresh keys None")
    for name, x in ((("values", fv),) if derived else (("keys", fk), ("values", fv))):
        if not torch.is_tensor(x) or x.shape != (T, hkv, d) or x.stride(-1) != 1 or x.stride(1) != d:
            raise ValueError(f"fresh keys and values are [{T}][{hkv}][{d}], each head row contiguous")
        if x.dtype != q.dtype or x.device != q.device:
            raise ValueError("fresh rows in q's dtype on q's device")
        if x.stride(0) % 8 or x.data_ptr() % 16:
            raise ValueError("fresh rows 16-byte aligned, their token stride a multiple of 8 elements")
    if firsts is not None and (not torch.is_tensor(firsts) or firsts.dtype != torch.int64 or firsts.device != q.device
                               or firsts.numel() != chunks or not firsts.is_contiguous()):
        raise ValueError("the first fresh positions are int64, one a chunk, on q's device")
    return fk, fv, firsts


def _prefill_launch(q, key_pages, value_pages, kind, tables, table_rows, starts, counts, positions, max_count, chunks,
                    page, key_scales, value_scales, multipliers, scale, out, lse, sinks, sliding, fresh=None,
                    workspace=None, int8_qk=False):
    k_kind = _check_kind(kind, key_scales)
    if int8_qk and k_kind != 3:
        raise ValueError("int8_qk multiplies INT8 queries with INT8 keys: int8 pages only")
    _require_device(q, "prefill's q")
    T, hq, d = q.shape
    hkv = key_pages.shape[-2]
    if value_pages.shape[-1] != d:
        raise ValueError("prompt chunks read keys and values of one width")
    if hq % hkv or q.stride(-1) != 1:
        raise ValueError("query heads a multiple of the KV heads, q's last dimension contiguous")
    want_q = torch.float16 if kind == "fp16" else torch.bfloat16
    if q.dtype != want_q:
        raise ValueError(f"q is {want_q} over {kind} pages, not {q.dtype}")
    device = q.device
    if d not in (64, 128, 256) or (d == 256 and k_kind == 3):      # (INT8 pages at 256 would spill: window rows)
        return _prefill_as_windows(q, key_pages, value_pages, kind, tables, table_rows, starts, counts, positions,
                                   max_count, chunks, page, key_scales, value_scales, multipliers, scale, out, lse,
                                   sinks, sliding, fresh, int8_qk)
    out = torch.empty_like(q) if out is None else out
    if out.dtype not in _DTYPE or out.stride(-1) != 1:
        raise ValueError("out is [tokens][heads][dim] BF16, FP16 or FP32, its last dimension contiguous")
    if lse is not None and (lse.dtype != torch.float32 or lse.stride(-1) != 1 or lse.stride(0) != hq):
        raise ValueError("lse is contiguous FP32 [tokens][heads]")
    km, vm, per_head = _multipliers(multipliers, hkv, device)
    p = _abi.PrefillParams()
    p.q, p.key_pages, p.value_pages = q.data_ptr(), key_pages.data_ptr(), value_pages.data_ptr()
    p.key_scales, p.value_scales, p.head_multipliers = _ptr(key_scales), _ptr(value_scales), _ptr(per_head)
    if tables.dtype == torch.int32:
        p.tables = tables.data_ptr()
    elif tables.dtype == torch.int64:
        p.tables64 = tables.data_ptr()
    else:
        raise ValueError("a page table is int32 or int64")
    p.table_rows, p.starts, p.counts, p.positions = _ptr(table_rows), _ptr(starts), _ptr(counts), positions.data_ptr()
    p.out, p.lse, p.sinks = out.data_ptr(), _ptr(lse), _ptr(sinks)
    p.q_stride_t, p.q_stride_h, p.out_stride_t, p.out_stride_h = q.stride(0), q.stride(1), out.stride(0), out.stride(1)
    p.table_stride = tables.stride(0) if tables.dim() == 2 else 0
    p.table_width = tables.shape[-1]
    p.chunks, p.max_count, p.heads, p.kv_heads, p.head_dim, p.page = chunks, max_count, hq, hkv, d, int(page)
    p.kind, p.page_dtype, p.out_dtype = k_kind, _page_dtype(key_pages, kind), _DTYPE[out.dtype]
    p.sliding = sliding
    p.scale = float(scale if scale is not None else d ** -0.5)
    p.key_multiplier, p.value_multiplier = km, vm
    p.int8_qk = int(bool(int8_qk))
    if fresh is not None:
        fk, fv, firsts = _check_fresh(fresh, q, hkv, d, chunks)
        state = _prefill_state(device, T, hq, d, workspace)
        p.fresh_keys, p.fresh_values, p.fresh_firsts, p.fresh_state = fk.data_ptr(), fv.data_ptr(), _ptr(firsts), state.data_ptr()
        p.fresh_stride_k, p.fresh_stride_v = fk.stride(0), fv.stride(0)
    _launch(device, "crit_pkv_prefill", "paged_kv_attention.prefill", p)
    return out


def _prefill_as_windows(q, key_pages, value_pages, kind, tables, table_rows, starts, counts, positions, max_count,
                        chunks, page, key_scales, value_scales, multipliers, scale, out, lse, sinks, sliding, fresh,
                        int8_qk, derive=None):
    """Prompt chunks at the head widths the matrix-core kernel does not take (16, 32; 256 over INT8 pages), and those whose keys are
    derived from the value rows: every chunk cut into window
    rows of up to MAX_COLUMNS tokens and read by attend()'s fused launch, as crit itself reads prompt rows with
    prompt_reader decode (device_attention.py:751-783). The rows' metadata is computed on the device from the chunks'
    (no length is read on the host)."""
    device, hq = q.device, q.shape[1]
    if q.shape[-1] not in HEAD_WIDTHS:
        raise ValueError(f"head widths are powers of two from 16 to 256, not {q.shape[-1]}")
    per = -(-int(max_count) // MAX_COLUMNS)                                   # window rows a chunk
    step = torch.arange(per, dtype=torch.int64, device=device) * MAX_COLUMNS   # each one's first column in its chunk
    zero = torch.zeros(chunks, dtype=torch.int64, device=device)
    first_token = zero if starts is None else starts.to(torch.int64)
    length = torch.full((chunks,), int(max_count), dtype=torch.int64, device=device) if counts is None else counts.to(torch.int64)
    table_of = torch.arange(chunks, dtype=torch.int64, device=device) if table_rows is None else table_rows.to(torch.int64)
    w_starts = (first_token[:, None] + step[None, :]).reshape(-1).to(torch.int32)
    w_firsts = (positions[:, None] + step[None, :]).reshape(-1).contiguous()
    w_counts = (length[:, None] - step[None, :]).clamp(0, MAX_COLUMNS).reshape(-1).to(torch.int32)
    w_rows = table_of[:, None].expand(chunks, per).reshape(-1).to(torch.int32)
    given = None
    if fresh is not None:      # a chunk's own rows sit beside q's tokens: row = position - (chunk position - first token)
        fk, fv, firsts = _check_fresh(fresh, q, value_pages.shape[-2], q.shape[-1], chunks, derive is not None)
        shift = positions - first_token
        own = positions if firsts is None else torch.maximum(firsts, positions)
        given = (fk, fv, shift[:, None].expand(chunks, per).reshape(-1).contiguous(),
                 own[:, None].expand(chunks, per).reshape(-1).contiguous())
    if tables.dtype != torch.int32:
        tables = tables.to(torch.int32)
    if out is None:
        out = torch.empty(q.shape[0], hq, value_pages.shape[-1], dtype=q.dtype, device=device)
    return attend(q, key_pages, value_pages, kind, tables, w_rows, w_starts, w_firsts, MAX_COLUMNS, page,
                  counts=w_counts, key_scales=key_scales, value_scales=value_scales, multipliers=multipliers,
                  scale=scale, out=out, lse=lse, fused=True, fresh=given, sinks=sinks, sliding=sliding, derive=derive,
                  int8_qk=int8_qk)


def prefill(q, key_pages, value_pages, kind, table, position, page, *, key_scales=None, value_scales=None,
            multipliers=(1.0, 1.0), scale=None, out=None, lse=None, int8_qk=False, fresh=None, flash=False,
            sinks=None, sliding=0, splits=None, workspace=None, derive=None):
    """A prompt chunk of one sequence: q [T][heads][dim] at positions position.. (their keys and values written),
    table [pages] int32 or int64 -> out [T][heads][dim] (and lse [T][heads] FP32 when given), causal. position: an
    int, or a one-element int64 device tensor read on the device. One matrix-core launch whatever `flash` says; a
    token's bits follow its own positions only. fresh: (keys, values) [T][kv_heads][dim] in q's dtype, the chunk's own
    as the projections gave them, or (keys, values, first): the chunk reads its own positions from `first` on (default:
    all of them; an int or a one-element int64 device tensor, clamped to the chunk's positions) from them, unscaled,
    and the earlier ones from the pages: two launches (the pages' positions, then the fresh rows) that hand the rows'
    states through `workspace` (FP32, prefill_state_floats(T, heads, dim); default: one the module keeps per device,
    grown outside a capture); a token's bits follow its own positions and `first`. int8_qk (INT8 pages): each query
    row rounded to INT8 codes at its own scale (amax / 127, half away from zero) and the scores taken as exact integer
    products of the codes on the matrix cores (v_mfma_i32_32x32x32_i8) times the row's and the keys' scales; fresh rows
    are still read in q's type. derive: a Derive (or its tuple), as attend() takes it: the keys derived from the value
    pages (key_pages None); such a chunk is read as window rows of up to MAX_COLUMNS tokens by attend()'s fused launch
    (a prompt token's bits are those of the same position decoded), with fresh rows too (a chunk's own value rows, their
    keys derived the same way); not with flash or int8_qk."""
    if derive is not None:
        if flash:
            raise ValueError("derive= reads keys from the value rows on the split and fused launches and prefill's "
                             "default one: the flash structures (flash=True, flash='cuda') take key pages")
        if int8_qk:
            raise ValueError("derive= derives 16-bit keys: not with int8_qk")
        if key_pages is not None:
            raise ValueError("derive= reads the value pages as keys too: key_pages None")
    _check_sinks(sinks, q)
    sliding = _check_sliding(sliding, None)
    T = q.shape[0]
    if T == 0:
        return torch.empty_like(q) if out is None else out
    if torch.is_tensor(position):
        positions = position.reshape(1)
        if positions.dtype != torch.int64 or positions.device != q.device:
            raise ValueError("a device position is a one-element int64 tensor on q's device")
    else:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("paged_kv_attention.prefill: a captured chunk takes its position as a device tensor")
        positions = torch.tensor([int(position)], dtype=torch.int64, device=q.device)
    if fresh is not None:
        if len(fresh) not in (2, 3):
            raise ValueError("fresh is (keys, values) or (keys, values, first)")
        first = fresh[2] if len(fresh) == 3 else None
        if first is not None and not torch.is_tensor(first):
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("paged_kv_attention.prefill: a captured chunk takes its first fresh position as a "
                                   "device tensor")
            first = torch.tensor([int(first)], dtype=torch.int64, device=q.device)
        elif first is not None:
            first = first.reshape(1)
        fresh = (fresh[0], fresh[1], first)
    if derive is not None:
        return _prefill_as_windows(q, None, value_pages, kind, table.reshape(1, -1), None, None, None, positions, T, 1, page,
                                   None, value_scales, multipliers, scale, out, lse, sinks, sliding, fresh, False, derive)
    return _prefill_launch(q, key_pages, value_pages, kind, table.reshape(1, -1), None, None, None, positions, T, 1,
                           page, key_scales, value_scales, multipliers, scale, out, lse, sinks, sliding, fresh,
                           workspace, int8_qk)


def prefill_rows(q, key_pages, value_pages, kind, tables, table_rows, starts, counts, positions, max_count, page, *,
                 key_scales=None, value_scales=None, multipliers=(1.0, 1.0), scale=None, out=None, lse=None,
                 sinks=None, sliding=0, fresh=None, workspace=None, int8_qk=False):
    """Several prompt chunks in one launch (where the reference launches prefill() once per row): chunk i is counts[i]
    <= max_count tokens from token starts[i] of q at positions positions[i].. of the sequence whose page table is
    tables[table_rows[i]]; tables [S][width] int32, table_rows/starts/counts [chunks] int32, positions [chunks] int64,
    all on the device and read there. fresh: (keys, values, firsts) parallel to q's tokens as prefill() takes them,
    firsts [chunks] int64 on the device or None (every chunk's own positions). Not part of the reference module's
    interface."""
    _check_sinks(sinks, q)
    sliding = _check_sliding(sliding, None)
    chunks = int(positions.shape[0])
    if chunks == 0:
        return torch.empty_like(q) if out is None else out
    if fresh is not None:
        if len(fresh) not in (2, 3):
            raise ValueError("fresh is (keys, values) or (keys, values, firsts)")
        fresh = (fresh[0], fresh[1], fresh[2] if len(fresh) == 3 else None)
    return _prefill_launch(q, key_pages, value_pages, kind, tables, table_rows, starts, counts, positions,
                           int(max_count), chunks, page, key_scales, value_scales, multipliers, scale, out, lse, sinks,
                           sliding, fresh, workspace, int8_qk)


def stream_read(data, sink=None):
    """Reads every byte of `data` (a contiguous device tensor, a multiple of 16 bytes) once with 16-byte loads: the
    streaming-read yardstick the benchmark times beside the nominal HBM peak."""
    _require_device(data, "stream_read's data")
    nbytes = data.numel() * data.element_size()
    sink = torch.zeros(64, dtype=torch.float32, device=data.device) if sink is None else sink
    _launch(data.device, "crit_pkv_stream_read", "paged_kv_attention.stream_read", data.data_ptr(), nbytes, sink.data_ptr())
    return sink


# -- pool bookkeeping on the device (reference: inference/attention-state/code/pages.py:646-684, 861-869) ----------------
def _i64_on(t, device, what, n=None):
    if not torch.is_tensor(t) or t.dtype != torch.int64 or t.device != device or not t.is_contiguous() or \
            (n is not None and t.numel() < n):
        raise ValueError(f"{what} is a contiguous int64 tensor on the tables' device" + (f" of {n} or more" if n else ""))
    return t


def _tables(round_tables, round_capacity):
    _require_device(round_tables, "the round tables")
    if round_tables.dtype != torch.int32 or round_tables.dim() != 2 or round_tables.stride(1) != 1 or \
            round_tables.shape[0] < 1 or round_tables.shape[1] < 1:
        raise ValueError("round tables are [round slots][table pages] int32, a row contiguous")
    _i64_on(round_capacity, round_tables.device, "the round slots' capacity", round_tables.shape[0])


def _stores(p, stores, layers, slots):
    """Fills p.stores from tensors [layers][...] whose layer holds `slots` rows back to back (keys, values, scales)."""
    stores = [s for s in stores if s is not None]
    if not 1 <= len(stores) <= _abi.MAX_STORES:
        raise ValueError(f"1 to {_abi.MAX_STORES} stores (keys, values, their scales)")
    device = stores[0].device
    for i, s in enumerate(stores):
        _require_device(s, "a store")
        if s.device != device or s.dim() < 2 or s.shape[0] != layers or not s[0].is_contiguous():
            raise ValueError(f"a store is [{layers} layers][...] on one device, each layer contiguous")
        layer_bytes = s[0].numel() * s.element_size()
        if slots < 1 or layer_bytes % slots:
            raise ValueError(f"a layer of a store holds {slots} rows of one size")
        p.stores[i].base, p.stores[i].layer_stride = s.data_ptr(), s.stride(0) * s.element_size()
        p.stores[i].row_bytes = layer_bytes // slots
    p.n_stores, p.layers = len(stores), layers
    return device


def slots_at(round_tables, round_capacity, slot, positions, page, dump, *, rows=None, out=None):
    """The KV slots of `positions` of the sequences bound to round slots `slot` (any shape, both int64): KVPool._slots_at
    (pages.py:655-660) in one launch: table[min(p // page, pages - 1)] * page + p % page where 0 <= p < the slot's
    capacity, the dump page's first slot (dump * page) elsewhere. rows: `slot` holds one entry a row and rows [n] names
    each position's row (the index_select of _reserve_round, pages.py:652-653). A round slot that does not exist reads
    as one without capacity. Returns out (int64, positions' shape)."""
    _tables(round_tables, round_capacity)
    device = round_tables.device
    _i64_on(slot, device, "slots_at's slot")
    _i64_on(positions, device, "slots_at's positions")
    if rows is not None:
        _i64_on(rows, device, "slots_at's rows", positions.numel())
    elif slot.numel() != positions.numel():
        raise ValueError("one round slot a position (or rows=)")
    if out is None:
        out = torch.empty_like(positions)
    else:
        _i64_on(out, device, "slots_at's out", positions.numel())
    p = _abi.SlotsParams()
    p.round_tables, p.round_capacity, p.slots, p.rows = round_tables.data_ptr(), round_capacity.data_ptr(), slot.data_ptr(), _ptr(rows)
    p.positions, p.out, p.n, p.n_slots = positions.data_ptr(), out.data_ptr(), positions.numel(), slot.numel()
    p.round_slots, p.table_stride, p.table_pages = round_tables.shape[0], round_tables.stride(0), round_tables.shape[1]
    p.page, p.dump = int(page), int(dump)
    _launch(device, "crit_pkv_slots_at", "paged_kv_attention.slots_at", p)
    return out


def compact(stores, slots, round_tables, round_capacity, start, emitted, path, moved, page, dump):
    """An accepted draft-tree path's rows to consecutive positions, KVPool._compact (pages.py:662-684) in one launch
    over every layer and store: for round row r (round slot r) where moved[r] == 0, node path[r][j] at position
    start[r] + path[r][j] moves to start[r] + j for 0 < j < emitted[r] with path[r][j] >= 0; then moved[:rows] = 1.
    Every slot outside the dump page ends as the reference leaves it; the dump page itself is read (a node past its
    slot's capacity) and never written (what the reference leaves there is one of several rows, undefined which).
    stores: the pool's tensors [layers][...] (keys, values, row scales; None entries skipped), each layer `slots` rows;
    path [rows][width] int64 or int32 (up to 256 columns); start, emitted, moved int64 [rows or more]."""
    _tables(round_tables, round_capacity)
    device = round_tables.device
    if not torch.is_tensor(path) or path.dim() != 2 or path.dtype not in (torch.int64, torch.int32) or \
            path.device != device or path.stride(1) != 1 or not 1 <= path.shape[1] <= _abi.MAX_PATH:
        raise ValueError(f"a tree path is [rows][1 .. {_abi.MAX_PATH} columns] int64 or int32 on the tables' device")
    rows = path.shape[0]
    if rows > round_tables.shape[0]:
        raise ValueError(f"{rows} rows read round slots 0 .. {rows - 1}; the tables hold {round_tables.shape[0]}")
    if rows == 0:
        return
    p = _abi.CompactParams()
    live = [s for s in stores if s is not None]
    if not live:
        raise ValueError("compact moves the rows of one store at least")
    if _stores(p, live, live[0].shape[0], int(slots)) != device:
        raise ValueError("stores on the tables' device")
    p.round_tables, p.round_capacity = round_tables.data_ptr(), round_capacity.data_ptr()
    p.start, p.emitted = _i64_on(start, device, "start", rows).data_ptr(), _i64_on(emitted, device, "emitted", rows).data_ptr()
    p.moved, p.path = _i64_on(moved, device, "moved", rows).data_ptr(), path.data_ptr()
    p.rows, p.round_slots, p.table_stride, p.path_stride = rows, round_tables.shape[0], round_tables.stride(0), path.stride(0)
    p.width, p.path_is_32, p.table_pages, p.page, p.dump = path.shape[1], int(path.dtype == torch.int32), round_tables.shape[1], int(page), int(dump)
    _launch(device, "crit_pkv_compact", "paged_kv_attention.compact", p)


def copy_pages(stores, slots, source, target, page):
    """Pages source[i] copied to pages target[i] in every layer of every store (the copies of KVPool._copy,
    pages.py:861-869, for all of a step's shared pages at once): source, target int64 [n] on the device, a pair with a
    negative id (or one past the layer's pages) skipped; no target is another pair's source or target. stores and slots as compact() takes them."""
    live = [s for s in stores if s is not None]
    if not live:
        raise ValueError("copy_pages copies the pages of one store at least")
    p = _abi.CopyPagesParams()
    device = _stores(p, live, live[0].shape[0], int(slots))
    _i64_on(source, device, "copy_pages' source")
    _i64_on(target, device, "copy_pages' target", source.numel())
    if source.numel() == 0:
        return
    p.source, p.target, p.n, p.page = source.data_ptr(), target.data_ptr(), source.numel(), int(page)
    p.pool_pages = int(slots) // int(page)
    _launch(device, "crit_pkv_copy_pages", "paged_kv_attention.copy_pages", p)


def start_round(round_lengths, start, moved, rows):
    """A round begins, KVPool.start_round (pages.py:623-628) in one launch: start[:rows] = round_lengths[:rows] (each
    row's valid length as the round finds it) and moved[:rows] = 0 (no row's tree path moved yet; moved may be None).
    int64 tensors on one device; capture-safe."""
    _require_device(round_lengths, "the round lengths")
    device, rows = round_lengths.device, int(rows)
    if rows < 0:
        raise ValueError("a round has zero rows or more")
    p = _abi.RoundParams()
    p.round_lengths = _i64_on(round_lengths, device, "the round lengths", rows).data_ptr()
    p.start = _i64_on(start, device, "start", rows).data_ptr()
    p.moved = None if moved is None else _i64_on(moved, device, "moved", rows).data_ptr()
    p.rows, p.commit = rows, 0
    _launch(device, "crit_pkv_round", "paged_kv_attention.start_round", p)


def commit_round(round_lengths, start, emitted, frontier, *, tree=None):
    """After a round's acceptance, KVPool.commit_round (pages.py:630-644) without the host: with tree=(stores, slots,
    round_tables, round_capacity, path, moved, page, dump) the accepted draft-tree path's rows move to consecutive
    positions first (compact(), once a round); then round_lengths[r] = frontier[r] where emitted[r] > 0, start[r] (the
    length the round found) where the row emitted nothing, for r < len(emitted). A second commit from the same start
    (a truncation) finds the path moved and sets the lengths again. int64 tensors on one device; capture-safe."""
    _require_device(round_lengths, "the round lengths")
    device = round_lengths.device
    rows = _i64_on(emitted, device, "emitted").numel()
    if tree is not None:
        stores, slots, round_tables, round_capacity, path, moved, page, dump = tree
        compact(stores, slots, round_tables, round_capacity, start, emitted, path[:rows], moved, page, dump)
    p = _abi.RoundParams()
    p.round_lengths = _i64_on(round_lengths, device, "the round lengths", rows).data_ptr()
    p.start = _i64_on(start, device, "start", rows).data_ptr()
    p.emitted, p.frontier = emitted.data_ptr(), _i64_on(frontier, device, "frontier", rows).data_ptr()
    p.rows, p.commit = rows, 1
    _launch(device, "crit_pkv_round", "paged_kv_attention.commit_round", p)


class StepBuffers:
    """A pool's step buffers at fixed device addresses, as KVPool holds them (pages.py:200-217): d_slots [step_tokens]
    int64; d_rows, d_starts, d_counts, d_offsets [step_rows] int32; d_firsts [step_rows] int64; d_tables [step_rows]
    [table_pages] int32; and a StepBatch's device tensors beside them (core/python/crit_plugins/device.py:590-616):
    starts_t [step_rows + 1] int32, positions_t and rows_t [step_tokens] int64. totals [4] int64: the step's tokens,
    window rows, window tokens and whether it overflowed the buffers. Made outside a capture; step_buffers() fills them."""

    def __init__(self, step_rows, step_tokens, table_pages, dump, device):
        if step_rows < 1 or step_tokens < step_rows or table_pages < 1:
            raise ValueError("step buffers hold one row or more, a token a row or more, and tables of one page or more")
        long, int32 = dict(dtype=torch.int64, device=device), dict(dtype=torch.int32, device=device)
        self.step_rows, self.step_tokens, self.table_pages, self.dump = int(step_rows), int(step_tokens), int(table_pages), int(dump)
        self.d_slots = torch.zeros(step_tokens, **long)
        self.positions_t, self.rows_t = torch.zeros(step_tokens, **long), torch.zeros(step_tokens, **long)
        self.starts_t = torch.zeros(step_rows + 1, **int32)
        self.d_rows, self.d_starts = torch.arange(step_rows, **int32), torch.zeros(step_rows, **int32)
        self.d_counts, self.d_offsets = torch.zeros(step_rows, **int32), torch.zeros(step_rows, **int32)
        self.d_firsts = torch.zeros(step_rows, **long)
        self.d_tables = torch.full((step_rows, table_pages), dump, **int32)
        self.totals = torch.zeros(4, **long)


def step_buffers(buffers, round_tables, round_capacity, round_lengths, slot, page, window, *, counts=None, count=1,
                 firsts=None):
    """A step over sequences bound to round slots, built on the device in one launch: what StepBatch.build
    (core/python/crit_plugins/device.py:600-616), reserve()'s slots (pages.py:337-349) and KVPool._step_buffers
    (pages.py:359-397) make on the host. Row r is `counts[r]` tokens (`count` each without counts) of the sequence in
    round slot slot[r] from position firsts[r] (without firsts: round_lengths[slot[r]], the first position without KV).
    Fills `buffers` (a StepBuffers): every token's slot, position and row, the rows' first tokens, and for the rows of
    up to `window` tokens their window entries (first token, count, first position, first partial row, page table);
    entries past the window rows are emptied, so attend() over all step_rows entries reads nothing for them.
    buffers.totals says afterwards whether the step fitted (the host does not wait for it). int64 tensors on the tables'
    device; capture-safe. Returns buffers."""
    _tables(round_tables, round_capacity)
    device = round_tables.device
    rows = _i64_on(slot, device, "step_buffers' slot").numel()
    if rows > buffers.step_rows or round_tables.shape[1] != buffers.table_pages or buffers.d_tables.device != device:
        raise ValueError(f"the step buffers hold {buffers.step_rows} rows of {buffers.table_pages} table pages on "
                         f"{buffers.d_tables.device}: {rows} rows of {round_tables.shape[1]} pages on {device} do not fit")
    p = _abi.StepParams()
    p.round_tables, p.round_capacity = round_tables.data_ptr(), round_capacity.data_ptr()
    p.round_lengths = None if round_lengths is None else \
        _i64_on(round_lengths, device, "the round lengths", round_tables.shape[0]).data_ptr()
    if round_lengths is None and firsts is None:
        raise ValueError("rows start at firsts or at the round lengths")
    p.slot = slot.data_ptr()
    p.counts = None if counts is None else _i64_on(counts, device, "step_buffers' counts", rows).data_ptr()
    p.firsts = None if firsts is None else _i64_on(firsts, device, "step_buffers' firsts", rows).data_ptr()
    p.d_slots, p.positions_t, p.rows_t = buffers.d_slots.data_ptr(), buffers.positions_t.data_ptr(), buffers.rows_t.data_ptr()
    p.starts_t, p.d_rows, p.d_starts = buffers.starts_t.data_ptr(), buffers.d_rows.data_ptr(), buffers.d_starts.data_ptr()
    p.d_counts, p.d_firsts, p.d_offsets = buffers.d_counts.data_ptr(), buffers.d_firsts.data_ptr(), buffers.d_offsets.data_ptr()
    p.d_tables, p.totals = buffers.d_tables.data_ptr(), buffers.totals.data_ptr()
    p.rows, p.round_slots, p.table_stride = rows, round_tables.shape[0], round_tables.stride(0)
    p.d_tables_stride, p.step_tokens, p.step_rows = buffers.d_tables.stride(0), buffers.step_tokens, buffers.step_rows
    p.count_each, p.window = int(count), int(window)
    p.table_pages, p.page, p.dump = buffers.table_pages, int(page), buffers.dump
    _launch(device, "crit_pkv_step_buffers", "paged_kv_attention.step_buffers", p)
    return buffers


# -- rows read back (reference: inference/attention-state/code/pages.py:455-493) -----------------------------------------
def _read(key_pages, value_pages, kind, n, shape, dtype, key_scales, value_scales, multipliers, slots=None, table=None,
          page=0, out=None):
    k_kind = _check_kind(kind, key_scales)
    _require_device(key_pages, "the key pages")
    device = key_pages.device
    if dtype not in _DTYPE:
        raise ValueError("rows are read back as float32, bfloat16 or float16")
    if key_pages.dim() < 2 or not key_pages.is_contiguous() or (value_pages is not None and (
            not value_pages.is_contiguous() or value_pages.device != device or value_pages.shape[-2] != key_pages.shape[-2])):
        raise ValueError("pages are contiguous [...][kv_heads][dim] on one device")
    hkv, d = key_pages.shape[-2], key_pages.shape[-1]
    dv = 0 if value_pages is None else value_pages.shape[-1]
    if d % 8 or dv % 8:
        raise ValueError("head widths are multiples of 8")
    km, vm, heads = _multipliers(multipliers, hkv, device)
    if out is None:
        out = (torch.empty(*shape, hkv, d, dtype=dtype, device=device),
               None if value_pages is None else torch.empty(*shape, hkv, dv, dtype=dtype, device=device))
    else:
        for o, width in zip(out, (d, dv)):
            if o is not None and (o.dtype != dtype or o.device != device or not o.is_contiguous() or
                                  o.numel() != n * hkv * width):
                raise ValueError("out holds (keys, values) [n][kv_heads][dim], contiguous, in the dtype asked for")
    p = _abi.ReadParams()
    p.key_pages, p.value_pages, p.key_scales, p.value_scales = key_pages.data_ptr(), _ptr(value_pages), _ptr(key_scales), _ptr(value_scales)
    p.head_multipliers, p.slots = _ptr(heads), _ptr(slots)
    if table is not None:
        p.table, p.table64 = (table.data_ptr(), None) if table.dtype == torch.int32 else (None, table.data_ptr())
    p.out_keys, p.out_values, p.n = out[0].data_ptr(), _ptr(out[1]), n
    p.pool_slots = key_pages.numel() // (hkv * d)
    p.kv_heads, p.head_dim, p.value_dim, p.page, p.kind = hkv, d, dv, int(page), k_kind
    p.page_dtype, p.out_dtype, p.key_multiplier, p.value_multiplier = _page_dtype(key_pages, kind), _DTYPE[dtype], km, vm
    _launch(device, "crit_pkv_read_rows", "paged_kv_attention.rows_at", p)
    return out


def rows_at(key_pages, value_pages, kind, slots, *, key_scales=None, value_scales=None, multipliers=(1.0, 1.0),
            dtype=torch.float32, out=None):
    """The keys and values at `slots` (any shape, int64, on the device) dequantised: KVPool.rows_at (pages.py:479-493)
    in one launch: float(stored) * the layer's multiplier or the row's scale, one FP32 product, in `dtype` (FP32 as the
    reference's). A negative slot, or one past the pages, reads as zeros. value_pages None: keys only. Returns (keys [..., kv_heads, dim],
    values)."""
    if not torch.is_tensor(slots) or slots.dtype != torch.int64 or slots.device != key_pages.device or not slots.is_contiguous():
        raise ValueError("slots are a contiguous int64 tensor on the pages' device")
    return _read(key_pages, value_pages, kind, slots.numel(), tuple(slots.shape), dtype, key_scales, value_scales,
                 multipliers, slots=slots, out=out)


def gather(key_pages, value_pages, kind, table, count, page, *, key_scales=None, value_scales=None,
           multipliers=(1.0, 1.0), dtype=torch.bfloat16, out=None):
    """A sequence's first `count` positions as contiguous rows in the compute dtype, dequantised: KVPool.gather
    (pages.py:455-477) in one launch; table [ceil(count / page) or more] int32 or int64 on the device."""
    if not torch.is_tensor(table) or table.dtype not in (torch.int32, torch.int64) or table.device != key_pages.device or \
            table.dim() != 1 or not table.is_contiguous() or table.numel() * page < count or count < 0 or page < 1:
        raise ValueError("a page table is a contiguous int32 or int64 tensor on the pages' device that covers `count` positions")
    return _read(key_pages, value_pages, kind, int(count), (int(count),), dtype, key_scales, value_scales, multipliers,
                 table=table, page=page, out=out)
