"""Sparse index selection on MI355X: the host side of crit's sparse-indexer kernels module (reference
kernels/techniques/attention/sparse-indexer/torch-ext/sparse_indexer/__init__.py: `scores` :101-127, `topk` :130-150,
`select` :235-262), with the same three calls, keyword arguments and error types, over the gfx950 kernels of
libcrit_pkv.so (crit_pkv_index_scores, crit_pkv_index_topk). There is no other implementation behind this module.

What the three calls compute:

    scores(q, keys, weights, ends)      FP32 [tokens][n]; entry (t, j) = sum over heads h of
                                        weights[t][h] * scale * max(0, q[t][h] . keys[j]) for j < ends[t], else -inf
    topk(s, ends, k)                    int32 [tokens][k]; the positions of row t's k largest entries among its first
                                        ends[t] (ties: the lower position first; NaN ranks below every number), written
                                        in ascending position order and padded with -1
    select(q, keys, weights, ends, k)   topk(scores(...)) with the score matrix held in a bounded workspace

Operands: q [tokens][heads][dim] BF16 or FP16; keys [n][dim] of q's dtype, or float8_e4m3fn codes with one FP32
key_scales[n] factor a row; weights FP32 [tokens][heads]; ends int32 [tokens]; scale defaults to dim ** -0.5.
`slots=` reads the keys where a pool keeps them: `keys` is then the whole store and key j is row slots[j] of it (one
list [n] for all tokens, or [groups][n] with the tokens cut into that many equal consecutive runs).

A token's result depends on that token's operands only, never on the launch it rode in. No call synchronises with the
host; when `out` (and select's `workspace`) are passed the only allocation left is topk's candidate room for long rows,
which comes from torch's caching allocator and so can be captured into a graph once the shape has run.
"""
from typing import Optional

import torch

from ..paged_kv_attention import _abi
from ..paged_kv_attention import _launch, _ptr, _require_device

__all__ = ["scores", "select", "topk"]

FP8 = torch.float8_e4m3fn
_HALF_TYPES = (torch.bfloat16, torch.float16)
_DIMS = (64, 128, 256)
_MAX_HEADS = 128
_LAUNCH_TOKENS = 65535      # the kernels' grid carries the token index in a 16-bit dimension


def _row_major(x):
    return x.stride(-1) == 1


def _slot_groups(slots, tokens):
    """Validates `slots` and returns (keys a token scores, tokens sharing one slot list)."""
    ok = torch.is_tensor(slots) and slots.dtype in (torch.int32, torch.int64) and 1 <= slots.dim() <= 2
    if not ok or not _row_major(slots):
        raise ValueError("slots: an int32/int64 tensor [n] or [groups][n] with unit stride along n")
    lists = 1 if slots.dim() == 1 else slots.shape[0]
    if lists == 0 or tokens % lists != 0:
        raise ValueError(f"slots: {lists} lists cannot be shared out evenly over {tokens} tokens")
    return slots.shape[-1], tokens // lists


def _score_operands(q, keys, weights, ends, key_scales):
    """Validates the operands every scoring call takes; returns (tokens, heads, dim, keys_are_e4m3)."""
    if q.dim() != 3 or q.dtype not in _HALF_TYPES or not _row_major(q):
        raise ValueError("q: a BF16/FP16 tensor [tokens][heads][dim] with unit stride along dim")
    _require_device(q, "the indexer's q")
    tokens, heads, dim = q.shape
    if dim not in _DIMS:
        raise ValueError(f"q: dim {dim} is not one of {_DIMS}")
    if heads < 1 or heads > _MAX_HEADS or heads & (heads - 1):
        raise ValueError(f"q: {heads} heads; the count must be a power of two no larger than {_MAX_HEADS}")
    if keys.dim() != 2 or keys.shape[1] != dim or not _row_major(keys):
        raise ValueError(f"keys: a tensor [n][{dim}] with unit stride along dim")
    coded = keys.dtype == FP8
    if coded:
        if key_scales is None or key_scales.dtype != torch.float32 or tuple(key_scales.shape) != (keys.shape[0],):
            raise ValueError(f"key_scales: E4M3 keys need one FP32 factor a row, [{keys.shape[0]}]")
    elif keys.dtype != q.dtype:
        raise ValueError(f"keys: dtype {keys.dtype} is neither q's ({q.dtype}) nor float8_e4m3fn")
    if tuple(weights.shape) != (tokens, heads) or weights.dtype != torch.float32 or not _row_major(weights):
        raise ValueError(f"weights: an FP32 tensor [{tokens}][{heads}]")
    if tuple(ends.shape) != (tokens,) or ends.dtype != torch.int32:
        raise ValueError(f"ends: an int32 tensor [{tokens}]")
    for name, x in (("keys", keys), ("weights", weights), ("ends", ends)):
        if x.device != q.device:
            raise ValueError(f"{name} is on {x.device}, q on {q.device}")
    return tokens, heads, dim, coded


def _picks_buffer(out, tokens, k, device):
    if out is None:
        return torch.empty(tokens, k, dtype=torch.int32, device=device)
    if tuple(out.shape) != (tokens, k) or out.dtype != torch.int32 or not _row_major(out):
        raise ValueError(f"out: an int32 tensor [{tokens}][{k}]")
    return out


def _token_runs(tokens, group, slots):
    """Cuts a call of more tokens than one launch takes into (first, last, slots) runs that keep slot groups whole."""
    cap = _LAUNCH_TOKENS
    if slots is None or slots.dim() == 1:
        return [(a, min(a + cap, tokens), slots) for a in range(0, tokens, cap)]
    lists = tokens // group
    if group > cap:     # one group is itself several launches, each over that group's own list
        return [(g * group + a, g * group + min(a + cap, group), slots[g])
                for g in range(lists) for a in range(0, group, cap)]
    whole = cap // group
    return [(g * group, min(g + whole, lists) * group, slots[g:g + whole]) for g in range(0, lists, whole)]


def scores(q, keys, weights, ends, *, key_scales=None, scale=None, out: Optional[torch.Tensor] = None,
           slots: Optional[torch.Tensor] = None):
    """FP32 [tokens][n] scores (see the module text); n is the keys' count, or the slots' when `slots` is given."""
    tokens, heads, dim, coded = _score_operands(q, keys, weights, ends, key_scales)
    if slots is None:
        n, group = keys.shape[0], max(tokens, 1)
    else:
        n, group = _slot_groups(slots, tokens)
    if out is None:
        out = torch.empty(tokens, n, dtype=torch.float32, device=q.device)
    elif out.dtype != torch.float32 or out.dim() != 2 or out.shape[0] < tokens or out.shape[1] < n or not _row_major(out):
        raise ValueError(f"out: an FP32 tensor of at least [{tokens}][{n}] with unit stride along n")
    if tokens == 0 or n == 0:
        return out
    if tokens > _LAUNCH_TOKENS:
        for first, last, these in _token_runs(tokens, group, slots):
            scores(q[first:last], keys, weights[first:last], ends[first:last], key_scales=key_scales, scale=scale,
                   out=out[first:last], slots=these)
        return out
    p = _abi.IndexScoresParams()
    p.q, p.keys, p.weights, p.ends, p.out = (x.data_ptr() for x in (q, keys, weights, ends, out))
    p.key_scales = _ptr(key_scales) if coded else None
    p.slots = _ptr(slots)
    p.q_stride_t, p.q_stride_h = q.stride(0), q.stride(1)
    p.key_stride, p.weights_stride, p.out_stride = keys.stride(0), weights.stride(0), out.stride(0)
    p.slots_stride = slots.stride(0) if slots is not None and slots.dim() == 2 else 0
    p.tokens, p.n, p.group, p.heads, p.dim = tokens, n, group, heads, dim
    p.key_dtype = 2 if coded else int(keys.dtype == torch.float16)
    p.q_dtype = _abi.F16 if q.dtype == torch.float16 else _abi.BF16
    p.slots_are_64 = int(slots is not None and slots.dtype == torch.int64)
    p.scale = float(dim ** -0.5 if scale is None else scale)
    _launch(q.device, "crit_pkv_index_scores", "sparse_indexer.scores", p)
    return out


def topk(s, ends, k, *, out: Optional[torch.Tensor] = None):
    """int32 [tokens][k] picks from FP32 scores s [tokens][n] (see the module text)."""
    if s.dim() != 2 or s.dtype != torch.float32 or not _row_major(s):
        raise ValueError("s: an FP32 tensor [tokens][n] with unit stride along n")
    _require_device(s, "the indexer's scores")
    tokens, n = s.shape
    if tuple(ends.shape) != (tokens,) or ends.dtype != torch.int32:
        raise ValueError(f"ends: an int32 tensor [{tokens}]")
    k = int(k)
    if k < 1:
        raise ValueError(f"k: {k}; at least one pick a token")
    out = _picks_buffer(out, tokens, k, s.device)
    if tokens == 0:
        return out
    # A long row is selected in slices whose candidates go through a buffer; the library says how large.
    with torch.cuda.device(s.device):
        room = int(_abi.load().crit_pkv_index_topk_work_bytes(tokens, n, k))
    work = torch.empty(room // 4, dtype=torch.int32, device=s.device) if room else None
    p = _abi.IndexTopkParams()
    p.scores, p.ends, p.out = s.data_ptr(), ends.data_ptr(), out.data_ptr()
    p.work, p.work_bytes = _ptr(work), room
    p.scores_stride, p.out_stride = s.stride(0), out.stride(0)
    p.tokens, p.n, p.k = tokens, n, k
    _launch(s.device, "crit_pkv_index_topk", "sparse_indexer.topk", p)
    return out


def select(q, keys, weights, ends, k, *, key_scales=None, scale=None, out: Optional[torch.Tensor] = None,
           workspace: Optional[torch.Tensor] = None, workspace_bytes=64 << 20, slots: Optional[torch.Tensor] = None):
    """topk(scores(...), ends, k) without ever holding the whole score matrix: tokens are taken in batches whose scores
    fit `workspace` (FP32, any shape; by default a fresh buffer of at most workspace_bytes). The picks are those of the
    two calls made separately. `slots` here is one list [n] for every token."""
    tokens, _, _, _ = _score_operands(q, keys, weights, ends, key_scales)
    if slots is not None and slots.dim() != 1:
        raise ValueError("slots: select takes one list [n]; per-group lists [groups][n] are for scores()")
    n = keys.shape[0] if slots is None else slots.shape[0]
    out = _picks_buffer(out, tokens, k, q.device)
    if tokens == 0:
        return out
    if n == 0:
        out.fill_(-1)
        return out
    if workspace is None:
        batch = min(tokens, max(1, (workspace_bytes // 4) // n))
        workspace = torch.empty(batch * n, dtype=torch.float32, device=q.device)
    else:
        if workspace.dtype != torch.float32 or workspace.numel() < n:
            raise ValueError(f"workspace: FP32 with at least {n} elements (one token's scores)")
        batch = min(tokens, workspace.numel() // n)
    flat = workspace.view(-1)
    first = 0
    while first < tokens:
        last = min(first + batch, tokens)
        held = flat[:(last - first) * n].view(last - first, n)
        scores(q[first:last], keys, weights[first:last], ends[first:last], key_scales=key_scales, scale=scale,
               out=held, slots=slots)
        topk(held, ends[first:last], k, out=out[first:last])
        first = last
    return out
