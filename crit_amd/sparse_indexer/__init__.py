"""Sparse index selection on MI355X: the host side of crit's sparse-indexer kernels module (reference
kernels/techniques/attention/sparse-indexer/torch-ext/sparse_indexer/__init__.py), same names, arguments and errors, over
the gfx950 kernels of libcrit_pkv.so (crit_pkv_index_scores, crit_pkv_index_topk).

    s = scores(q, keys, weights, ends)                # FP32 [tokens][keys]
    picked = topk(s, ends, k)                         # int32 [tokens][k]: ascending positions, -1 past the valid ones
    picked = select(q, keys, weights, ends, k)        # both, tokens in groups so the scores stay within a workspace
    s = scores(q, store, weights, ends, slots=slots)  # keys read in place: key j is store[slots[j]], no gathered copy

The score of token t over key s is the sum over its heads h of weights[t][h] x scale x ReLU(q[t][h] . keys[s]) (q
[tokens][heads][dim] BF16 or FP16; keys [n][dim] in q's dtype, or E4M3 codes as float8_e4m3fn with FP32 key_scales [n];
weights FP32 [tokens][heads]; scale default dim ** -0.5) for s below ends[t] (int32 [tokens]); keys at or past it score
-inf. topk keeps, per token, the k largest scores among its valid keys (all of them where it has k or fewer), ties to the
lower position, a NaN below every number, and writes their positions in ascending order, then -1. A token's scores and
picks are its own (not its neighbours', not the launch's shape). Nothing syncs with the host; with `out` (and select's
`workspace`) given nothing is allocated, so a graph captures a call. There is no other implementation behind this module.
"""
from typing import Optional

import torch

from ..paged_kv_attention import _abi
from ..paged_kv_attention import _launch, _ptr, _require_device

__all__ = ["scores", "select", "topk"]

FP8 = torch.float8_e4m3fn
_LAUNCH_TOKENS = 65535


def _check_slots(slots, tokens, rows):
    """(n, tokens a group) of `slots`: int32 or int64 [n] or [groups][n] on the keys' device, contiguous rows."""
    if not torch.is_tensor(slots) or slots.dtype not in (torch.int32, torch.int64) or slots.dim() not in (1, 2) or \
            slots.stride(-1) != 1:
        raise ValueError("slots are int32 or int64 [n] or [groups][n], each row contiguous")
    groups = slots.shape[0] if slots.dim() == 2 else 1
    if groups < 1 or tokens % groups:
        raise ValueError(f"{tokens} tokens are not {groups} equal groups (a group's tokens share its slots)")
    return slots.shape[-1], tokens // groups


def _check_scores(q, keys, weights, ends, key_scales):
    if q.dim() != 3 or q.dtype not in (torch.bfloat16, torch.float16) or q.stride(-1) != 1:
        raise ValueError("q is [tokens][heads][dim] BF16 or FP16, each head row contiguous")
    _require_device(q, "the indexer's q")
    t, h, d = q.shape
    if d not in (64, 128, 256) or h & (h - 1) or h > 128:
        raise ValueError(f"heads a power of two up to 128 and a dim of 64, 128 or 256, not {h} x {d}")
    if keys.dim() != 2 or keys.shape[1] != d or keys.stride(-1) != 1:
        raise ValueError(f"keys are [n][{d}], each row contiguous")
    fp8 = keys.dtype == FP8
    if not fp8 and keys.dtype != q.dtype:
        raise ValueError("keys are in q's dtype, or E4M3 codes (float8_e4m3fn) with key_scales")
    if fp8 and (key_scales is None or key_scales.dtype != torch.float32 or key_scales.shape != (keys.shape[0],)):
        raise ValueError("E4M3 keys take key_scales FP32 [n]")
    if weights.shape != (t, h) or weights.dtype != torch.float32 or weights.stride(-1) != 1:
        raise ValueError(f"weights are FP32 [{t}][{h}]")
    if ends.shape != (t,) or ends.dtype != torch.int32:
        raise ValueError(f"ends are int32 [{t}]")
    if keys.device != q.device or weights.device != q.device or ends.device != q.device:
        raise ValueError("q, keys, weights and ends live on one device")
    return t, h, d, fp8


def scores(q, keys, weights, ends, *, key_scales=None, scale=None, out: Optional[torch.Tensor] = None,
           slots: Optional[torch.Tensor] = None):
    """Every token's score over keys 0 .. n - 1 (FP32 [tokens][n]; -inf at or past ends[t]). slots: the keys in place,
    key j the store's row slots[j] ([n], or [groups][n] with the tokens in equal runs, a group a sequence); n is then
    the slots' count."""
    t, h, d, fp8 = _check_scores(q, keys, weights, ends, key_scales)
    n, group = (keys.shape[0], max(1, t)) if slots is None else _check_slots(slots, t, keys.shape[0])
    if out is None:
        out = torch.empty(t, n, dtype=torch.float32, device=q.device)
    if out.shape[0] < t or out.shape[1] < n or out.dtype != torch.float32 or out.stride(-1) != 1:
        raise ValueError(f"out is FP32 [{t}][{n}] or wider, rows contiguous")
    if t == 0 or n == 0:
        return out
    if t > _LAUNCH_TOKENS:      # a launch takes that many: longer calls go in runs of whole groups
        if slots is None or slots.dim() == 1:
            runs = [(t0, min(t0 + _LAUNCH_TOKENS, t), slots) for t0 in range(0, t, _LAUNCH_TOKENS)]
        elif group <= _LAUNCH_TOKENS:
            per = _LAUNCH_TOKENS // group
            runs = [(g0 * group, min(g0 + per, t // group) * group, slots[g0:g0 + per]) for g0 in range(0, t // group, per)]
        else:
            runs = [(g0 * group + t0, g0 * group + min(t0 + _LAUNCH_TOKENS, group), slots[g0])
                    for g0 in range(t // group) for t0 in range(0, group, _LAUNCH_TOKENS)]
        for first, last, these in runs:
            scores(q[first:last], keys, weights[first:last], ends[first:last], key_scales=key_scales, scale=scale,
                   out=out[first:last], slots=these)
        return out
    p = _abi.IndexScoresParams()
    p.q, p.keys, p.key_scales, p.weights, p.ends = q.data_ptr(), keys.data_ptr(), _ptr(key_scales) if fp8 else None, \
        weights.data_ptr(), ends.data_ptr()
    p.slots, p.out = _ptr(slots), out.data_ptr()
    p.q_stride_t, p.q_stride_h, p.key_stride, p.weights_stride = q.stride(0), q.stride(1), keys.stride(0), weights.stride(0)
    p.out_stride = out.stride(0)
    p.slots_stride = slots.stride(0) if slots is not None and slots.dim() == 2 else 0
    p.tokens, p.n, p.group, p.heads, p.dim = t, n, group, h, d
    p.key_dtype = 2 if fp8 else (1 if keys.dtype == torch.float16 else 0)
    p.q_dtype = _abi.F16 if q.dtype == torch.float16 else _abi.BF16
    p.slots_are_64 = int(slots is not None and slots.dtype == torch.int64)
    p.scale = float(scale if scale is not None else d ** -0.5)
    _launch(q.device, "crit_pkv_index_scores", "sparse_indexer.scores", p)
    return out


def topk(s, ends, k, *, out: Optional[torch.Tensor] = None):
    """The positions of each token's k largest scores below its end (s FP32 [tokens][n]), ascending, then -1 (int32
    [tokens][k])."""
    if s.dim() != 2 or s.dtype != torch.float32 or s.stride(-1) != 1:
        raise ValueError("scores are FP32 [tokens][n], rows contiguous")
    _require_device(s, "the indexer's scores")
    t, n = s.shape
    if ends.shape != (t,) or ends.dtype != torch.int32:
        raise ValueError(f"ends are int32 [{t}]")
    if k < 1:
        raise ValueError("k is at least 1")
    if out is None:
        out = torch.empty(t, k, dtype=torch.int32, device=s.device)
    if out.shape != (t, k) or out.dtype != torch.int32 or out.stride(-1) != 1:
        raise ValueError(f"out is int32 [{t}][{k}]")
    if t == 0:
        return out
    p = _abi.IndexTopkParams()
    p.scores, p.ends, p.out = s.data_ptr(), ends.data_ptr(), out.data_ptr()
    # long rows: the slices' k best, then the k best of those (the same picks); their room is the caching allocator's,
    # as the reference's is, so a graph captures the call once its shape has run
    with torch.cuda.device(s.device):
        room = int(_abi.load().crit_pkv_index_topk_work_bytes(t, n, int(k)))
    work = torch.empty(room // 4, dtype=torch.int32, device=s.device) if room else None
    p.work, p.work_bytes = _ptr(work), room
    p.scores_stride, p.out_stride, p.tokens, p.n, p.k = s.stride(0), out.stride(0), t, n, int(k)
    _launch(s.device, "crit_pkv_index_topk", "sparse_indexer.topk", p)
    return out


def select(q, keys, weights, ends, k, *, key_scales=None, scale=None, out: Optional[torch.Tensor] = None,
           workspace: Optional[torch.Tensor] = None, workspace_bytes=64 << 20, slots: Optional[torch.Tensor] = None):
    """topk(scores(...)) over groups of tokens whose scores fit the workspace (FP32; default a buffer of
    workspace_bytes), the same positions as one call (each token's scores and choice are its own). slots: the keys in
    place, as scores takes them (one list of slots for every token)."""
    t, h, d, _ = _check_scores(q, keys, weights, ends, key_scales)
    if slots is not None and slots.dim() != 1:
        raise ValueError("select takes one list of slots [n] (its tokens go in groups of its own): scores takes "
                         "[groups][n]")
    n = keys.shape[0] if slots is None else slots.shape[0]
    if out is None:
        out = torch.empty(t, k, dtype=torch.int32, device=q.device)
    if out.shape != (t, k) or out.dtype != torch.int32 or out.stride(-1) != 1:
        raise ValueError(f"out is int32 [{t}][{k}]")
    if t == 0:
        return out
    if n == 0:
        return out.fill_(-1)
    room = workspace.numel() if workspace is not None else workspace_bytes // 4
    group = max(1, min(t, room // n))
    if workspace is None:
        workspace = torch.empty(group * n, dtype=torch.float32, device=q.device)
    elif workspace.dtype != torch.float32 or workspace.numel() < n:
        raise ValueError(f"the workspace is FP32 with room for one token's {n} scores at least")
    for t0 in range(0, t, group):
        g = min(group, t - t0)
        s = workspace.view(-1)[:g * n].view(g, n)
        scores(q[t0:t0 + g], keys, weights[t0:t0 + g], ends[t0:t0 + g], key_scales=key_scales, scale=scale, out=s,
               slots=slots)
        topk(s, ends[t0:t0 + g], k, out=out[t0:t0 + g])
    return out
