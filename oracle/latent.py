"""Latent attention (multi-head latent attention in its absorbed form), restated on the CPU in float64. Test
infrastructure only: nothing that ships may import this.

Follows inference/attention-state/code/latent_attention.py:16-33 (the operation's reference) and the cache's write rule
of kernels/techniques/attention/latent-attention/torch-ext/latent_attention/__init__.py:71-94 (rows of latent then rotary
key; an E4M3 cache codes each part at its own scale max|x| / 448, at least 1e-30, IEEE divisions). Pinned
(tests/test_oracle.py) by a scalar loop over a tiny case, by ordinary attention over keys [latent | rope] and values
latent (oracle.attend.reference, itself pinned), by the sink's closed form, and the write rule by the E4M3 encoder's
pinned vectors through oracle.append.encode.
"""
import torch


def latent_attention(q_latent, q_rope, latent, rope, seen, scale, sinks=None):
    """q_latent [T][H][R], q_rope [T][H][P] over latent [N][R], rope [N][P], seen [T][N] bool -> (out [T][H][R], lse
    [T][H]) in float64; sinks [H] (or None): one more score a head, with no value. A token that sees nothing (and has no
    sink) gives zeros and -inf."""
    ql, qr, c, k = q_latent.double(), q_rope.double(), latent.double(), rope.double()
    s = (torch.einsum("thr,nr->thn", ql, c) + torch.einsum("thp,np->thn", qr, k)) * scale
    s = s.masked_fill(~seen[:, None, :], float("-inf"))
    if sinks is not None:
        s = torch.cat([s, sinks.double().view(1, -1, 1).expand(s.shape[0], -1, 1)], dim=-1)
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - torch.where(lse == float("-inf"), torch.zeros_like(lse), lse)[..., None])
    p = torch.where(lse[..., None] == float("-inf"), torch.zeros_like(p), p)
    if sinks is not None:
        p = p[..., :-1]
    return torch.einsum("thn,nr->thr", p, c), lse


def write(latent, rope, slots, cache, scales=None):
    """latent [N][R] and rope [N][P] into rows `slots` of cache [pages][page][R + P] in its dtype; an E4M3 cache with
    scales [pages][page][2]."""
    flat = cache.view(-1, cache.shape[-1])
    if cache.dtype == torch.float8_e4m3fn:
        codes, found = [], []
        for x in (latent.float(), rope.float()):
            amax = x.abs().amax(-1)
            s = (amax / torch.full_like(amax, 448.0)).clamp(min=1e-30)
            codes.append((x / s[:, None]).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8))
            found.append(s)
        flat.view(torch.uint8).index_copy_(0, slots, torch.cat(codes, dim=-1))
        scales.view(-1, 2).index_copy_(0, slots, torch.stack(found, dim=-1))
        return
    flat.index_copy_(0, slots, torch.cat([latent.to(cache.dtype), rope.to(cache.dtype)], dim=-1))


def stored(cache, scales, table, n, page, rank):
    """Positions 0 .. n - 1 of the sequence with page table `table` as the cache holds them: (latent [n][R], rope
    [n][P]) float64, codes times their scales for an E4M3 cache (scales [pages][page][2], or [..][1]: one a row)."""
    positions = torch.arange(n)
    slots = table[positions // page].long() * page + positions % page
    rows = cache.view(-1, cache.shape[-1])[slots].double()
    latent, rope = rows[:, :rank], rows[:, rank:]
    if scales is not None:
        s = scales.view(-1, scales.shape[-1])[slots].double()
        latent, rope = latent * s[:, :1], rope * s[:, -1:]
    return latent, rope
