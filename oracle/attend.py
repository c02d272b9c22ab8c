"""Attention over paged KV, restated on the CPU. Test infrastructure only.

Conventions: query head h reads KV head h // (HQ // HKV); a token at position p sees positions n <= p of its sequence
(and, with a sliding window w, only n > p - w); softmax in the natural base over scores q.k * scale; a row that sees no
position gives output 0 and log-sum-exp -inf.
"""
import math

import torch

from . import append


# -- the float64 reference over stored values (test_paged_kv_attention.py:71-81) ---------------------------------------
def reference(q, keys, values, seen, scale, late=None):
    """q [HQ][D] float64 over keys [n][HKV][D], values [n][HKV][DV] where seen [n] (bool) -> (out [HQ][DV], lse [HQ]).
    A head that sees nothing gets zeros and -inf. late = (queries [HQ][D], position): the positions from `position` on
    are scored with those queries instead (an int8_qk chunk's fresh rows meet the queries as they are, the pages' rows
    their INT8 codes: _kernels.py:668-671, 708-709)."""
    hq, hkv = q.shape[0], keys.shape[1]
    group = hq // hkv
    out, lse = [], []
    neg = torch.tensor(float("-inf"), dtype=torch.float64)
    for h in range(hq):
        k, v = keys[:, h // group], values[:, h // group]
        s = (k @ q[h]) * scale
        if late is not None:
            s = torch.where(torch.arange(k.shape[0]) >= late[1], (k @ late[0][h]) * scale, s)
        s = torch.where(seen, s, neg)
        if not bool(seen.any()):
            out.append(torch.zeros(values.shape[-1], dtype=torch.float64))
            lse.append(neg.clone())
            continue
        lse.append(torch.logsumexp(s, 0))
        out.append(torch.softmax(s, 0) @ v)
    return torch.stack(out), torch.stack(lse)


def stored_rows(key_pages, value_pages, table, n, page, kind, key_scales=None, value_scales=None,
                multipliers=(1.0, 1.0)):
    """Positions 0..n-1 of the sequence with page table `table`, decoded to float64: keys [n][HKV][D], values
    [n][HKV][DV] (test_paged_kv_attention.py:50-60)."""
    hkv, d, dv = key_pages.shape[-2], key_pages.shape[-1], value_pages.shape[-1]
    ids = append.slots(table, torch.arange(n), page)
    k = key_pages.reshape(-1, hkv, d)[ids]
    v = value_pages.reshape(-1, hkv, dv)[ids]
    ks = key_scales.reshape(-1, hkv)[ids] if key_scales is not None else None
    vs = value_scales.reshape(-1, hkv)[ids] if value_scales is not None else None
    return (append.decode_rows(k, ks, kind, multipliers[0]), append.decode_rows(v, vs, kind, multipliers[1]))


def seen_by(first, count, c, n, parents=None, sliding=0):
    """Which of positions 0 .. n - 1 column c of a window row at `first` sees (_kernels.py:325-333): without parents
    the positions <= first + c; with parents (each column's parent column, -1 for none, parents before children)
    every position below first and, of the window, the positions of c's ancestors and c's own. A sliding window of w
    positions drops positions <= first + c - w either way."""
    positions = torch.arange(n)
    if parents is None:
        seen = positions <= first + c
    else:
        mine, at = {c}, int(parents[c])
        while at >= 0:
            mine.add(at)
            at = int(parents[at])
        seen = torch.tensor([p < first or (p - first) in mine for p in range(n)], dtype=torch.bool)
    if sliding:
        seen = seen & (positions > first + c - sliding)
    return seen


def listed(blocks, block_size, n):
    """Which of positions 0 .. n - 1 lie in one of a token's listed KV blocks (device_attention.py:1315-1317, the test at
    test_paged_kv_attention.py:391-392): block ids of block_size positions each, -1 for none."""
    ids = torch.as_tensor(blocks, dtype=torch.int64)
    ids = ids[ids >= 0]
    return (torch.arange(n) // block_size)[:, None].eq(ids[None, :]).any(1)


def with_fresh(keys, values, fresh, q_dtype):
    """Positions from `first` on take their keys and values from the fresh rows (row = position - shift), 16-bit in
    q's dtype and unscaled, instead of the pages' decoded ones (_kernels.py:272-274, 291-345: the scores of a fresh
    position times the scale only, its probability times 1; device_attention.py:1136-1145 says the same of the torch
    path). fresh = (fresh keys [N][HKV][D], fresh values [N][HKV][DV], shift, first)."""
    fk, fv, shift, first = fresh
    n = keys.shape[0]
    lo = max(int(first), 0)
    if lo >= n:
        return keys, values
    keys, values = keys.clone(), values.clone()
    keys[lo:] = fk[lo - shift:n - shift].to(q_dtype).double()
    values[lo:] = fv[lo - shift:n - shift].to(q_dtype).double()
    return keys, values


def int8_rows(q):
    """Each query row [.., D] (FP32 values of the 16-bit queries) to INT8 codes at its own scale and back, in float64
    (_kernels.py:637-643): scale = max(amax / 127, 1e-30) in FP32, codes = q / scale rounded half away from zero
    (|code| <= 127). The scores of an int8_qk chunk are the exact products of these codes and the keys' codes times
    both scales (_kernels.py:668-671), i.e. attention with the queries replaced by codes x scale."""
    qf = q.float()
    scale = (qf.abs().amax(-1, keepdim=True) / 127.0).clamp(min=1e-30)
    x = qf / scale
    codes = torch.where(x >= 0, x + 0.5, x - 0.5).trunc().clamp(-128, 127)
    return codes.double() * scale.double()


def window_reference(q, key_pages, value_pages, kind, table, first, count, page, scale, key_scales=None,
                     value_scales=None, multipliers=(1.0, 1.0), sliding=0, q_dtype=torch.bfloat16, parents=None,
                     blocks=None, block_size=None, fresh=None, int8_qk=False):
    """One window row in float64: q [count][HQ][D] (rounded to q_dtype first, as the kernels read it) at positions
    first .. first + count - 1 -> (out [count][HQ][DV], lse [count][HQ]). parents: the row's draft tree (seen_by);
    blocks [count][k] with block_size: each column's listed KV blocks (listed); fresh: with_fresh's tuple; int8_qk: the
    queries as int8_rows gives them against the pages' positions, as they are against the fresh ones."""
    n = first + count
    keys, values = stored_rows(key_pages, value_pages, table, n, page, kind, key_scales, value_scales, multipliers)
    if fresh is not None:
        keys, values = with_fresh(keys, values, fresh, q_dtype)
    qd = q.to(q_dtype).double()
    as_given = None
    if int8_qk:
        as_given, qd = (qd, max(int(fresh[3]), 0)) if fresh is not None else None, int8_rows(q.to(q_dtype))
    outs, lses = [], []
    for c in range(count):
        seen = seen_by(first, count, c, n, parents, sliding)
        if blocks is not None:
            seen = seen & listed(blocks[c], block_size, n)
        o, l = reference(qd[c], keys, values, seen, scale, None if as_given is None else (as_given[0][c], as_given[1]))
        outs.append(o)
        lses.append(l)
    return torch.stack(outs), torch.stack(lses)


# -- the reference's CPU/torch path: gather, then SDPA (pages.py:455-477, device_attention.py:1148-1166) ---------------
def gather(key_pages, value_pages, table, count, page, kind, compute, key_scales=None, value_scales=None,
           multipliers=(1.0, 1.0)):
    """A sequence's first `count` positions as contiguous rows in the compute dtype, dequantised (pages.py:455-477):
    index_select of whole pages, reshape, cut."""
    index = torch.as_tensor(table, dtype=torch.int64)[:math.ceil(count / page)]
    n = index.numel() * page
    hkv, d, dv = key_pages.shape[-2], key_pages.shape[-1], value_pages.shape[-1]
    k = key_pages.index_select(0, index).reshape(n, hkv, d)[:count]
    v = value_pages.index_select(0, index).reshape(n, hkv, dv)[:count]
    if kind == "fp8":
        return (k.float() * multipliers[0]).to(compute), (v.float() * multipliers[1]).to(compute)
    if kind in append.ROW_SCALED:
        ks = key_scales.index_select(0, index).reshape(n, hkv)[:count]
        vs = value_scales.index_select(0, index).reshape(n, hkv)[:count]
        return (k.float() * ks[..., None]).to(compute), (v.float() * vs[..., None]).to(compute)
    return k.to(compute), v.to(compute)


def rows_at(key_pages, value_pages, slots, kind, key_scales=None, value_scales=None, multipliers=(1.0, 1.0)):
    """The keys and values at `slots` (any shape, int64) dequantised to FP32 (pages.py:479-493): index_select of the
    rows, .float(), times the layer's multiplier (fp8) or the row's scale. Pages [pages][page][HKV][dim]."""
    hkv, d, dv = key_pages.shape[-2], key_pages.shape[-1], value_pages.shape[-1]
    flat = slots.reshape(-1)
    k = key_pages.reshape(-1, hkv, d).index_select(0, flat).float()
    v = value_pages.reshape(-1, hkv, dv).index_select(0, flat).float()
    if kind == "fp8":
        k, v = k * multipliers[0], v * multipliers[1]
    elif kind in append.ROW_SCALED:
        k = k * key_scales.reshape(-1, hkv).index_select(0, flat)[..., None]
        v = v * value_scales.reshape(-1, hkv).index_select(0, flat)[..., None]
    shape = tuple(slots.shape)
    return k.view(*shape, hkv, d), v.view(*shape, hkv, dv)


def sdpa_rows(queries, rows, gather_row, scale, out):
    """The reference's CPU attention path (device_attention.py:1148-1166): per batch row (first token, count, first
    position) gather its KV with gather_row(r, n) and run torch's scaled_dot_product_attention with GQA; one token sees
    everything held, a chunk from position 0 is plain causal, a later chunk takes the offset mask."""
    heads = queries.shape[1]
    for r, (first, count, position) in enumerate(rows):
        keys, values = gather_row(r, position + count)
        q = queries[first:first + count].transpose(0, 1).unsqueeze(0).to(keys.dtype)
        k, v = keys.transpose(0, 1).unsqueeze(0), values.transpose(0, 1).unsqueeze(0)
        mask, causal = None, count > 1 and position == 0
        if count > 1 and position > 0:
            seen = torch.arange(position + count)
            mask = seen[None, :] <= (position + torch.arange(count))[:, None]
        found = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, is_causal=causal,
                                                                 scale=scale, enable_gqa=heads != keys.shape[1])
        out[first:first + count] = found[0].transpose(0, 1).to(out.dtype)
    return out


def windows_dense(q, keys, values, position, scale, sliding=0, sinks=None):
    """One row of tokens at positions position.. over its gathered keys [n][HKV][D] and values in FP32, causal
    (device_attention.py:1301-1335 without trees and block lists) -> (out [count][HQ][DV] FP32, lse [count][HQ])."""
    count, hq, d = q.shape
    hkv = keys.shape[1]
    g = hq // hkv
    n = torch.arange(keys.shape[0])
    seen = (n[None, :] <= (position + torch.arange(count))[:, None])
    if sliding:
        seen = seen & (n[None, :] > (position + torch.arange(count))[:, None] - sliding)
    qq = q.float().view(count, hkv, g, d)
    s = torch.einsum("ckgd,nkd->ckgn", qq, keys.float()) * scale
    s = s.masked_fill(~seen[:, None, None, :], float("-inf"))
    top = s.amax(-1)
    if sinks is not None:
        top = torch.maximum(top, sinks.view(1, hkv, g))
    sub = torch.where(top == float("-inf"), 0.0, top)
    p = torch.exp(s - sub[..., None])
    total = p.sum(-1)
    if sinks is not None:
        total = total + torch.exp(sinks.view(1, hkv, g) - sub)
    o = torch.einsum("ckgn,nkd->ckgd", p, values.float()) / total.clamp(min=1e-30)[..., None]
    out = torch.where(total[..., None] > 0, o, 0.0).view(count, hq, -1)
    lse = torch.where(total > 0, top + torch.log(total.clamp(min=1e-30)), float("-inf")).view(count, hq)
    return out, lse


# -- keys derived from the value rows (kernels/.../paged_kv_attention/__init__.py:52-58) --------------------------------
def derived_keys(rows, weight, eps, freqs, rotary_dim, start=0):
    """float64 keys of the stored rows [n][HKV][D] (float64) at positions start..: rope(rms_norm(r) * weight, p) with
    rms_norm(r) = r / sqrt(mean(r * r) + eps), weight [D] or None, the "half" rotation over the first rotary_dim values
    (value i with value i + rotary_dim / 2, the rest kept) at the angle fp32(p) * freqs[i] taken as an FP32 product, as
    the kernels take it (tests/test_derived_keys.py:68-81 of the reference)."""
    y = rows / torch.sqrt((rows * rows).mean(-1, keepdim=True) + eps)
    if weight is not None:
        y = y * weight.double()
    pos = torch.arange(start, start + rows.shape[0], dtype=torch.float32)
    angle = (pos[:, None] * freqs.float()[None, :]).double()[:, None, :]
    half = rotary_dim // 2
    a, b = y[..., :half], y[..., half:rotary_dim]
    turned = torch.cat([a * angle.cos() - b * angle.sin(), b * angle.cos() + a * angle.sin()], -1)
    return torch.cat([turned, y[..., rotary_dim:]], -1)


# -- the torch fallback over page tables (device_attention.py:1204-1288) ------------------------------------------------
CHUNK = 1024      # positions a pass (device_attention.py:53)


def windows_online(q, key_pages, value_pages, kind, tables, rows, starts, counts, firsts, columns, page, scale,
                   key_scales=None, value_scales=None, multipliers=(1.0, 1.0), extent=None, sliding=0, sinks=None,
                   chunk=CHUNK):
    """Window rows in FP32 as the reference's fallback computes them (windows_torch, device_attention.py:1204-1288,
    without trees, block lists and fresh rows): row by row and column by column, a masked online softmax over passes of
    `chunk` positions of the row's page table (a position past the table's last page reads that page's) up to `extent`
    (None: every position the tables hold), the rows read back dequantised to FP32 (rows_at); a sink logit folded in
    after the passes. q [tokens][HQ][D]; tables [S][width] int32; rows, starts, counts (None: `columns` each), firsts one
    a row. Returns (out [tokens][HQ][DV] FP32, lse [tokens][HQ] FP32), rows no window holds left zero / -inf."""
    tokens, hq, d = q.shape
    hkv, dv = key_pages.shape[-2], value_pages.shape[-1]
    g = hq // hkv
    width = tables.shape[1]
    limit = width * page
    extent = limit if extent is None else extent
    extent = max(chunk, math.ceil(min(extent, limit) / chunk) * chunk)
    out = torch.zeros(tokens, hq, dv)
    found = torch.full((tokens, hq), float("-inf"))
    for r in range(len(rows)):
        table = tables[int(rows[r])]
        count = min(int(counts[r]), columns) if counts is not None else columns
        first = int(firsts[r])
        for c in range(count):
            qq = q[int(starts[r]) + c].float().view(hkv, g, d)
            m = torch.full((hkv, g), float("-inf"))
            l = torch.zeros(hkv, g)
            acc = torch.zeros(hkv, g, dv)
            for s0 in range(0, extent, chunk):
                n = torch.arange(s0, s0 + chunk)
                entry = table[(n // page).clamp(max=width - 1)]
                keys, values = rows_at(key_pages, value_pages, entry.long() * page + n % page, kind, key_scales,
                                       value_scales, multipliers)
                seen = n <= first + c
                if sliding:
                    seen = seen & (n > first + c - sliding)
                s = torch.einsum("kgd,nkd->kgn", qq, keys) * scale
                s = s.masked_fill(~seen[None, None, :], float("-inf"))
                top = torch.maximum(m, s.amax(-1))
                sub = torch.where(top == float("-inf"), 0.0, top)
                p = torch.exp(s - sub[..., None])
                alpha = torch.exp(m - sub)
                l = l * alpha + p.sum(-1)
                acc = acc * alpha[..., None] + torch.einsum("kgn,nkd->kgd", p, values)
                m = top
            if sinks is not None:      # _sink_fold (device_attention.py:1291-1298): one more position with no value
                sink = sinks.float().view(hkv, g)
                top = torch.maximum(m, sink)
                sub = torch.where(top == float("-inf"), 0.0, top)
                keep = torch.exp(m - sub)
                m, l, acc = top, l * keep + torch.exp(sink - sub), acc * keep[..., None]
            t = int(starts[r]) + c
            out[t] = torch.where(l[..., None] > 0, acc / l.clamp(min=1e-30)[..., None], 0.0).view(hq, dv)
            found[t] = torch.where(l > 0, m + torch.log(l.clamp(min=1e-30)), float("-inf")).view(hq)
    return out, found


# -- online softmax steps (kernels/core/python/crit_kcore/attention_softmax.py:37-101), natural base --------------------
def step(s, m):
    """One block of scores s [rows][positions] (masked ones -inf) against running maxima m [rows] -> (p, alpha,
    m_new); a row that has seen nothing keeps -inf and gets p = 0, alpha = 0."""
    m_new = torch.maximum(m, s.amax(dim=1))
    m_sub = torch.where(m_new == float("-inf"), torch.zeros_like(m_new), m_new)
    return torch.exp(s - m_sub[:, None]), torch.exp(m - m_sub), m_new


def fold(m_run, l_run, m, l):
    """A partial state (m, l) into the running one -> (m_new, l_new, keep, take): out = out * keep + partial * take."""
    m_new = torch.maximum(m_run, m)
    m_sub = torch.where(m_new == float("-inf"), torch.zeros_like(m_new), m_new)
    keep, take = torch.exp(m_run - m_sub), torch.exp(m - m_sub)
    return m_new, l_run * keep + l * take, keep, take


def finish(acc, l):
    """acc / l per row, 0 where l == 0."""
    ok = l != 0
    return torch.where(ok[:, None], acc / torch.where(ok, l, torch.ones_like(l))[:, None], torch.zeros_like(acc))


def lse(m, l):
    """m + log l, -inf where l == 0."""
    return torch.where(l != 0, m + torch.log(torch.where(l != 0, l, torch.ones_like(l))), torch.full_like(m, -math.inf))


# -- log-sum-exp merge across parts (inference/partitioned-attention/plugin.py:52-64) ------------------------------------
def merge(outs, lses):
    """Partials of the same queries over disjoint keys: outs [parts][T][HQ][DV], lses [parts][T][HQ] (-inf: the part
    saw no key) -> (out FP32, lse FP32); a token no part saw gets zeros and -inf."""
    outs, lses = torch.stack(list(outs)).float(), torch.stack(list(lses)).float()
    top = lses.amax(0)
    sub = torch.where(top == float("-inf"), 0.0, top)
    weights = torch.where(lses == float("-inf"), 0.0, torch.exp(lses - sub))
    total = weights.sum(0)
    out = (weights[..., None] * outs).sum(0) / total.clamp(min=1e-30)[..., None]
    out = torch.where(total[..., None] > 0, out, 0.0)
    return out, torch.where(total > 0, sub + torch.log(total.clamp(min=1e-30)), float("-inf"))


# -- the host technique (inference/partitioned-attention/code/implementation.py:22-138), Python floats -------------------
def owner(position, world):
    """The rank that owns a position: position mod world (implementation.py:34-35)."""
    return position % world


def global_position(local, world, rank):
    """implementation.py:42-43."""
    return local * world + rank


def attention_partial(query, rows, value_width, query_position, scale=None):
    """rows of (global position, key, value) one rank holds -> (output tuple, log normalizer); positions past the
    query are masked; an empty shard gives zeros and -inf (implementation.py:71-116)."""
    scale = 1 / math.sqrt(len(query)) if scale is None else scale
    logits, values = [], []
    for position, key, value in rows:
        if position > query_position:
            continue
        logits.append(math.fsum(a * b for a, b in zip(query, key)) * scale)
        values.append(value)
    if not logits:
        return (0.0,) * value_width, -math.inf
    top = max(logits)
    weights = [math.exp(x - top) for x in logits]
    total = math.fsum(weights)
    output = tuple(math.fsum((w / total) * row[c] for w, row in zip(weights, values)) for c in range(value_width))
    return output, top + math.log(total)


def merge_partials(partials):
    """(output, log normalizer) pairs of disjoint shards -> the whole's; all-empty input raises
    (implementation.py:119-138)."""
    partials = list(partials)
    top = max(l for _, l in partials)
    if top == -math.inf:
        raise ValueError("attention has no visible keys")
    weights = [math.exp(l - top) for _, l in partials]
    total = math.fsum(weights)
    width = len(partials[0][0])
    output = tuple(math.fsum((w / total) * o[c] for w, (o, _) in zip(weights, partials)) for c in range(width))
    return output, top + math.log(total)
