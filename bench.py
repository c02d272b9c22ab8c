"""Benchmark of the paged-KV hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|c3] [--no-extras] [--no-cpu]

A step is one pass of the hot path over one synthetic batch: for each of 32 layers, one KV append (one new token per
sequence) and one paged decode attention over the whole context. The default workload is the Llama-3-8B-shaped bf16
configuration (32 query heads, 8 KV heads, head_dim 128, page 16, batch 64, contexts uniform in [1024, 8192], pages
randomly permuted in a pool 1.25x the needed size). Inputs are resident in HBM before the timed region starts.

Prints ONE JSON line on stdout (everything else goes to stderr): the whole-step rate in algorithmic GB/s, the decode
kernel's roofline fraction from HIP-event timing of that kernel alone, and the reference's CPU path (gather + SDPA and
index_copy append, FP32, restated in oracle/) timed on this host on a bounded sample of the same workload.
"""
import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, vendor figure

DECODE_KERNEL = "attend_mfma_kernel"      # the split launch's kernel (the dominant one)


def profiled_traffic(workload, piece):
    """HBM bytes one split launch of `workload` moves, from the counter runs summarised under profiles/ (rocprofv3 --pmc
    FETCH_SIZE and WRITE_SIZE of this file, each scaled by what it reads for a kernel of known size), or None when
    no summary covers this kernel at this piece: the figure belongs to the kernel and the launch shape it was taken on."""
    import re
    path = os.path.join(ROOT, "profiles", f"{DECODE_KERNEL}_{workload}_decode.md")
    try:
        text = open(path, encoding="utf-8").read()
    except OSError:
        return None, None
    found = re.search(r"HBM traffic per launch \(piece (\d+)\): ([\d,]+) B", text)
    if not found or int(found.group(1)) != int(piece) or DECODE_KERNEL not in text:
        return None, None
    return int(found.group(2).replace(",", "")), os.path.relpath(path, ROOT)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


WORKLOADS = {
    # name: (kind, batch, ctx_lo, ctx_hi, hq, hkv, d, layers, value scale, outliers)
    "c2": dict(kind="bf16", batch=64, lo=1024, hi=8192, hq=32, hkv=8, d=128, layers=32, std=0.5, outliers=False,
               name="llama3-8b-shaped paged decode, bf16 KV: B=64, ctx~U[1024,8192], 32q/8kv x128, page 16, 32 layers x (append + attend)"),
    "c3": dict(kind="fp8", batch=128, lo=2048, hi=16384, hq=32, hkv=8, d=128, layers=32, std=1.0, outliers=True,
               name="llama3-8b-shaped paged decode, FP8 E4M3 KV (per-(layer, kv-head) scales): B=128, ctx~U[2048,16384], 32 layers x (append + attend)"),
}


class Workload:
    def __init__(self, spec, device, seed=0, layers=None):
        import crit_amd.paged_kv_attention as pk
        self.pk, self.spec, self.device = pk, spec, device
        g = torch.Generator().manual_seed(seed)
        B, page = spec["batch"], 16
        self.page, self.kind = page, spec["kind"]
        self.layers = layers or spec["layers"]
        hkv, d, hq = spec["hkv"], spec["d"], spec["hq"]
        # ctx = positions already in the cache; the step appends position ctx and attends over ctx + 1 positions
        self.ctx = torch.randint(spec["lo"], spec["hi"] + 1, (B,), generator=g)
        need = int(((self.ctx + 1 + page - 1) // page).sum())
        self.n_pages = int(need * 1.25)
        perm = torch.randperm(self.n_pages, generator=g)
        width = int(((self.ctx.max() + 1 + page - 1) // page + 15) // 16 * 16)
        tables = torch.full((B, width), self.n_pages, dtype=torch.int32)      # unused entries: the dump page
        at = 0
        for s in range(B):
            w = int((self.ctx[s] + 1 + page - 1) // page)
            tables[s, :w] = perm[at:at + w].to(torch.int32)
            at += w
        self.tables = tables.to(device)
        store = torch.bfloat16 if self.kind == "bf16" else torch.float8_e4m3fn
        self.k, self.v = [], []
        gen = torch.Generator(device=device).manual_seed(seed)
        self.mult = []
        for layer in range(self.layers):
            shape = (self.n_pages + 1, page, hkv, d)
            pages = []
            for _ in range(2):
                x = torch.randn(shape, device=device, dtype=torch.bfloat16, generator=gen) * spec["std"]
                if spec["outliers"]:
                    hot = torch.rand(shape, device=device, generator=gen) < 0.01
                    x = torch.where(hot, x * 20, x)
                pages.append(x)
            if self.kind == "fp8":
                # per-(layer, kv-head) scales: amax / 448 over the rows (keys' row, then values')
                m = torch.stack([p.float().abs().amax(dim=(0, 1, 3)) / 448.0 for p in pages]).contiguous()
                self.mult.append(m)
                pages = [(p.float() / m[i][None, None, :, None]).clamp(-448, 448).to(store) for i, p in enumerate(pages)]
            else:
                self.mult.append((1.0, 1.0))
            self.k.append(pages[0])
            self.v.append(pages[1])
        self.rows = torch.arange(B, dtype=torch.int32, device=device)
        self.starts = torch.arange(B, dtype=torch.int32, device=device)
        self.counts = torch.ones(B, dtype=torch.int32, device=device)
        self.firsts = self.ctx.to(torch.int64).to(device)
        slots = torch.stack([tables[s, int(self.ctx[s]) // page].long() * page + int(self.ctx[s]) % page for s in range(B)])
        self.slots = slots.to(device)
        self.q = (torch.randn(B, hq, d, device=device, generator=gen) * spec["std"]).to(torch.bfloat16)
        self.new_k = (torch.randn(B, hkv, d, device=device, generator=gen) * spec["std"]).to(torch.bfloat16)
        self.new_v = (torch.randn(B, hkv, d, device=device, generator=gen) * spec["std"]).to(torch.bfloat16)
        self.out = torch.empty(B, hq, d, dtype=torch.bfloat16, device=device)
        self.parts = pk.partitions(device, hkv, self.kind, d, d)
        self.piece = pk.piece_size(d, d, self.kind, hkv)
        self.workspace = torch.empty(pk.workspace_floats(B, hq, self.parts, d), dtype=torch.float32, device=device)
        e = 2 if self.kind == "bf16" else 1
        tokens = int((self.ctx + 1).sum())
        self.decode_bytes = tokens * hkv * (d + d) * e            # per layer: K and V of every visible position
        self.append_bytes = B * hkv * (d + d) * (e + 2)           # per layer: page bytes written + bf16 inputs read
        self.tokens = tokens

    def append(self, layer):
        self.pk.write(self.new_k, self.new_v, self.slots, self.k[layer], self.v[layer], self.kind,
                      multipliers=self.mult[layer])

    def attend(self, layer, phases=0):
        self.pk.attend(self.q, self.k[layer], self.v[layer], self.kind, self.tables, self.rows, self.starts, self.firsts,
                       1, self.page, counts=self.counts, offsets=self.starts, tokens=self.q.shape[0],
                       multipliers=self.mult[layer], partitions=self.parts, piece=self.piece, out=self.out,
                       workspace=self.workspace, phases=phases)

    def step(self):
        for layer in range(self.layers):
            self.append(layer)
            self.attend(layer)


def timed(fn, reps, warmup=1):
    """Average milliseconds of fn() over reps calls, by HIP events on the current stream (the launch stream)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps


def kernel_ms(w, phases):
    """Average duration of one launch phase over every layer (cold: each layer's pages are different memory)."""
    w.attend(0, phases)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for layer in range(w.layers):
        w.attend(layer, phases)
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / w.layers


def cpu_baseline(spec, seconds=20.0):
    """The reference's CPU path (FP32 pages: index_copy append, then per row gather + SDPA) restated in oracle/,
    timed on this host over ONE layer and the first 8 sequences of the workload; the rate counts the same algorithmic
    bytes as the GPU figure (the GPU configuration's element size) for those sequences."""
    from oracle import append as oa
    from oracle import attend as oatt
    g = torch.Generator().manual_seed(0)
    B, page, hkv, d, hq = 8, 16, spec["hkv"], spec["d"], spec["hq"]
    ctx = torch.randint(spec["lo"], spec["hi"] + 1, (spec["batch"],), generator=g)[:B]
    need = int(((ctx + 1 + page - 1) // page).sum())
    n_pages = int(need * 1.25)
    perm = torch.randperm(n_pages, generator=g)
    tables, at = [], 0
    for s in range(B):
        wd = int((ctx[s] + 1 + page - 1) // page)
        tables.append(perm[at:at + wd])
        at += wd
    k = torch.randn(n_pages + 1, page, hkv, d, generator=g) * spec["std"]
    v = torch.randn(n_pages + 1, page, hkv, d, generator=g) * spec["std"]
    q = torch.randn(B, hq, d, generator=g)
    nk, nv = torch.randn(B, hkv, d, generator=g), torch.randn(B, hkv, d, generator=g)
    slots = torch.stack([oa.slots(tables[s], torch.tensor([int(ctx[s])]), page)[0] for s in range(B)])
    rows = [(s, 1, int(ctx[s])) for s in range(B)]
    out = torch.empty(B, hq, d)

    def one():
        oa.write(nk, nv, slots, k, v, "fp32", dump_slot=n_pages * page)
        oatt.sdpa_rows(q, rows, lambda r, n: oatt.gather(k, v, tables[r], n, page, "fp32", torch.float32), d ** -0.5, out)
    one()
    reps, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds or reps < 2:
        one()
        reps += 1
    dt = (time.perf_counter() - t0) / reps
    e = 2 if spec["kind"] == "bf16" else 1
    nbytes = int((ctx + 1).sum()) * hkv * 2 * d * e + B * hkv * 2 * d * (e + 2)
    return {"value": round(nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"1 layer x first 8 of {spec['batch']} sequences ({int((ctx + 1).sum())} positions), FP32 pages, "
                      f"{reps} reps, {dt * 1e3:.1f} ms each; bytes counted at the GPU configuration's element size",
            "host_cpus": os.cpu_count()}


def graph_timed(fn, launches=20, reps=5):
    """Average milliseconds of one fn() launch replayed from a captured HIP graph of `launches` of them: the host's cost
    of a call drops out, what is left is the kernels' own time and the gaps the hardware leaves between them."""
    fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(launches):
            fn()
    ms = timed(graph.replay, reps, 2) / launches
    del graph
    return ms


def append_sweep(pk, device, kind):
    """KV append GB/s against the token count (algorithmic bytes: page bytes written + bf16 inputs read): `us` is
    call to call through the Python module (the host's 7 us a call bound the small sizes), `kernel_us` the same launch
    replayed from a captured graph (the kernel's own time)."""
    hkv, d, found = 8, 128, {}
    store = torch.bfloat16 if kind == "bf16" else torch.float8_e4m3fn
    e = 2 if kind == "bf16" else 1
    n_slots = 1 << 20
    k = torch.zeros(n_slots, hkv, d, dtype=store, device=device)
    v = torch.zeros_like(k)
    g = torch.Generator(device=device).manual_seed(1)
    for T in (64, 1024, 4152, 16384, 65536, 262144):
        keys = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
        values = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
        slots = torch.randperm(n_slots, device=device, generator=g)[:T]
        call = lambda: pk.write(keys, values, slots, k, v, kind, multipliers=(0.02, 0.03))
        ms = timed(call, 20, 3)
        kernel = graph_timed(call)
        nbytes = T * hkv * 2 * d * (e + 2)
        found[str(T)] = {"us": round(ms * 1e3, 2), "kernel_us": round(kernel * 1e3, 2),
                         "kernel_frac_of_peak": round(nbytes / kernel / 1e6 / HBM_PEAK_GBPS, 4)}
    return found


def append_rope(pk, device):
    """KV append with the keys' rotary embedding fused in (write's rope=), and with their RMS norm in front of it as
    well (norm=), beside the plain append of the same rows: 8 KV heads x 128, bf16 inputs; bytes as the plain append's
    (the table's rows are read besides: 512 B a token; the norm's 128 weights stay in cache)."""
    hkv, d, found = 8, 128, {}
    n_slots = 1 << 20
    g = torch.Generator(device=device).manual_seed(2)
    angle = torch.arange(8192, dtype=torch.float64, device=device)[:, None] / \
        (10000.0 ** (torch.arange(d // 2, dtype=torch.float64, device=device) / (d // 2)))[None, :]
    table = torch.cat([angle.cos(), angle.sin()], 1).float().contiguous()
    weight = torch.rand(d, device=device, generator=g) + 0.5
    for kind in ("bf16", "fp8"):
        store = torch.bfloat16 if kind == "bf16" else torch.float8_e4m3fn
        e = 2 if kind == "bf16" else 1
        k = torch.zeros(n_slots, hkv, d, dtype=store, device=device)
        v = torch.zeros_like(k)
        found[kind] = {}
        for T in (64, 4152, 262144):
            keys = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
            values = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
            slots = torch.randperm(n_slots, device=device, generator=g)[:T]
            positions = torch.randint(0, 8192, (T,), device=device, generator=g)
            plain = timed(lambda: pk.write(keys, values, slots, k, v, kind, multipliers=(0.02, 0.03)), 20, 3)
            fused = timed(lambda: pk.write(keys, values, slots, k, v, kind, multipliers=(0.02, 0.03),
                                           rope=(table, positions)), 20, 3)
            normed = timed(lambda: pk.write(keys, values, slots, k, v, kind, multipliers=(0.02, 0.03),
                                            rope=(table, positions), norm=(weight, 1e-6)), 20, 3)
            nbytes = T * hkv * 2 * d * (e + 2)
            found[kind][str(T)] = {"plain_us": round(plain * 1e3, 2), "rope_us": round(fused * 1e3, 2),
                                   "norm_rope_us": round(normed * 1e3, 2),
                                   "norm_rope_GB/s": round(nbytes / normed / 1e6, 1)}
        del k, v
    return found


def long_context(pk, device):
    """Split-K partitioned decode over long contexts (40 query heads, 8 KV heads, bf16, random page placement in a
    200k-token pool): contiguous splits of `chunk` positions, then the log-sum-exp merge. One layer, one token a row."""
    hq, hkv, d, page, found = 40, 8, 128, 16, {}
    pool_tokens = 200_000 * 4 + 64
    n_pages = pool_tokens // page
    g = torch.Generator(device=device).manual_seed(3)
    k = torch.randn(n_pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    v = torch.randn(n_pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    for batch in (1, 4):
        for ctx in (32_768, 131_072, 200_000):
            width = (ctx + page - 1) // page
            perm = torch.randperm(n_pages, device=device, generator=g)[:batch * width].view(batch, width).to(torch.int32)
            tables = torch.full((batch, (width + 15) // 16 * 16), n_pages, dtype=torch.int32, device=device)
            tables[:, :width] = perm
            q = torch.randn(batch, hq, d, device=device, generator=g).to(torch.bfloat16)
            rows = torch.arange(batch, dtype=torch.int32, device=device)
            firsts = torch.full((batch,), ctx - 1, dtype=torch.int64, device=device)
            out = torch.empty(batch, hq, d, dtype=torch.bfloat16, device=device)
            nbytes = batch * ctx * hkv * 2 * d * 2
            for chunk in (512, 2048):
                parts = pk.flash_parts(tables.shape[1] * page, chunk)
                ws = torch.empty(pk.workspace_floats(batch, hq, parts, d), dtype=torch.float32, device=device)
                call = lambda phases=0: pk.attend(q, k, v, "bf16", tables, rows, rows, firsts, 1, page, flash=True,
                                                  chunk=chunk, out=out, workspace=ws, phases=phases)
                total = timed(call, 10, 2)
                split = timed(lambda: call(1), 10, 2)
                # (GB/s = algorithmic bytes / us: the fractions of the 8 TB/s peak, with the merge and of the split launch alone)
                found[f"B{batch}_ctx{ctx}_chunk{chunk}"] = {
                    "us": round(total * 1e3, 1), "split_us": round(split * 1e3, 1),
                    "frac": round(nbytes / total / 1e6 / HBM_PEAK_GBPS, 3), "split_frac": round(nbytes / split / 1e6 / HBM_PEAK_GBPS, 3)}
            # (the default reader beside them: partitions x pieces, a partition's pieces b, b + P, ... one unit)
            total = timed(lambda: pk.attend(q, k, v, "bf16", tables, rows, rows, firsts, 1, page, out=out), 10, 2)
            found[f"B{batch}_ctx{ctx}_default_reader"] = {"us": round(total * 1e3, 1), "frac": round(nbytes / total / 1e6 / HBM_PEAK_GBPS, 3)}
    return found


def block_sparse(pk, device):
    """Block-sparse decode (attend's blocks=): every row lists k KV blocks of 64 positions, sorted and distinct, out of a
    65,536-token context (32 query heads, 8 KV heads, bf16, random page placement); only the listed blocks are read,
    so the algorithmic bytes are rows x k x 64 positions x KV heads x (D + DV) x 2. One layer, one token a row; the
    caller's 4 partitions (the reference's PIECE_PARTITIONS) and the most the list's pieces allow."""
    hq, hkv, d, page, ctx, bs, found = 32, 8, 128, 16, 65_536, 64, {}
    batch = 64
    width = ctx // page
    n_pages = batch * width
    g = torch.Generator(device=device).manual_seed(5)
    k = torch.randn(n_pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    v = torch.randn(n_pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    tables = torch.randperm(n_pages, device=device, generator=g).view(batch, width).to(torch.int32)
    q = torch.randn(batch, hq, d, device=device, generator=g).to(torch.bfloat16)
    rows = torch.arange(batch, dtype=torch.int32, device=device)
    firsts = torch.full((batch,), ctx - 1, dtype=torch.int64, device=device)
    out = torch.empty(batch, hq, d, dtype=torch.bfloat16, device=device)
    for listed in (16, 64, 256):
        ids = torch.stack([torch.randperm(ctx // bs, device=device, generator=g)[:listed].sort().values for _ in range(batch)])
        blocks = ids.to(torch.int32)
        nbytes = batch * listed * bs * hkv * 2 * d * 2
        for parts in (4, 32):
            ws = torch.empty(pk.workspace_floats(batch, hq, parts, d), dtype=torch.float32, device=device)
            ms = timed(lambda: pk.attend(q, k, v, "bf16", tables, rows, rows, firsts, 1, page, blocks=blocks, block_size=bs,
                                         partitions=parts, out=out, workspace=ws), 10, 2)
            found[f"k{listed}_partitions{parts}"] = {"us": round(ms * 1e3, 1), "GB/s": round(nbytes / ms / 1e6, 1)}
    return found


def mixed_prefill(pk, device):
    """Chunked prefill over paged KV mixed with decode in one batch (32 query heads, 8 KV heads, bf16): 8 chunks of 512
    new tokens on seeded prefixes in [0, 8192] plus 56 decode rows; one layer: append of all 4,152 tokens, one
    prefill launch for the 8 chunks, one decode launch for the 56 rows."""
    hq, hkv, d, page = 32, 8, 128, 16
    gcpu = torch.Generator().manual_seed(5)
    prefixes = torch.randint(0, 8193, (8,), generator=gcpu).tolist()
    ctxs = torch.randint(1024, 8193, (56,), generator=gcpu).tolist()
    lengths = [p + 512 for p in prefixes] + [c + 1 for c in ctxs]
    widths = [(n + page - 1) // page for n in lengths]
    n_pages = int(sum(widths) * 1.25)
    g = torch.Generator(device=device).manual_seed(5)
    k = torch.randn(n_pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    v = torch.randn(n_pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    perm = torch.randperm(n_pages, generator=gcpu)
    tables = torch.full((64, (max(widths) + 15) // 16 * 16), n_pages, dtype=torch.int32)
    at = 0
    for s, w in enumerate(widths):
        tables[s, :w] = perm[at:at + w].to(torch.int32)
        at += w
    T = 8 * 512 + 56
    slots = []
    for s in range(8):
        pos = torch.arange(prefixes[s], prefixes[s] + 512)
        slots.append(tables[s][pos // page].long() * page + pos % page)
    for i, c in enumerate(ctxs):
        slots.append(tables[8 + i][c // page].long().view(1) * page + c % page)
    slots = torch.cat(slots).to(device)
    tables = tables.to(device)
    q = torch.randn(T, hq, d, device=device, generator=g).to(torch.bfloat16)
    nk = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
    nv = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
    out = torch.empty(T, hq, d, dtype=torch.bfloat16, device=device)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    chunk_rows, chunk_starts, chunk_counts = i32(list(range(8))), i32([512 * s for s in range(8)]), i32([512] * 8)
    positions = torch.tensor(prefixes, dtype=torch.int64, device=device)
    d_rows, d_starts = i32(list(range(8, 64))), i32([4096 + i for i in range(56)])
    d_firsts = torch.tensor(ctxs, dtype=torch.int64, device=device)
    parts, piece = pk.partitions(device, hkv, "bf16", d, d), pk.piece_size(d, d, "bf16", hkv)
    ws = torch.empty(pk.workspace_floats(56, hq, parts, d), dtype=torch.float32, device=device)
    append = lambda: pk.write(nk, nv, slots, k, v, "bf16")
    prefill = lambda: pk.prefill_rows(q, k, v, "bf16", tables, chunk_rows, chunk_starts, chunk_counts, positions, 512,
                                      page, out=out)
    decode = lambda: pk.attend(q, k, v, "bf16", tables, d_rows, d_starts, d_firsts, 1, page, partitions=parts,
                               piece=piece, out=out, workspace=ws)
    flops = sum(4 * hq * d * sum(p + t + 1 for t in range(512)) for p in prefixes)
    t_append, t_prefill, t_decode = timed(append, 20, 3), timed(prefill, 10, 2), timed(decode, 20, 3)
    step = timed(lambda: (append(), prefill(), decode()), 10, 2)
    return {"prefixes": prefixes, "prefill_GFLOP": round(flops / 1e9, 1), "prefill_us": round(t_prefill * 1e3, 1),
            "prefill_TFLOP/s": round(flops / t_prefill / 1e9, 1),
            "prefill_frac_of_bf16_mfma_peak": round(flops / t_prefill / 1e9 / 2500.0, 4),
            "append_us": round(t_append * 1e3, 1), "append_tokens": T,
            "append_GB/s": round(T * hkv * 2 * d * 4 / t_append / 1e6, 1),
            "decode_us": round(t_decode * 1e3, 1), "step_us": round(step * 1e3, 1)}


def prefill_by_kind(pk, device):
    """The mixed batch's 8 prompt chunks (512 tokens each on prefixes in [0, 8192]) over pages of every 8-bit kind,
    and over INT8 pages with int8_qk (integer scores)."""
    hq, hkv, d, page = 32, 8, 128, 16
    gcpu = torch.Generator().manual_seed(5)
    prefixes = torch.randint(0, 8193, (8,), generator=gcpu).tolist()
    widths = [(p + 512 + page - 1) // page for p in prefixes]
    n_pages = int(sum(widths) * 1.25)
    perm = torch.randperm(n_pages, generator=gcpu)
    tables = torch.full((8, (max(widths) + 15) // 16 * 16), n_pages, dtype=torch.int32)
    at = 0
    for s, w in enumerate(widths):
        tables[s, :w] = perm[at:at + w].to(torch.int32)
        at += w
    tables = tables.to(device)
    g = torch.Generator(device=device).manual_seed(9)
    q = torch.randn(4096, hq, d, device=device, generator=g).to(torch.bfloat16)
    out = torch.empty_like(q)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    rows, starts, counts = i32(list(range(8))), i32([512 * s for s in range(8)]), i32([512] * 8)
    positions = torch.tensor(prefixes, dtype=torch.int64, device=device)
    flops = sum(4 * hq * d * sum(p + t + 1 for t in range(512)) for p in prefixes)
    found = {}
    for kind in ("fp8", "fp8:row", "int8"):
        store = torch.int8 if kind == "int8" else torch.float8_e4m3fn
        kf = torch.randn(n_pages + 1, page, hkv, d, device=device, generator=g)
        vf = torch.randn(n_pages + 1, page, hkv, d, device=device, generator=g)
        ks = vs = None
        if kind == "fp8":
            k, v = (kf / 0.02).clamp(-448, 448).to(store), (vf / 0.02).clamp(-448, 448).to(store)
        else:
            top = 448.0 if kind == "fp8:row" else 127.0
            ks, vs = kf.abs().amax(-1) / top, vf.abs().amax(-1) / top
            k, v = kf / ks[..., None], vf / vs[..., None]
            k, v = (k.round().to(store), v.round().to(store)) if kind == "int8" else (k.to(store), v.to(store))
        del kf, vf
        for iqk in ((False, True) if kind == "int8" else (False,)):
            call = lambda: pk.prefill_rows(q, k, v, kind, tables, rows, starts, counts, positions, 512, page,
                                           key_scales=ks, value_scales=vs, multipliers=(0.02, 0.02), out=out, int8_qk=iqk)
            t = timed(call, 10, 2)
            found[kind + (" int8_qk" if iqk else "")] = {"us": round(t * 1e3, 1), "TFLOP/s": round(flops / t / 1e9, 1)}
    return found


def pool_bookkeeping(pk, device):
    """The pool's device-side bookkeeping at the 8B shape (32 layers, 8 KV heads x 128, page 16, bf16): a decode step's
    slots, a draft-tree round's move of accepted rows (64 rows, 5 of 8 columns emitted), and copies of 256 shared pages;
    the torch indexing the reference runs for the last two (pages.py:676-683, 861-869) timed beside them. Bytes are those
    read plus those written."""
    layers, hkv, d, page, pages, B, width = 32, 8, 128, 16, 4096, 64, 8
    g = torch.Generator(device=device).manual_seed(5)
    slots = (pages + 1) * page
    k = torch.randn(layers, slots, hkv, d, device=device, generator=g).to(torch.bfloat16)
    v = torch.randn(layers, slots, hkv, d, device=device, generator=g).to(torch.bfloat16)
    table_pages = pages // B
    tables = torch.randperm(pages, device=device, generator=g).to(torch.int32).view(B, table_pages).contiguous()
    capacity = torch.full((B,), table_pages * page, dtype=torch.int64, device=device)
    lengths = torch.randint(100, 900, (B,), device=device, generator=g)
    slot_ids = torch.arange(B, device=device)
    found = {}
    out = torch.empty(B, dtype=torch.int64, device=device)
    ms = timed(lambda: pk.slots_at(tables, capacity, slot_ids, lengths, page, pages, out=out), 50, 3)
    found["slots_at_64_positions_us"] = round(ms * 1e3, 2)
    many = torch.randint(0, table_pages * page, (4152,), device=device, generator=g)
    rows = torch.randint(0, B, (4152,), device=device, generator=g)
    ms = timed(lambda: pk.slots_at(tables, capacity, slot_ids, many, page, pages, rows=rows), 50, 3)
    found["slots_at_4152_positions_us"] = round(ms * 1e3, 2)
    # a decode step's buffers (slots, window entries, tables) and the round's lengths, on the device, beside the host's
    # way of building the same step (Python lists -> pinned tensors -> six copies: pages.py:359-397)
    buffers = pk.StepBuffers(B, B, table_pages, pages, device)
    start = torch.zeros(B, dtype=torch.int64, device=device)
    ones = torch.ones(B, dtype=torch.int64, device=device)
    ms = timed(lambda: pk.step_buffers(buffers, tables, capacity, lengths, slot_ids, page, 16), 50, 3)
    found["step_buffers_64_rows"] = {"us": round(ms * 1e3, 2)}
    ms = graph_timed(lambda: pk.step_buffers(buffers, tables, capacity, lengths, slot_ids, page, 16))
    found["step_buffers_64_rows"]["kernel_us"] = round(ms * 1e3, 2)
    ms = timed(lambda: pk.commit_round(lengths, start, ones, lengths), 50, 3)
    found["commit_round_64_rows_us"] = round(ms * 1e3, 2)
    host_tables, host_lengths = tables.tolist(), lengths.tolist()
    h_slots = torch.zeros(B, dtype=torch.int64, pin_memory=True)
    h_meta = torch.zeros(B, 4, dtype=torch.int64, pin_memory=True)
    h_tables = torch.zeros(B, table_pages, dtype=torch.int32, pin_memory=True)

    def host_step():
        slots_l = [host_tables[r][host_lengths[r] // page] * page + host_lengths[r] % page for r in range(B)]
        h_slots.copy_(torch.tensor(slots_l, dtype=torch.int64))
        for r in range(B):
            h_meta[r] = torch.tensor([r, 1, host_lengths[r], r], dtype=torch.int64)
            h_tables[r] = torch.tensor(host_tables[r], dtype=torch.int32)
        buffers.d_slots.copy_(h_slots, non_blocking=True)
        buffers.d_starts.copy_(h_meta[:, 0], non_blocking=True)
        buffers.d_counts.copy_(h_meta[:, 1], non_blocking=True)
        buffers.d_firsts.copy_(h_meta[:, 2], non_blocking=True)
        buffers.d_offsets.copy_(h_meta[:, 3], non_blocking=True)
        buffers.d_tables.copy_(h_tables, non_blocking=True)
    ms = timed(host_step, 10, 2)
    found["step_buffers_64_rows"]["host_lists_and_copies_us"] = round(ms * 1e3, 2)
    path = torch.tensor([0, 2, 3, 5, 6, -1, -1, -1], device=device).repeat(B, 1)
    emitted = torch.full((B,), 5, dtype=torch.int64, device=device)
    moved = torch.zeros(B, dtype=torch.int64, device=device)

    def compact():
        moved.zero_()
        pk.compact([k, v], slots, tables, capacity, lengths, emitted, path, moved, page, pages)
    nbytes = B * 4 * hkv * d * 2 * layers * 2 * 2
    ms = timed(compact, 20, 3)
    found["compact_64_rows_4_moves"] = {"us": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1)}
    columns = torch.arange(width, device=device)
    keep = (columns[None, :] < emitted[:, None]) & (columns[None, :] > 0) & (path >= 0)
    where = lambda p: pk.slots_at(tables, capacity, slot_ids[:, None].expand(B, width).contiguous(), p.contiguous(), page, pages)
    source = where(torch.where(keep, lengths[:, None] + path, -1)).reshape(-1)
    target = where(torch.where(keep, lengths[:, None] + columns[None, :], -1)).reshape(-1)

    def torch_compact():
        for flat in (k, v):
            flat.index_copy_(1, target, flat.index_select(1, source))
    ms = timed(torch_compact, 5, 1)
    found["compact_64_rows_4_moves"]["torch_indexing_us"] = round(ms * 1e3, 2)
    n = 256
    ids = torch.randperm(pages, device=device, generator=g)
    source, target = ids[:n].contiguous(), ids[n:2 * n].contiguous()
    nbytes = n * page * hkv * d * 2 * layers * 2 * 2
    ms = timed(lambda: pk.copy_pages([k, v], slots, source, target, page), 20, 3)
    found["copy_256_pages"] = {"us": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1)}
    kp, vp = k.view(layers, pages + 1, page, hkv, d), v.view(layers, pages + 1, page, hkv, d)
    pairs = list(zip(source.tolist(), target.tolist()))

    def torch_copies():
        for a, b in pairs:
            kp[:, b].copy_(kp[:, a])
            vp[:, b].copy_(vp[:, a])
    ms = timed(torch_copies, 3, 1)
    found["copy_256_pages"]["torch_page_by_page_us"] = round(ms * 1e3, 2)
    # rows read back (KVPool.gather / rows_at): 262,144 rows of one layer at random slots, bf16 pages to bf16 and FP8
    # pages to bf16 and FP32; bytes read + written
    del kp, vp, v
    n = 262144
    where = torch.randint(0, slots, (n,), device=device, generator=g)
    k16, v16 = k[0], k[1]
    k8, v8 = k[2].view(torch.float8_e4m3fn)[:, :, :d].contiguous(), k[3].view(torch.float8_e4m3fn)[:, :, :d].contiguous()
    for name, kk, vv, kind, e, dtype in (("bf16_to_bf16", k16, v16, "bf16", 2, torch.bfloat16),
                                         ("fp8_to_bf16", k8, v8, "fp8", 1, torch.bfloat16),
                                         ("fp8_to_fp32", k8, v8, "fp8", 1, torch.float32)):
        out = (torch.empty(n, hkv, d, dtype=dtype, device=device), torch.empty(n, hkv, d, dtype=dtype, device=device))
        ms = timed(lambda: pk.rows_at(kk, vv, kind, where, multipliers=(0.02, 0.03), dtype=dtype, out=out), 20, 3)
        nbytes = n * hkv * 2 * d * (e + out[0].element_size())
        found[f"rows_at_262144_{name}"] = {"us": round(ms * 1e3, 2), "GB/s": round(nbytes / ms / 1e6, 1)}
    return found


def latent_decode(device):
    """Latent-attention (MLA) decode at DeepSeek's geometry (rank 512, rotary 64, page 64): 64 rows of one token at
    contexts ~U[1024, 8192], for the 16 heads a GPU of eight holds and for all 128, BF16 and E4M3 (one scale a row: a
    KV pool's fp8:row pages) caches. Bytes: the cache rows read once (the algorithmic figure); flops: 2 (2 R + P) a
    position and head. The split launch alone (phases=1) and with its merge, replayed from a captured graph. At 128
    heads the many-heads kernel reads (tile_rows 128); the rows `*_128_heads_by_tile_rows` set it against the small
    tiles at 64, 8 and 1 batch rows, which is the trade its default makes."""
    import crit_amd.latent_attention as la
    R, P, page, B = 512, 64, 64, 64
    lengths = torch.randint(1024, 8193, (B,), generator=torch.Generator().manual_seed(7)).tolist()
    held = [math.ceil((n + 1) / page) for n in lengths]
    width = (max(held) + 15) // 16 * 16
    pages = sum(held) + 1
    g = torch.Generator(device=device).manual_seed(21)
    order = torch.randperm(pages - 1, device=device, generator=g).to(torch.int32)
    tables = torch.full((B, width), pages - 1, dtype=torch.int32, device=device)
    at = 0
    for s, w in enumerate(held):
        tables[s, :w] = order[at:at + w]
        at += w
    rows = torch.arange(B, dtype=torch.int32, device=device)
    firsts = torch.tensor(lengths, dtype=torch.int64, device=device)
    total = sum(n + 1 for n in lengths)
    layers = 4      # caches of different memory, read in turn: 4 x 330 MB (BF16) against 256 MB of MALL, so every launch is cold
    found = {"positions": total, "piece": la.PIECE, "layers_read_in_turn": layers}
    values = [torch.randn(pages, page, R + P, device=device, generator=g) * 0.5 for _ in range(layers)]
    for kind in ("bf16", "fp8_row_scales"):
        if kind == "bf16":
            caches, scales, e = [v.to(torch.bfloat16) for v in values], [None] * layers, 2
        else:
            scales = [(v.abs().amax(-1, keepdim=True) / 448.0).clamp(min=1e-30).contiguous() for v in values]
            caches, e = [(v / s).clamp(-448, 448).to(torch.float8_e4m3fn) for v, s in zip(values, scales)], 1
        for heads in (16, 128):
            q = (torch.randn(B, heads, R + P, device=device, generator=g) * 0.5).to(torch.bfloat16)
            out = torch.empty(B, heads, R, dtype=torch.bfloat16, device=device)

            def call(phases=0):
                for cache, sc in zip(caches, scales):
                    la.attend(q, cache, tables, rows, rows, firsts, 1, page, rank=R, out=out, scales=sc, phases=phases)
            call()
            split = graph_timed(lambda: call(1), 3) / layers
            both = graph_timed(call, 3) / layers
            nbytes, flops = total * (R + P) * e, total * heads * 2 * (2 * R + P)
            tiles = la.tile_rows(heads, R, P, page, int(kind != "bf16"))
            found[f"{kind}_{heads}_heads"] = {
                "tile_rows": tiles, "piece": la.PIECE_MANY_HEADS if tiles == 128 else la.PIECE,
                "partitions": la.partitions(device, heads, R, P, page, int(kind != "bf16")), "split_us": round(split * 1e3, 1),
                "with_merge_us": round(both * 1e3, 1), "split_GB/s": round(nbytes / split / 1e6, 1),
                "split_frac_of_hbm_peak": round(nbytes / split / 1e6 / HBM_PEAK_GBPS, 4),
                "split_TFLOP/s": round(flops / split / 1e9, 1),
                "split_frac_of_bf16_mfma_peak": round(flops / split / 1e9 / 2500.0, 4)}
            if heads == 128:
                trade = {}
                for n in (64, 8, 1):
                    for tiles in (128, 16):
                        def some(phases=0):
                            for cache, sc in zip(caches, scales):
                                la.attend(q[:n], cache, tables, rows[:n], rows[:n], firsts[:n], 1, page, rank=R, out=out[:n],
                                          scales=sc, phases=phases, tile_rows=tiles)
                        some()
                        trade[f"{n}_rows_tile_rows_{tiles}_us"] = round(graph_timed(some, 3) / layers * 1e3, 1)
                found[f"{kind}_128_heads_by_tile_rows"] = trade
        del caches, scales
    return found


def index_selection(device):
    """Sparse index selection at DeepSeek-V3.2's indexer geometry (64 heads of 128, the 2,048 best keys): scores and
    top-k over 8,192 and 50,000 keys for 1, 4, 256 and 2,048 tokens near the end of the keys, BF16 and E4M3 keys, each
    call replayed from a captured graph. Scores: 2 H D flops a token and key on the matrix pipe; top-k: a token's scores
    read five times (4 digit passes and the ordered pass), from L2 after the first."""
    import crit_amd.sparse_indexer as si
    H, D, K = 64, 128, 2048
    g = torch.Generator(device=device).manual_seed(17)
    found = {"heads": H, "dim": D, "k": K}
    for n in (8192, 50000):
        keys = (torch.randn(n, D, device=device, generator=g) * 0.5).to(torch.bfloat16)
        key_scales = (keys.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        codes = (keys.float() / key_scales[:, None]).to(torch.float8_e4m3fn)
        for tokens in (1, 4, 256, 2048):
            q = (torch.randn(tokens, H, D, device=device, generator=g) * 0.5).to(torch.bfloat16)
            w = torch.randn(tokens, H, device=device, generator=g) * H ** -0.5
            ends = (n - torch.randint(0, 64, (tokens,), device=device, generator=g)).to(torch.int32)
            s = torch.empty(tokens, n, dtype=torch.float32, device=device)
            picked = torch.empty(tokens, K, dtype=torch.int32, device=device)
            launches = 20 if tokens <= 4 else 3
            bf16 = graph_timed(lambda: si.scores(q, keys, w, ends, out=s), launches)
            fp8 = graph_timed(lambda: si.scores(q, codes, w, ends, key_scales=key_scales, out=s), launches)
            top = graph_timed(lambda: si.topk(s, ends, K, out=picked), launches)
            flops = 2.0 * tokens * n * H * D
            found[f"{n}_keys_{tokens}_tokens"] = {
                "scores_bf16_us": round(bf16 * 1e3, 1), "scores_e4m3_us": round(fp8 * 1e3, 1),
                "scores_bf16_TFLOP/s": round(flops / bf16 / 1e9, 1), "topk_us": round(top * 1e3, 1)}
    # A decode step's shape: every sequence's one token over its own keys, read in place from a store of pages of 64
    # rows at random places (slots [sequences][n]): HBM-bound, a key row read once.
    n, page = 49984, 64
    for sequences in (16, 64):
        rows = sequences * n
        store = (torch.randn(rows, D, device=device, generator=g) * 0.5).to(torch.bfloat16)
        store_scales = (store.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        codes = (store.float() / store_scales[:, None]).to(torch.float8_e4m3fn)
        pages = torch.randperm(rows // page, device=device, generator=g)[:sequences * (n // page)].view(sequences, -1)
        slots = (pages[:, :, None] * page + torch.arange(page, device=device)[None, None, :]).reshape(sequences, n)
        slots = slots.to(torch.int32).contiguous()
        q = (torch.randn(sequences, H, D, device=device, generator=g) * 0.5).to(torch.bfloat16)
        w = torch.randn(sequences, H, device=device, generator=g) * H ** -0.5
        ends = (n - torch.randint(0, 64, (sequences,), device=device, generator=g)).to(torch.int32)
        s = torch.empty(sequences, n, dtype=torch.float32, device=device)
        picked = torch.empty(sequences, K, dtype=torch.int32, device=device)
        bf16 = graph_timed(lambda: si.scores(q, store, w, ends, out=s, slots=slots), 5)
        fp8 = graph_timed(lambda: si.scores(q, codes, w, ends, key_scales=store_scales, out=s, slots=slots), 5)
        top = graph_timed(lambda: si.topk(s, ends, K, out=picked), 5)
        found[f"decode_step_{sequences}_sequences_of_{n}_keys_in_place"] = {
            "scores_bf16_us": round(bf16 * 1e3, 1), "scores_bf16_GB/s_of_key_rows": round(rows * D * 2 / bf16 / 1e6, 1),
            "scores_e4m3_us": round(fp8 * 1e3, 1), "scores_e4m3_GB/s_of_key_rows": round(rows * D / fp8 / 1e6, 1),
            "topk_us": round(top * 1e3, 1)}
        del store, codes, slots
    return found


def reference_shapes(pk, device, only=None):
    """The shapes the reference publishes its decode and append rows on (its paged-kv-attention README: 24 query / 4 KV
    heads x 256 over `fp8:row` pages of 64, 24 / 2 x 256 bf16, 56 / 8 x 128 int8 row-scaled; 1 and 8 rows; 1, 5 and 8
    columns; 4K, 16K and 200K positions; `write` of 1 / 256 / 4,096 tokens into 8,192 shuffled slots), one layer,
    replayed from a captured graph over four caches read in turn (each launch cold), each with its fraction of the
    8 TB/s HBM peak. The reference's own figures are for another card (RTX 5090) and are context, not a target. Widths
    256-wide heads take the matrix-core kernel in two 128-wide halves, 56 / 8 x 128 as the 128-wide pools do. `only`
    (--shape): run just the rows whose name contains it, for a profile of one shape."""
    found = {}
    g = torch.Generator(device=device).manual_seed(11)
    shapes = (("24q_4kv_x256_fp8row_page64", 24, 4, 256, 64, "fp8:row"), ("24q_2kv_x256_bf16_page16", 24, 2, 256, 16, "bf16"),
              ("56q_8kv_x128_int8_page16", 56, 8, 128, 16, "int8"))
    for name, hq, hkv, d, page, kind in shapes:
        e = 2 if kind == "bf16" else 1
        store = torch.bfloat16 if kind == "bf16" else (torch.int8 if kind == "int8" else torch.float8_e4m3fn)
        for ctx, rows_cases in ((4096, ((1, 1), (8, 1))), (16384, ((1, 1), (8, 1))), (200_000, ((1, 1), (1, 5), (1, 8), (8, 1)))):
            if only:
                rows_cases = tuple(c for c in rows_cases if only in f"{name}_{c[0]}_rows_{c[1]}_cols_ctx{ctx}")
                if not rows_cases:
                    continue
            most = max(b for b, _ in rows_cases)
            width = ((ctx + 8 + page - 1) // page + 15) // 16 * 16
            pages = most * width
            layers = 4 if pages * page * hkv * d * e * 2 < (1 << 30) else 2      # (caches read in turn: every launch cold)
            caches = []
            for _ in range(layers):
                if kind == "bf16":
                    k = torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
                    v = torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
                    caches.append((k, v, None, None))
                else:
                    if kind == "int8":
                        k = torch.randint(-100, 100, (pages + 1, page, hkv, d), device=device, dtype=torch.int8, generator=g)
                        v = torch.randint(-100, 100, (pages + 1, page, hkv, d), device=device, dtype=torch.int8, generator=g)
                    else:
                        k = (torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g) * 50).to(store)
                        v = (torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g) * 50).to(store)
                    ks = torch.rand(pages + 1, page, hkv, device=device, generator=g) * 0.01 + 0.001
                    caches.append((k, v, ks, ks.clone()))
            tables = torch.randperm(pages, device=device, generator=g).to(torch.int32).view(most, width).contiguous()
            for batch, columns in rows_cases:
                rows = torch.arange(batch, dtype=torch.int32, device=device)
                starts = rows * columns
                firsts = torch.full((batch,), ctx - columns, dtype=torch.int64, device=device)
                q = torch.randn(batch * columns, hq, d, device=device, generator=g).to(torch.bfloat16)
                out = torch.empty_like(q)
                at = [0]

                def launch(piece=None):
                    at[0] = (at[0] + 1) % layers
                    k, v, ks, vs = caches[at[0]]
                    pk.attend(q, k, v, kind, tables, rows, starts, firsts, columns, page, out=out, key_scales=ks,
                              value_scales=vs, piece=piece)
                ms = graph_timed(launch, 8)
                nbytes = batch * ctx * hkv * (2 * d * e + (8 if kind != "bf16" else 0))
                found[f"{name}_{batch}_rows_{columns}_cols_ctx{ctx}"] = {
                    "us": round(ms * 1e3, 1), "frac_of_hbm_peak": round(nbytes / ms / 1e6 / HBM_PEAK_GBPS, 3)}
                if batch == 1 and columns == 1 and ctx <= 16384:
                    # (one short row: what an engine of single sequences gets with the reference's own largest piece, 128
                    # positions, instead of the default, which is sized for full batches)
                    found[f"{name}_{batch}_rows_{columns}_cols_ctx{ctx}"]["piece_128_us"] = round(graph_timed(lambda: launch(128), 8) * 1e3, 1)
            del caches
            torch.cuda.empty_cache()
    # prefill(): one chunk of 16 / 256 / 2,048 tokens after 1,024 positions, bf16 24 / 2 x 256 (the reference's prefill rows)
    hq, hkv, d, page = 24, 2, 256, 16
    pages = (1024 + 2048) // page + 16
    k = torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    v = torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g)
    table = torch.randperm(pages, device=device, generator=g).to(torch.int32)
    for T in (16, 256, 2048):
        if only and only not in f"prefill_{T}_tokens_after_1024_bf16_24q_2kv_x256":
            continue
        q = torch.randn(T, hq, d, device=device, generator=g).to(torch.bfloat16)
        out = torch.empty_like(q)
        position = torch.tensor([1024], dtype=torch.int64, device=device)
        ms = graph_timed(lambda: pk.prefill(q, k, v, "bf16", table, position, page, out=out), 8)
        flops = 4 * hq * d * sum(1024 + t + 1 for t in range(T))
        found[f"prefill_{T}_tokens_after_1024_bf16_24q_2kv_x256"] = {
            "us": round(ms * 1e3, 1), "TFLOP/s": round(flops / ms / 1e9, 1), "frac_of_bf16_mfma_peak": round(flops / ms / 1e9 / 2500.0, 4)}
    # write(): tokens into 8,192 shuffled slots, bf16 24 / 2 x 256 (the reference's append row)
    hkv, d = 2, 256
    k = torch.zeros(8192, hkv, d, dtype=torch.bfloat16, device=device)
    v = torch.zeros_like(k)
    for T in (1, 256, 4096):
        if only and only not in f"write_{T}_tokens_into_8192_slots_bf16_2kv_x256":
            continue
        keys = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
        values = torch.randn(T, hkv, d, device=device, generator=g).to(torch.bfloat16)
        slots = torch.randperm(8192, device=device, generator=g)[:T]
        ms = graph_timed(lambda: pk.write(keys, values, slots, k, v, "bf16"), 20)
        found[f"write_{T}_tokens_into_8192_slots_bf16_2kv_x256"] = {"us": round(ms * 1e3, 2), "GB/s": round(T * hkv * 2 * d * 4 / ms / 1e6, 1)}
    return found


def narrow_heads(pk, device):
    """Decode over 64-wide heads (32 query / 8 KV heads x 64, the shape of the small models: a step's batch of 64 rows,
    contexts ~U[1024, 8192], pages of 16), which the bandwidth kernel reads in pairs of KV heads as 128-wide ones: the
    split launch alone (`phases=1`) and with its merge, replayed from a captured graph over four layers' caches read in
    turn (each launch cold), BF16 and FP8 pages, each with its fraction of the 8 TB/s HBM peak."""
    found = {}
    g = torch.Generator(device=device).manual_seed(23)
    hq, hkv, d, page, rows = 32, 8, 64, 16, 64
    ctx = torch.randint(1024, 8193, (rows,), generator=torch.Generator().manual_seed(5))
    width = ((8192 + 8 + page - 1) // page + 15) // 16 * 16
    pages = width * rows
    tables = torch.randperm(pages, device=device, generator=g).to(torch.int32).view(rows, width).contiguous()
    r = torch.arange(rows, dtype=torch.int32, device=device)
    firsts = (ctx - 1).to(torch.int64).to(device)
    q = torch.randn(rows, hq, d, device=device, generator=g).to(torch.bfloat16)
    out = torch.empty_like(q)
    for kind, store in (("bf16", torch.bfloat16), ("fp8", torch.float8_e4m3fn)):
        fresh = lambda: (torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g) * 0.5).to(store)
        ks, vs = [fresh() for _ in range(4)], [fresh() for _ in range(4)]
        at = [0]

        def launch(phases):
            at[0] = (at[0] + 1) % 4
            pk.attend(q, ks[at[0]], vs[at[0]], kind, tables, r, r, firsts, 1, page, out=out, multipliers=(0.02, 0.03), phases=phases)
        split = graph_timed(lambda: launch(1), 12)
        both = graph_timed(lambda: launch(0), 12)
        nbytes = int(ctx.sum()) * hkv * 2 * d * (2 if kind == "bf16" else 1)
        found[kind] = {"piece": pk.piece_size(d, d, kind, hkv), "positions": int(ctx.sum()), "split_us": round(split * 1e3, 1),
                       "with_merge_us": round(both * 1e3, 1), "split_GB/s": round(nbytes / split / 1e6, 1),
                       "split_frac_of_hbm_peak": round(nbytes / split / 1e6 / HBM_PEAK_GBPS, 4)}
        del ks, vs
        torch.cuda.empty_cache()
    return found


def known_traffic(pk, device):
    """Two launches of known HBM traffic for scaling the FETCH_SIZE and WRITE_SIZE counters of a profile of one of the
    --*-only runs (with --calibrate): stream_read_kernel over 512 MiB, and write_rows of 262,144 tokens of 8 KV heads x
    128 (BF16 to BF16 pages)."""
    data = torch.zeros(512 << 20, dtype=torch.uint8, device=device)
    sink = torch.zeros(64, device=device)
    pk.stream_read(data, sink)
    T, hkv, d = 262144, 8, 128
    ck = torch.zeros(1 << 20, hkv, d, dtype=torch.bfloat16, device=device)
    cv = torch.zeros_like(ck)
    keys = torch.randn(T, hkv, d, device=device).to(torch.bfloat16)
    values = torch.randn(T, hkv, d, device=device).to(torch.bfloat16)
    slots = torch.randperm(1 << 20, device=device)[:T]
    pk.write(keys, values, slots, ck, cv, "bf16")
    torch.cuda.synchronize()
    log(f"[bench] calibration: stream_read_kernel reads {data.numel()} bytes a launch; write_rows of {T} tokens reads "
        f"{2 * T * hkv * d * 2 + T * 8} bytes and writes {2 * T * hkv * d * 2} bytes")


def verify_windows(pk, device):
    """Verify windows of a draft (8B shape, 32 query / 8 KV heads x 128, pages of 16): 64 rows at contexts ~U[1024, 8192],
    each a window of 1, 4, 5 or 8 columns, bf16 and fp8 pages; microseconds a launch (split + merge) over four layers of
    different memory, replayed from a captured graph. The rows are read once for four tiles of 16-bit pages (two of
    FP8 pages) a workgroup; one column is the decode step for comparison."""
    hq, hkv, d, page, B, found = 32, 8, 128, 16, 64, {}
    g = torch.Generator(device=device).manual_seed(5)
    ctx = torch.randint(1024, 8193, (B,), generator=torch.Generator().manual_seed(1))
    held = [(int(n) + 8 + page - 1) // page for n in ctx]
    width = (max(held) + 15) // 16 * 16
    pages = sum(held) + 1
    order = torch.randperm(pages, device=device, generator=g).to(torch.int32)
    tables = torch.full((B, width), pages, dtype=torch.int32, device=device)
    at = 0
    for s, w in enumerate(held):
        tables[s, :w] = order[at:at + w]
        at += w
    rows = torch.arange(B, dtype=torch.int32, device=device)
    for kind in ("bf16", "fp8"):
        store = torch.bfloat16 if kind == "bf16" else torch.float8_e4m3fn
        ks = [(torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g) * 0.5).to(store) for _ in range(4)]
        vs = [(torch.randn(pages + 1, page, hkv, d, device=device, dtype=torch.bfloat16, generator=g) * 0.5).to(store) for _ in range(4)]
        for columns in (1, 4, 5, 8):
            starts = rows * columns
            firsts = (ctx - columns).to(torch.int64).to(device)
            q = torch.randn(B * columns, hq, d, device=device, generator=g).to(torch.bfloat16)
            out = torch.empty_like(q)
            i = [0]

            def launch():
                i[0] = (i[0] + 1) % 4
                pk.attend(q, ks[i[0]], vs[i[0]], kind, tables, rows, starts, firsts, columns, page, out=out,
                          multipliers=(0.02, 0.03))
            found[f"{kind}_{columns}_columns_us"] = round(graph_timed(launch, 8) * 1e3, 1)
        del ks, vs
        torch.cuda.empty_cache()
    return found


def small_batches(pk, device):
    """What a piece costs a batch that does not fill the chip: one layer's decode launch (split + merge, 8B shape) for
    4 sequences of about 2,000 positions and for one of 8,000, at the default piece and at pieces of 256 positions
    (attend's piece=, the plugin's `piece` option: fixed per pool either way). Microseconds a launch over four layers of
    different memory, replayed from a captured graph (the host's cost of a call is not in the figure)."""
    hq, hkv, d, page, found = 32, 8, 128, 16, {}
    g = torch.Generator(device=device).manual_seed(3)
    for kind in ("bf16", "fp8"):
        store = torch.bfloat16 if kind == "bf16" else torch.float8_e4m3fn
        for name, lengths in (("4_rows_of_2000", [1900, 2000, 2100, 2048]), ("1_row_of_8000", [8000])):
            B = len(lengths)
            width = ((max(lengths) + page) // page + 15) // 16 * 16
            pages = B * width
            k = (torch.randn(4, pages + 1, page, hkv, d, device=device, generator=g) * 0.5).to(store)
            v = (torch.randn(4, pages + 1, page, hkv, d, device=device, generator=g) * 0.5).to(store)
            tables = torch.randperm(pages, device=device, generator=g).to(torch.int32).view(B, width).contiguous()
            rows = torch.arange(B, dtype=torch.int32, device=device)
            firsts = torch.tensor(lengths, dtype=torch.int64, device=device)
            q = torch.randn(B, hq, d, device=device, generator=g).to(torch.bfloat16)
            out = torch.empty_like(q)
            at = [0]

            def launch(piece):
                at[0] = (at[0] + 1) % 4
                pk.attend(q, k[at[0]], v[at[0]], kind, tables, rows, rows, firsts, 1, page, out=out, piece=piece,
                          multipliers=(0.02, 0.03))
            default = pk.piece_size(d, d, kind, hkv)
            found[f"{kind}_{name}"] = {f"piece_{default}_us": round(graph_timed(lambda: launch(default), 16) * 1e3, 1),
                                       "piece_256_us": round(graph_timed(lambda: launch(256), 16) * 1e3, 1)}
    return found


def captured_step(pk, device):
    """A decode step of a small batch (4 sequences of about 2,000 positions, 32 layers, 8B shape, bf16) launched eagerly
    and replayed from one HIP graph: slots of the next positions from the bound tables, then append + attention a
    layer, nothing read on the host; the lengths grow on the device between steps. At the default piece and at pieces of
    256 positions (small_batches())."""
    layers, hq, hkv, d, page, B = 32, 32, 8, 128, 16, 4
    pages_each = 160
    pages = B * pages_each
    g = torch.Generator(device=device).manual_seed(6)
    k = (torch.randn(layers, pages + 1, page, hkv, d, device=device, generator=g) * 0.5).to(torch.bfloat16)
    v = (torch.randn(layers, pages + 1, page, hkv, d, device=device, generator=g) * 0.5).to(torch.bfloat16)
    tables = torch.randperm(pages, device=device, generator=g).to(torch.int32).view(B, pages_each).contiguous()
    capacity = torch.full((B,), pages_each * page, dtype=torch.int64, device=device)
    lengths = torch.tensor([1900, 2000, 2100, 2048], dtype=torch.int64, device=device)
    slot_ids = torch.arange(B, dtype=torch.int64, device=device)
    starts = torch.arange(B, dtype=torch.int32, device=device)
    keys = torch.randn(layers, B, hkv, d, device=device, generator=g).to(torch.bfloat16)
    values = torch.randn(layers, B, hkv, d, device=device, generator=g).to(torch.bfloat16)
    q = torch.randn(layers, B, hq, d, device=device, generator=g).to(torch.bfloat16)
    out = torch.empty(layers, B, hq, d, dtype=torch.bfloat16, device=device)
    slots = torch.empty(B, dtype=torch.int64, device=device)
    parts = pk.partitions(device, hkv, "bf16", d, d)
    workspace = torch.empty(pk.workspace_floats(B, hq, parts, d), dtype=torch.float32, device=device)
    one = torch.ones(B, dtype=torch.int64, device=device)

    found = {"layers": layers, "batch": B, "launches": 1 + layers * 3 + 1}
    for piece in (pk.piece_size(d, d, "bf16", hkv), 256):
        def step():
            pk.slots_at(tables, capacity, slot_ids, lengths, page, pages, out=slots)
            for layer in range(layers):
                pk.write(keys[layer], values[layer], slots, k[layer], v[layer], "bf16")
                pk.attend(q[layer], k[layer], v[layer], "bf16", tables, slot_ids, starts, lengths, 1, page,
                          out=out[layer], workspace=workspace, piece=piece)
            lengths.add_(one)
        step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        found[f"piece_{piece}"] = {"eager_ms": round(timed(step, 20, 2), 3), "graph_replay_ms": round(timed(graph.replay, 20, 2), 3)}
        del graph
    return found


def prefill_fresh(pk, device):
    """The mixed batch's 8 prompt chunks over FP8 pages (one multiplier pair), once reading every position from the
    pages and once with fresh=: each chunk's own 512 positions from 16-bit rows as the projections gave them, its
    prefix from the pages (two launches through the rows' states)."""
    hq, hkv, d, page = 32, 8, 128, 16
    gcpu = torch.Generator().manual_seed(5)
    prefixes = torch.randint(0, 8193, (8,), generator=gcpu).tolist()
    widths = [(p + 512 + page - 1) // page for p in prefixes]
    n_pages = int(sum(widths) * 1.25)
    g = torch.Generator(device=device).manual_seed(7)
    k = (torch.randn(n_pages + 1, page, hkv, d, device=device, generator=g) / 0.02).clamp(-448, 448).to(torch.float8_e4m3fn)
    v = (torch.randn(n_pages + 1, page, hkv, d, device=device, generator=g) / 0.02).clamp(-448, 448).to(torch.float8_e4m3fn)
    perm = torch.randperm(n_pages, generator=gcpu)
    tables = torch.full((8, (max(widths) + 15) // 16 * 16), n_pages, dtype=torch.int32)
    at = 0
    for s, w in enumerate(widths):
        tables[s, :w] = perm[at:at + w].to(torch.int32)
        at += w
    tables = tables.to(device)
    q = torch.randn(4096, hq, d, device=device, generator=g).to(torch.bfloat16)
    fk = torch.randn(4096, hkv, d, device=device, generator=g).to(torch.bfloat16)
    fv = torch.randn(4096, hkv, d, device=device, generator=g).to(torch.bfloat16)
    out = torch.empty_like(q)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=device)
    rows, starts, counts = i32(list(range(8))), i32([512 * s for s in range(8)]), i32([512] * 8)
    positions = torch.tensor(prefixes, dtype=torch.int64, device=device)
    flops = sum(4 * hq * d * sum(p + t + 1 for t in range(512)) for p in prefixes)
    ws = torch.empty(pk.prefill_state_floats(4096, hq, d), dtype=torch.float32, device=device)
    call = lambda fresh: pk.prefill_rows(q, k, v, "fp8", tables, rows, starts, counts, positions, 512, page,
                                         multipliers=(0.02, 0.02), out=out, fresh=fresh, workspace=ws)
    t_pages, t_fresh = timed(lambda: call(None), 10, 2), timed(lambda: call((fk, fv, None)), 10, 2)
    return {"prefill_GFLOP": round(flops / 1e9, 1), "pages_only_us": round(t_pages * 1e3, 1),
            "pages_only_TFLOP/s": round(flops / t_pages / 1e9, 1), "with_fresh_rows_us": round(t_fresh * 1e3, 1),
            "with_fresh_rows_TFLOP/s": round(flops / t_fresh / 1e9, 1),
            "state_bytes": 2 * 4096 * hq * (d + 4) * 4}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--prefill-only", action="store_true",
                    help="run only the mixed prefill + decode batch of the extras (for counter runs on prefill_kernel)")
    ap.add_argument("--pool-only", action="store_true",
                    help="run only the pool bookkeeping of the extras (slots, the move of accepted rows, page copies)")
    ap.add_argument("--latent-only", action="store_true", help="run only the latent-attention decode of the extras")
    ap.add_argument("--index-only", action="store_true", help="run only the sparse index selection of the extras")
    ap.add_argument("--heads64-only", action="store_true", help="run only the decode over 64-wide heads of the extras")
    ap.add_argument("--shape", default=None, help="with --shapes-only: only the rows whose name contains this")
    ap.add_argument("--append-only", action="store_true",
                    help="run only the KV append with rope and norm fused in beside the plain append (for counter runs on write_rows)")
    ap.add_argument("--shapes-only", action="store_true",
                    help="run only the decode and append rows at the shapes the reference publishes its own on")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one KV append of 262,144 tokens: with the stream-read probe, two kernels of known "
                         "read and write sizes against which FETCH_SIZE / WRITE_SIZE counters are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no cross-GPU part (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (the CPU oracle is a checker, not a product path)")
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    import crit_amd.paged_kv_attention as pk
    if args.prefill_only:
        found = mixed_prefill(pk, device)
        log(f"[bench] mixed prefill + decode: {found}")
        print(json.dumps({"mixed_prefill_decode_bf16": found}), flush=True)
        return
    if args.latent_only:
        found = latent_decode(device)
        log(f"[bench] latent-attention decode: {found}")
        print(json.dumps({"latent_attention_decode": found}), flush=True)
        return
    if args.index_only:
        found = index_selection(device)
        log(f"[bench] sparse index selection: {found}")
        print(json.dumps({"sparse_index_selection": found}), flush=True)
        return
    if args.heads64_only:
        if args.calibrate:
            known_traffic(pk, device)
        found = narrow_heads(pk, device)
        log(f"[bench] decode over 64-wide heads: {found}")
        print(json.dumps({"heads_of_64_decode": found}), flush=True)
        return
    if args.shapes_only:
        found = reference_shapes(pk, device, args.shape)
        log(f"[bench] the reference's published shapes: {found}")
        print(json.dumps({"reference_published_shapes": found}), flush=True)
        return
    if args.append_only:
        found = append_rope(pk, device)
        log(f"[bench] append with rope and norm: {found}")
        print(json.dumps({"append_with_rope_and_norm": found}), flush=True)
        return
    if args.pool_only:
        found = pool_bookkeeping(pk, device)
        log(f"[bench] pool bookkeeping: {found}")
        print(json.dumps({"pool_bookkeeping_bf16": found}), flush=True)
        return
    spec = WORKLOADS[args.workload]
    log(f"[bench] building workload {args.workload}: {spec['name']}")
    w = Workload(spec, device)
    log(f"[bench] {w.tokens} positions, pool {w.n_pages} pages/layer, decode {w.decode_bytes / 1e9:.3f} GB/layer, "
        f"partitions {w.parts}, piece {w.piece}")
    for _ in range(args.warmup):
        w.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        w.step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    step_bytes = (w.decode_bytes + w.append_bytes) * w.layers
    value = step_bytes / ms_per_step / 1e6

    split_ms = kernel_ms(w, 1)
    # (the merge alone, replayed from a captured graph: a 7 us kernel timed call to call would show the host's calls)
    merge_ms = graph_timed(lambda: w.attend(0, 2))
    append_ms = timed(lambda: w.append(0), 50, 5)
    achieved = w.decode_bytes / split_ms / 1e6
    traffic, traffic_source = profiled_traffic(args.workload, w.piece)
    sink = torch.zeros(64, device=device)
    read_ms, read_bytes = None, 0
    for layer in range(min(4, w.layers)):
        flat = w.k[layer].view(torch.uint8).reshape(-1)
        flat = flat[:flat.numel() // 16 * 16]
        ms = timed(lambda: pk.stream_read(flat, sink), 1, 0)
        read_ms, read_bytes = (ms if read_ms is None else min(read_ms, ms)), flat.numel()
    stream_gbps = read_bytes / read_ms / 1e6
    result = {
        "metric": "paged decode attention + KV append, algorithmic HBM GB/s over one 32-layer decode step",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if w.kind == "bf16" else "fp8_e4m3 KV, bf16 q, f32 accumulate", "data": "synthetic",
        "config": {"workload": spec["name"], "positions": w.tokens, "partitions": w.parts, "piece": w.piece},
        "roofline": {"bound": "hbm", "kernel": f"{DECODE_KERNEL} (split launch)", "achieved": round(achieved, 1),
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "launch_ms": round(split_ms, 4), "merge_ms": round(merge_ms, 4),
                     "algorithmic_bytes_per_launch": w.decode_bytes,
                     "stream_read_GB/s": round(stream_gbps, 1)},
        "append": {"us_per_launch": round(append_ms * 1e3, 2), "tokens": spec["batch"],
                   "GB/s": round(w.append_bytes / append_ms / 1e6, 2)},
        "fraction_of_peak": round(value / HBM_PEAK_GBPS, 4),
    }
    log(f"[bench] step {ms_per_step:.3f} ms; split launch {split_ms:.4f} ms = {achieved:.0f} GB/s; merge {merge_ms:.4f} ms; "
        f"append {append_ms * 1e3:.1f} us; stream read {stream_gbps:.0f} GB/s")
    del w
    torch.cuda.empty_cache()
    if args.calibrate:
        T, hkv, d = 262144, 8, 128
        ck = torch.zeros(1 << 20, hkv, d, dtype=torch.bfloat16, device=device)
        cv = torch.zeros_like(ck)
        keys = torch.randn(T, hkv, d, device=device).to(torch.bfloat16)
        values = torch.randn(T, hkv, d, device=device).to(torch.bfloat16)
        slots = torch.randperm(1 << 20, device=device)[:T]
        pk.write(keys, values, slots, ck, cv, "bf16")
        torch.cuda.synchronize()
        log(f"[bench] calibration: stream_read_kernel reads {read_bytes} bytes a launch; write_rows of {T} tokens reads "
            f"{2 * T * hkv * d * 2 + T * 8} bytes and writes {2 * T * hkv * d * 2} bytes")
        del ck, cv, keys, values, slots
        torch.cuda.empty_cache()
    if not args.no_extras:
        extras = {}
        other = "c3" if args.workload == "c2" else "c2"
        ospec = WORKLOADS[other]
        log(f"[bench] the other decode workload at its full size: {other}, {ospec['layers']} layers")
        ow = Workload(ospec, device)
        for _ in range(2):
            ow.step()
        ms = timed(ow.step, 3, 0)
        osplit = kernel_ms(ow, 1)
        otraffic, osource = profiled_traffic(other, ow.piece)
        extras[other] = {"workload": ospec["name"], "layers": ow.layers, "positions": ow.tokens, "piece": ow.piece,
                         "ms_per_step": round(ms, 3), "ms_per_layer": round(ms / ow.layers, 4),
                         "GB/s": round((ow.decode_bytes + ow.append_bytes) * ow.layers / ms / 1e6, 1),
                         "fraction_of_peak": round((ow.decode_bytes + ow.append_bytes) * ow.layers / ms / 1e6 / HBM_PEAK_GBPS, 4),
                         "split_launch_ms": round(osplit, 4), "split_launch_GB/s": round(ow.decode_bytes / osplit / 1e6, 1),
                         "frac": round(ow.decode_bytes / osplit / 1e6 / HBM_PEAK_GBPS, 4)}
        # the other workload's dominant kernel against its roofline, beside the default workload's
        result[f"roofline_{other}"] = {"bound": "hbm", "kernel": f"{DECODE_KERNEL} (split launch)",
                                       "achieved": round(ow.decode_bytes / osplit / 1e6, 1), "peak": HBM_PEAK_GBPS,
                                       "unit": "GB/s", "frac": round(ow.decode_bytes / osplit / 1e6 / HBM_PEAK_GBPS, 4),
                                       "traffic": otraffic, "traffic_source": osource, "launch_ms": round(osplit, 4),
                                       "algorithmic_bytes_per_launch": ow.decode_bytes, "workload": other}
        # the same launches with pieces twice as long (attend's piece=, a deployment's choice through the plugin's
        # `piece` option: fixed per pool like the default; halves the units' fixed costs, and a small batch's units)
        ow.piece *= 2
        olong = kernel_ms(ow, 1)
        extras[other]["split_launch_GB/s_with_pieces_twice_as_long"] = round(ow.decode_bytes / olong / 1e6, 1)
        log(f"[bench] {other}: {extras[other]}")
        del ow
        torch.cuda.empty_cache()
        extras["append_GB/s_by_tokens"] = {kind: append_sweep(pk, device, kind) for kind in ("bf16", "fp8")}
        log(f"[bench] append sweep: {extras['append_GB/s_by_tokens']}")
        extras["append_with_rope"] = append_rope(pk, device)
        log(f"[bench] append with the keys' rope fused in: {extras['append_with_rope']}")
        extras["long_context_splitk_bf16"] = long_context(pk, device)
        log(f"[bench] long context: {extras['long_context_splitk_bf16']}")
        torch.cuda.empty_cache()
        extras["block_sparse_decode_bf16"] = block_sparse(pk, device)
        log(f"[bench] block-sparse decode: {extras['block_sparse_decode_bf16']}")
        extras["mixed_prefill_decode_bf16"] = mixed_prefill(pk, device)
        log(f"[bench] mixed prefill + decode: {extras['mixed_prefill_decode_bf16']}")
        extras["prefill_8bit_pages"] = prefill_by_kind(pk, device)
        log(f"[bench] prefill over 8-bit pages: {extras['prefill_8bit_pages']}")
        extras["prefill_fp8_pages_fresh_rows"] = prefill_fresh(pk, device)
        log(f"[bench] prefill over FP8 pages, with fresh rows: {extras['prefill_fp8_pages_fresh_rows']}")
        torch.cuda.empty_cache()
        extras["reference_published_shapes"] = reference_shapes(pk, device)
        log(f"[bench] the reference's published shapes: {extras['reference_published_shapes']}")
        torch.cuda.empty_cache()
        extras["heads_of_64_decode"] = narrow_heads(pk, device)
        log(f"[bench] decode over 64-wide heads, 32q / 8kv, 64 rows: {extras['heads_of_64_decode']}")
        torch.cuda.empty_cache()
        extras["verify_windows_64_rows"] = verify_windows(pk, device)
        log(f"[bench] verify windows, 64 rows: {extras['verify_windows_64_rows']}")
        torch.cuda.empty_cache()
        extras["small_batches_by_piece"] = small_batches(pk, device)
        log(f"[bench] small batches, default piece and 256: {extras['small_batches_by_piece']}")
        extras["captured_decode_step_bf16"] = captured_step(pk, device)
        log(f"[bench] a small batch's decode step, eager and from one graph: {extras['captured_decode_step_bf16']}")
        extras["pool_bookkeeping_bf16"] = pool_bookkeeping(pk, device)
        log(f"[bench] pool bookkeeping: {extras['pool_bookkeeping_bf16']}")
        torch.cuda.empty_cache()
        extras["latent_attention_decode"] = latent_decode(device)
        log(f"[bench] latent-attention decode: {extras['latent_attention_decode']}")
        extras["sparse_index_selection"] = index_selection(device)
        log(f"[bench] sparse index selection: {extras['sparse_index_selection']}")
        result["extra"] = extras
        # The other kernels' headline fractions, nested in `roofline` beside the dominant kernel's: each entry names its
        # kernel and workload, its time, and the fraction of the peak that bounds it (HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s).
        also = [{"kernel": f"{DECODE_KERNEL} (split launch)", "workload": other, "us": round(osplit * 1e3, 1),
                 "bound": "hbm", "frac": extras[other]["frac"], "traffic": otraffic, "step_frac": extras[other]["fraction_of_peak"]}]
        for kind, sweep in extras["append_GB/s_by_tokens"].items():
            for tokens in ("4152", "16384", "262144"):
                also.append({"kernel": "write_rows", "workload": f"append {tokens} tokens {kind}", "us": sweep[tokens]["kernel_us"],
                             "bound": "hbm", "frac": sweep[tokens]["kernel_frac_of_peak"]})
        mixed = extras["mixed_prefill_decode_bf16"]
        also.append({"kernel": "prefill_kernel", "workload": "c5: 8 chunks x 512 tokens on prefixes up to 8192, bf16",
                     "us": mixed["prefill_us"], "bound": "mfma", "TFLOP/s": mixed["prefill_TFLOP/s"],
                     "frac": mixed["prefill_frac_of_bf16_mfma_peak"]})
        for name, found in extras["latent_attention_decode"].items():
            if isinstance(found, dict) and "split_us" in found:
                also.append({"kernel": "latent_heads_kernel" if found.get("tile_rows") == 128 else "latent_kernel", "workload": f"64 rows ctx~U[1024,8192] rank 512 + rope 64, {name}",
                             "us": found["split_us"], "with_merge_us": found["with_merge_us"], "bound": "hbm",
                             "frac": found["split_frac_of_hbm_peak"], "mfma_frac": found["split_frac_of_bf16_mfma_peak"]})
        for kind, found in extras["heads_of_64_decode"].items():
            also.append({"kernel": f"{DECODE_KERNEL} (split launch, pairs of 64-wide heads)", "workload": f"64 rows ctx~U[1024,8192] 32q/8kv x 64, {kind}",
                         "us": found["split_us"], "with_merge_us": found["with_merge_us"], "bound": "hbm", "frac": found["split_frac_of_hbm_peak"]})
        result["roofline"]["also"] = also
    if not args.no_cpu:
        log("[bench] timing the CPU reference path (about 20 s)")
        result["cpu_baseline"] = cpu_baseline(spec)
        log(f"[bench] cpu: {result['cpu_baseline']}")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
