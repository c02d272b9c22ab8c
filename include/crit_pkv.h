/* crit_pkv: C ABI of the MI355X (gfx950) paged-KV kernels.
 *
 * The boundary a host binds (ctypes, cgo, JNI ...): plain pointers and sizes, one POD parameter struct per entry
 * point, the caller's HIP stream. Every buffer is caller-owned device memory, the counters of a launch included
 * (crit_pkv_attend_params.launch_state): the library keeps no state between calls, so two owners' launches, eager or
 * replayed from captured graphs, never meet in memory neither of them passed. Nothing here allocates, synchronises or
 * reads a length on the host: row lengths and positions are read on the device, so one launch shape (a captured HIP
 * graph) serves every length.
 *
 * Each entry point replaces the kernel launches behind one function of the reference's kernels module
 * (kernels/techniques/attention/paged-kv-attention/torch-ext/paged_kv_attention/__init__.py); the pattern of the ABI
 * (parameter struct mirrored by the host, int error codes, an error-string function, a params-size cross-check)
 * follows the reference's own C ABI for its CUDA tile (cuda_window.cu:1482-1535).
 *
 * Return value of every launch: 0 = launched; > 0 = a HIP runtime error code; < 0 = one of CRIT_PKV_E_* (the launch
 * was refused before anything ran). crit_pkv_error() names any of them.
 */
#ifndef CRIT_PKV_H
#define CRIT_PKV_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CRIT_PKV_ABI_VERSION 20

/* Page kinds: the values of KINDS in the reference module (__init__.py:78). */
#define CRIT_PKV_KIND_16BIT 0   /* bf16 or fp16 pages (page_dtype says which) */
#define CRIT_PKV_KIND_FP8 1     /* E4M3FN codes, value = code * multiplier (per layer, or per KV head) */
#define CRIT_PKV_KIND_FP8_ROW 2 /* E4M3FN codes, one FP32 scale per (slot, KV head) */
#define CRIT_PKV_KIND_INT8 3    /* INT8 codes, one FP32 scale per (slot, KV head) */

/* Element types of 16-bit/32-bit float buffers. */
#define CRIT_PKV_F32 0
#define CRIT_PKV_BF16 1
#define CRIT_PKV_F16 2

#define CRIT_PKV_E_GEOMETRY (-1)    /* shapes the kernels do not take (head dims, group size, columns, page, piece) */
#define CRIT_PKV_E_DTYPE (-2)       /* a dtype/kind combination the kernels do not take */
#define CRIT_PKV_E_NULL (-3)        /* a required pointer is NULL */
#define CRIT_PKV_E_WORKSPACE (-4)   /* partitions/piece/workspace pointers inconsistent */
#define CRIT_PKV_E_SCRATCH (-5)     /* crit_pkv_attend_static: the launch needs more than the static scratch holds */

#define CRIT_PKV_MAX_COLUMNS 64

/* ---- append ------------------------------------------------------------------------------------------------------
 * Replaces write() -> _write_kernel (__init__.py:289-324, _kernels.py:112-150); the torch rule it must reproduce
 * bit for bit is KVPool.write (inference/attention-state/code/pages.py:439-453, 872-895).
 * keys [tokens][kv_heads][head_dim], values [tokens][kv_heads][value_dim]: element (t, h, i) at
 * base + t*stride_t + h*stride_h + i (strides in elements, last dimension contiguous). Pages: any storage laid out
 * [slots][kv_heads][dim]; row (slot, head) starts at (slot*kv_heads + head)*dim. A slot below 0 is skipped.
 * values/value_pages NULL: keys only. */
typedef struct crit_pkv_write_params {
    const void* keys;
    const void* values;             /* NULL: keys only */
    const int64_t* slots;           /* [tokens] */
    void* key_pages;
    void* value_pages;              /* NULL with values NULL */
    float* key_scales;              /* [slots][kv_heads], kinds FP8_ROW and INT8; else NULL */
    float* value_scales;
    const float* head_multipliers;  /* optional [2][kv_heads] FP32 (keys' then values'), kind FP8: overrides the two
                                       scalars below with one multiplier per KV head; NULL: the scalars */
    int64_t tokens;
    int64_t key_stride_t, key_stride_h, value_stride_t, value_stride_h;
    int32_t kv_heads, head_dim, value_dim;
    int32_t kind;                   /* CRIT_PKV_KIND_* */
    int32_t page_dtype;             /* kind 16BIT: CRIT_PKV_BF16 or CRIT_PKV_F16 */
    int32_t in_dtype;               /* CRIT_PKV_F32, _BF16 or _F16: the dtype of keys and values */
    float key_multiplier, value_multiplier;   /* kind FP8: code = e4m3(clamp(x / multiplier, -448, 448)) */
    /* Rotary embedding of the keys on their way in: the reference's rope() (inference/fused-norms/code/
     * torch_norms.py:89-147; called as rope_pair before write by the model plugins) over the whole head width, fused
     * into the append. rope_table NULL: none. Else a [rope_rows][head_dim] FP32 table, cos of every pair then sin
     * (torch_norms.py:104-106), read at rope_positions[t] clamped to its rows; pairs (j, j + head_dim / 2), or
     * (2j, 2j + 1) with rope_interleaved; rope_scale multiplies cos and sin. a cos - b sin and b cos + a sin in
     * FP32, rounded to in_dtype as rope() rounds to its output's type, then appended as given keys would be. Head
     * widths 64, 128, 256; rows 16-byte aligned; values no wider than keys. */
    const float* rope_table;
    const int64_t* rope_positions;  /* [tokens] */
    int64_t rope_rows;
    int32_t rope_interleaved;
    float rope_scale;
    /* RMS norm of each key head in front of the rotation: the reference's rms_norm_rope() (inference/fused-norms/code/
     * torch_norms.py:149-176; the keys' half of rms_norm_rope_pair, :307-316, called at inference/model-template/code/
     * blocks.py:160-170). norm_weight NULL: none. Else FP32 [head_dim], 16-byte aligned, with rope_table: each key head
     * becomes x / sqrt(mean(x^2) + norm_eps) * (norm_weight[i] + norm_offset) in FP32, is rotated in FP32 and rounded
     * once to in_dtype, then appended. The sum of squares is taken in a fixed order (squares rounded one by one, groups
     * of 8 consecutive elements in order, the groups by a balanced tree of adjacent pairs); division, square root and
     * reciprocal are correctly rounded. */
    const float* norm_weight;
    float norm_eps, norm_offset;
} crit_pkv_write_params;

int crit_pkv_write(const crit_pkv_write_params* p, void* stream);

/* ---- decode / verify windows ---------------------------------------------------------------------------------------
 * Replaces attend() -> _window_kernel + _merge_kernel (__init__.py:396-576, _kernels.py:359-478, 558-604) and, with
 * piece = the chunk and partitions = ceil(table positions / chunk), attend(flash=...) (__init__.py:641-712).
 * Row r is counts[r] (<= columns) tokens of one sequence: tokens starts[r].. of q/out, column c at position
 * firsts[r] + c, page table tables[rows[r]]; column c sees positions n <= firsts[r] + c (and n > firsts[r] + c -
 * sliding when sliding > 0). Positions are read in pieces of `piece` positions; piece i belongs to partition
 * i % partitions. Partition b of (row, column, head) writes its unnormalised output, running maximum and sum at
 * index ((prow + c)*heads + head)*partitions + b of the three partial arrays, prow = offsets ? offsets[r] -
 * offsets[0] : r*columns; the merge folds partitions 0 .. min(partitions, ceil((firsts[r]+c+1)/piece)) - 1 in order and
 * writes out (and lse). fused != 0: one launch folds the partitions itself, same bits, no partial arrays. */
typedef struct crit_pkv_attend_params {
    const void* q;                  /* [tokens][heads][head_dim] bf16 or f16 */
    const void* key_pages;
    const void* value_pages;
    const float* key_scales;        /* row-scaled kinds */
    const float* value_scales;
    const float* head_multipliers;  /* optional [2][kv_heads], kind FP8 */
    const int32_t* tables;          /* [S][table_width] */
    const void* rows;               /* [n_rows] int32, or int64 with rows_are_64: the table row of each batch row */
    const int32_t* starts;          /* [n_rows] */
    const int32_t* counts;          /* [n_rows] or NULL: `columns` each */
    const int64_t* firsts;          /* [n_rows] */
    const int32_t* offsets;         /* [n_rows] or NULL */
    float* partial_out;             /* [partial rows * heads * partitions][value_dim] */
    float* partial_max;             /* [partial rows * heads * partitions] (base-2 units) */
    float* partial_sum;
    void* out;                      /* [tokens][heads][value_dim], out_dtype */
    float* lse;                     /* [tokens][heads] or NULL */
    const float* sinks;             /* [heads] or NULL */
    const int32_t* parents;         /* draft trees (_kernels.py:155-165, 325-329): [tokens] int32 ... */
    const int64_t* parents64;       /* ... or int64 (at most one of the two non-NULL): token starts[r] + c holds the
                                       column of its parent in row r's window, -1 for none, parents before children.
                                       Column c then sees every position below firsts[r] and, of the window, the
                                       positions firsts[r] + a of its ancestors a and itself. NULL, NULL: column c
                                       sees positions <= firsts[r] + c. */
    const int32_t* blocks;          /* block-sparse lists (attend's blocks=, _kernels.py:483-556): [tokens][blocks_k] KV
                                       block ids of block_size positions each, -1 for none, no id twice in a list. A
                                       token then sees, of the positions above, only those of its listed blocks, which
                                       are all the launch reads: a list is read as one run of blocks_k * block_size
                                       positions, in pieces of `piece`, piece i in partition i % partitions, and the
                                       merge folds min(partitions, ceil(blocks_k * block_size / piece)) partials.
                                       NULL: every position. Not with fused or sliding. */
    int64_t q_stride_t, q_stride_h, out_stride_t, out_stride_h, table_stride;
    int64_t blocks_stride;          /* elements between two tokens' lists */
    int32_t table_width, n_rows, columns, heads, kv_heads, head_dim, value_dim, page;
    int32_t kind, page_dtype, out_dtype;
    int32_t partitions, piece;
    int32_t fused;
    int32_t sliding;
    int32_t phases;                 /* 0: the split launch then the merge; 1: the split launch only; 2: the merge only
                                       (for timing one kernel; ignored when fused) */
    int32_t blocks_k, block_size;   /* ids a list (1 .. 1024), positions a block (>= 1) */
    float scale, key_multiplier, value_multiplier;
    /* Fresh rows (attend's fresh=, __init__.py:417-421, _kernels.py:272-274, 291-345): row r reads its positions from
     * fresh_firsts[i] on from rows `position - fresh_shifts[i]` of fresh_keys / fresh_values ([fresh_rows][kv_heads][dim]
     * in q's type, each head row contiguous, token rows fresh_stride_k / _v elements apart) instead of the pages,
     * unscaled; i = r with fresh_per_row, else 0 (one shift and first for every row). All four pointers or none. Not
     * with block lists. Such launches take the generic kernel whatever the head width. */
    const void* fresh_keys;
    const void* fresh_values;
    const int64_t* fresh_shifts;
    const int64_t* fresh_firsts;
    int64_t fresh_stride_k, fresh_stride_v, fresh_rows;
    int32_t fresh_per_row;
    /* rows holds int64 entries (a captured round hands the reader its round slots as they are, int64:
     * inference/attention-state/code/device_attention.py:573, core/python/crit_plugins/device.py:661,681). */
    int32_t rows_are_64;
    /* The launch's two counters (next unit, workgroups done): 8 bytes of device memory, 8-byte aligned, zero before the
     * first launch that uses them; a launch leaves them zero when its last workgroup ends. Resident workgroups draw
     * their units of work from them, which keeps every compute unit busy when the rows' lengths differ. Launches that
     * may run at the same time (other streams, another owner's captured graph replaying) take different counters;
     * launches one after another on a stream share theirs. The reference keeps such state per owner in its module
     * (__init__.py:141-171); here it is the caller's, like every other buffer. NULL: units are dealt to the
     * workgroups in turn, no counters (the same bits; slower on ragged batches). */
    uint32_t* launch_state;
    /* Keys derived from the value rows on read (the reference's derive=, paged_kv_attention/__init__.py:52-58, 82-121):
     * a layer that caches one row a position and KV head reads it as its value and, normed and rotated, as its key:
     * k = rope(rms_norm(r) * weight, position), r the row as stored (codes times their scale or multiplier),
     * rms_norm(r) = r / sqrt(mean(r * r) + derive_eps), the "half" rotation over the first derive_rot values at the
     * angle fp32(position) * freqs[i], all in FP32. derive_table: FP32 freqs [derive_rot / 2], then, with
     * derive_weighted, the weight [head_dim]; NULL: keys from key_pages. With it key_pages and key_scales are not
     * read (may be NULL); head_dim == value_dim; derive_rot any even width from 2 up to head_dim; no blocks. Fresh rows
     * come as values only (fresh_keys NULL): a fresh position's key is derived from its fresh value row. */
    const float* derive_table;
    float derive_eps;
    int32_t derive_rot;
    int32_t derive_weighted;
    /* INT8 pages, fused launches: each query row read as INT8 codes at its own scale (amax / 127, at least 1e-30,
     * rounded half away from zero) and a page position's score as the exact product of the two rows' codes times both
     * scales (prefill's int8_qk, __init__.py:1284-1285, _kernels.py:637-643, 668-671, for the prompt chunks that are
     * read as window rows); fresh positions keep the queries' 16 bits. Not with blocks or derive. Such launches take
     * the generic kernel whatever the head width. */
    int32_t int8_qk;
} crit_pkv_attend_params;

int crit_pkv_attend(const crit_pkv_attend_params* p, void* stream);

/* crit_pkv_attend for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): no counterpart in the reference, whose module allocates its workspaces itself.
 * The same launches and the same bits as crit_pkv_attend, with the partial arrays and the launch counters taken from
 * a static device array of CRIT_PKV_STATIC_SCRATCH_BYTES that the library holds on every GPU it runs on until the
 * process ends; partial_out, partial_max, partial_sum and launch_state of `p` are not read. Inputs and outputs are
 * the caller's as before. Calls nothing that allocates. Refused with CRIT_PKV_E_SCRATCH when 256 + n_rows * columns *
 * heads * partitions * (value_dim + 2) * 4 bytes exceed the array (fused launches need the 256 only). A launch
 * that any check refuses queues nothing on the stream. Precondition the library cannot check (offsets are device
 * memory): with offsets, offsets[r] - offsets[0] + columns <= n_rows * columns for every row, as rows packed by
 * their counts have it; a row past that bound would write its partials beyond the array.
 * Every call on one GPU uses that GPU's one array: calls that may overlap there (two streams, two threads, a graph
 * replaying beside eager calls) race on the partials and the counters; run them one after another. */
#define CRIT_PKV_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)
int crit_pkv_attend_static(const crit_pkv_attend_params* p, void* stream);

/* ---- merge of shard partials ---------------------------------------------------------------------------------------
 * Replaces PartitionedAttention.merge (inference/partitioned-attention/plugin.py:52-64): outs [parts][n][value_dim]
 * (in_dtype), lses [parts][n] FP32 (-inf: the part saw no key) -> out [n][value_dim] FP32, lse [n] FP32, n = tokens
 * * heads. A row no part saw gets zeros and -inf. */
typedef struct crit_pkv_merge_params {
    const void* outs;
    const float* lses;
    float* out;
    float* lse;
    int64_t rows;                   /* tokens * heads */
    int32_t parts, value_dim, in_dtype;
} crit_pkv_merge_params;

int crit_pkv_merge(const crit_pkv_merge_params* p, void* stream);

/* ---- prompt chunks ---------------------------------------------------------------------------------------------------
 * Replaces prefill() -> _prefill_kernel (__init__.py:1245-1332, _kernels.py:610-726), and a batch of them in one
 * launch (the reference launches one per row, device_attention.py:901-916).
 * Chunk i is counts[i] tokens starting at token starts[i] of q/out, at positions positions[i] .. of the sequence whose
 * page table is tables + table_rows[i]*table_stride; token t sees positions n <= positions[i] + t (causal). All
 * metadata is on the device. max_count bounds counts[] (it sizes the grid). */
typedef struct crit_pkv_prefill_params {
    const void* q;
    const void* key_pages;
    const void* value_pages;
    const float* key_scales;
    const float* value_scales;
    const float* head_multipliers;
    const int32_t* tables;          /* int32 page tables, or ... */
    const int64_t* tables64;        /* ... int64 ones (exactly one of the two is non-NULL) */
    const int32_t* table_rows;      /* [chunks] or NULL: chunk i reads table row i */
    const int32_t* starts;          /* [chunks] or NULL: 0 */
    const int32_t* counts;          /* [chunks] or NULL: max_count */
    const int64_t* positions;       /* [chunks] */
    void* out;
    float* lse;                     /* or NULL */
    const float* sinks;             /* or NULL */
    int64_t q_stride_t, q_stride_h, out_stride_t, out_stride_h, table_stride;
    int32_t table_width, chunks, max_count, heads, kv_heads, head_dim, page;
    int32_t kind, page_dtype, out_dtype;
    int32_t sliding;
    float scale, key_multiplier, value_multiplier;
    /* A chunk's own keys and values as the projections gave them (the reference's fresh=, __init__.py:1250-1255,
     * 1301-1308; _kernels.py:616-650): [tokens][kv_heads][head_dim] in q's type, parallel to q's tokens, each head row
     * contiguous, token rows fresh_stride_k / fresh_stride_v elements apart. Chunk i then reads its positions from
     * fresh_firsts[i] on (clamped to the chunk's own positions; NULL: all of them) from these rows, unscaled, and the
     * earlier ones from the pages. Both NULL: every position from the pages. With them, fresh_state is FP32 scratch of
     * tokens x heads x (head_dim + 4) floats (tokens: q's rows the chunks cover, counted from row 0), 16-byte
     * aligned, that the call's two launches hand the rows' running states through. */
    const void* fresh_keys;
    const void* fresh_values;
    const int64_t* fresh_firsts;
    float* fresh_state;
    int64_t fresh_stride_k, fresh_stride_v;
    /* INT8 pages only (the reference's int8_qk, __init__.py:1245, _kernels.py:637-643, 668-671): each query row is
     * rounded to INT8 codes at its own scale (amax / 127, half away from zero) and the scores are exact integer
     * products of query and key codes times the two scales. Fresh rows, where given, are still read in q's type. */
    int32_t int8_qk;
} crit_pkv_prefill_params;

int crit_pkv_prefill(const crit_pkv_prefill_params* p, void* stream);

/* ---- pool bookkeeping on the device --------------------------------------------------------------------------------
 * What KVPool does with torch indexing for rounds that run without the host (inference/attention-state/code/
 * pages.py): the slots of positions through the bound page tables, the move of an accepted draft-tree path's rows,
 * and the copy of a shared page before it is written. One launch each, nothing read on the host, so a decode step's
 * slots -> append -> attention chain is captured as one HIP graph. */

/* A store of rows the pool holds per layer: a layer's rows start at base + layer * layer_stride (bytes); row `slot`
 * is row_bytes bytes at slot * row_bytes (keys: kv_heads * head_dim elements; row scales: kv_heads floats).
 * row_bytes and layer_stride are multiples of 4; stores whose base, stride and row_bytes are multiples of 16 move
 * 16 bytes a lane. */
typedef struct crit_pkv_store {
    void* base;
    int64_t layer_stride;
    int64_t row_bytes;
} crit_pkv_store;

#define CRIT_PKV_MAX_STORES 4       /* keys, values, key scales, value scales */
#define CRIT_PKV_MAX_PATH 256       /* columns of a tree path */

/* Replaces KVPool._slots_at and the index_select before it in _reserve_round (pages.py:646-660):
 *   s = rows ? slots[rows[i]] : slots[i];   p = positions[i]
 *   out[i] = 0 <= p < round_capacity[s] ? round_tables[s][min(p / page, table_pages - 1)] * page + p % page
 *                                       : dump * page
 * A round slot outside 0 .. round_slots - 1 (the reference's indexing would raise) reads as capacity 0. */
typedef struct crit_pkv_slots_params {
    const int32_t* round_tables;    /* [round_slots][table_stride >= table_pages] */
    const int64_t* round_capacity;  /* [round_slots] */
    const int64_t* slots;           /* the round slot of each token, or of each row with `rows` */
    const int64_t* rows;            /* optional [n]: the row of each token */
    const int64_t* positions;       /* [n] */
    int64_t* out;                   /* [n] */
    int64_t n, round_slots, table_stride, n_slots;   /* n_slots: entries of `slots` (bounds rows[i]) */
    int32_t table_pages, page, dump;
} crit_pkv_slots_params;

int crit_pkv_slots_at(const crit_pkv_slots_params* p, void* stream);

/* Replaces KVPool._compact (pages.py:662-684), called by commit_round for a draft tree: for round row r (round slot
 * r) and column 0 < j < min(width, emitted[r]) with path[r][j] >= 0, where moved[r] == 0, the row of every store and
 * layer at position start[r] + path[r][j] is copied to position start[r] + j (slots as crit_pkv_slots_at finds them:
 * a position outside the slot's capacity is the dump page's first slot). All of a row's sources are read before any
 * of its targets is written, as index_copy_(index_select()) does. A target outside the capacity (the dump page's
 * first slot) is not written: the reference leaves one of the rows sent there, which one is undefined, and a source
 * outside the capacity must read the dump page as it was before the move whichever row's workgroup runs first. Then
 * moved[r] = 1 for every r < rows (a second launch on the same stream). */
typedef struct crit_pkv_compact_params {
    const int32_t* round_tables;
    const int64_t* round_capacity;
    const int64_t* start;           /* [rows] */
    const int64_t* emitted;         /* [rows] */
    const void* path;               /* [rows][path_stride >= width], int64, or int32 with path_is_32 */
    int64_t* moved;                 /* [rows] */
    crit_pkv_store stores[CRIT_PKV_MAX_STORES];
    int64_t rows, round_slots, table_stride, path_stride;
    int32_t n_stores, layers, width, path_is_32, table_pages, page, dump;
} crit_pkv_compact_params;

int crit_pkv_compact(const crit_pkv_compact_params* p, void* stream);

/* Replaces the copies of KVPool._copy (pages.py:861-869: a page shared with a fork is copied before it is written),
 * for n pages at once: every store's rows source[i] * page .. + page - 1 of every layer are copied to the rows of
 * target[i]. A pair with a negative id (or one past pool_pages) is skipped. No target may be another pair's source or target. */
typedef struct crit_pkv_copy_pages_params {
    const int64_t* source;          /* [n] page ids */
    const int64_t* target;          /* [n] */
    crit_pkv_store stores[CRIT_PKV_MAX_STORES];
    int64_t n;
    int64_t pool_pages;             /* pages a layer holds: a pair with an id at or past it is skipped; 0: not checked */
    int32_t n_stores, layers, page;
} crit_pkv_copy_pages_params;

int crit_pkv_copy_pages(const crit_pkv_copy_pages_params* p, void* stream);

/* Replaces KVPool.start_round and the length update that ends KVPool.commit_round (pages.py:623-644), for round rows
 * 0 .. rows - 1 (round slot r is row r), one launch, nothing read on the host:
 *   commit == 0 (a round begins):  start[r] = round_lengths[r];  moved[r] = 0 (moved may be NULL)
 *   commit != 0 (after acceptance): round_lengths[r] = emitted[r] > 0 ? frontier[r] : start[r]
 * A held row (it emitted nothing) keeps the length the round found; a second commit from the same start (a truncation)
 * sets the lengths again from it. The tree path's move (crit_pkv_compact) comes before a commit, as in the reference. */
typedef struct crit_pkv_round_params {
    int64_t* round_lengths;         /* [>= rows] */
    int64_t* start;                 /* [>= rows] */
    int64_t* moved;                 /* [>= rows], commit == 0 only; optional */
    const int64_t* emitted;         /* [rows], commit != 0 */
    const int64_t* frontier;        /* [rows], commit != 0 */
    int64_t rows;
    int32_t commit;
} crit_pkv_round_params;

int crit_pkv_round(const crit_pkv_round_params* p, void* stream);

/* Replaces, for rows of sequences bound to round slots, what the host builds every step: StepBatch.build's starts,
 * positions and rows (core/python/crit_plugins/device.py:600-616), the slots reserve() finds (pages.py:337-349) and
 * KVPool._step_buffers' window rows (pages.py:359-397). Row r holds counts[r] tokens (count_each without counts; a
 * negative count reads as 0) of the sequence in round slot slot[r], the first at firsts[r] (without firsts: at
 * round_lengths[slot[r]], the sequence's first position without KV). With tokens_before(r) the tokens of the rows
 * before r, for each token j of row r, at i = tokens_before(r) + j:
 *   positions_t[i] = first + j;  rows_t[i] = r;  d_slots[i] = the slot of first + j as crit_pkv_slots_at finds it
 *   starts_t[r] = tokens_before(r);  starts_t[rows] = the tokens of all rows
 * and for the w-th row whose count is at most `window` (a window row, in row order):
 *   d_rows[w] = w; d_starts[w] = tokens_before(r); d_counts[w] = count; d_firsts[w] = first;
 *   d_offsets[w] = the tokens of the window rows before it; d_tables[w][:] = round_tables[slot[r]][:] (the dump page's
 *   id for a slot outside 0 .. round_slots - 1 and past table_pages)
 * Window entries from the number of window rows up to step_rows - 1 are set empty (count 0, table all dump page), so a
 * launch over all step_rows entries reads nothing for them. totals[0..3] = tokens, window rows, window tokens, and 1
 * if the tokens exceed step_tokens or the window rows step_rows (what exceeds is not written; the reference raises
 * ValueError on the host there, pages.py:365-368), else 0. One launch; capture-safe. rows <= 32768. */
typedef struct crit_pkv_step_params {
    const int32_t* round_tables;    /* [round_slots][table_stride >= table_pages] */
    const int64_t* round_capacity;  /* [round_slots] */
    const int64_t* round_lengths;   /* [round_slots]; may be NULL with firsts */
    const int64_t* slot;            /* [rows] */
    const int64_t* counts;          /* optional [rows] */
    const int64_t* firsts;          /* optional [rows] */
    int64_t* d_slots;               /* [step_tokens] */
    int64_t* positions_t;           /* optional [step_tokens] */
    int64_t* rows_t;                /* optional [step_tokens] */
    int32_t* starts_t;              /* optional [rows + 1] */
    int32_t* d_rows;                /* optional [step_rows] */
    int32_t* d_starts;              /* [step_rows] */
    int32_t* d_counts;              /* [step_rows] */
    int64_t* d_firsts;              /* [step_rows] */
    int32_t* d_offsets;             /* [step_rows] */
    int32_t* d_tables;              /* [step_rows][d_tables_stride >= table_pages] */
    int64_t* totals;                /* [4] */
    int64_t rows, round_slots, table_stride, d_tables_stride, step_tokens, step_rows, count_each, window;
    int32_t table_pages, page, dump;
} crit_pkv_step_params;

int crit_pkv_step_buffers(const crit_pkv_step_params* p, void* stream);

/* ---- latent attention ---------------------------------------------------------------------------------------------
 * Replaces attend() of crit's latent-attention kernels module (kernels/techniques/attention/latent-attention/torch-ext/
 * latent_attention/__init__.py:153-229 and its _window_kernel / _merge_kernel), which crit's attention plugin calls for
 * pools of keys only with one KV head (inference/attention-state/code/device_attention.py:444-519): multi-head latent
 * attention, absorbed. cache [pages][page][rank + rope]: a position's latent, then its rotary key; the latent is the
 * position's value too. q [tokens][heads][rank + rope]; out [tokens][heads][rank]. Batch rows, tables, rows, starts,
 * counts, firsts and columns as crit_pkv_attend_params; causal inside the window:
 *   s[n] = scale * (q_latent . latent[n] + q_rope . rope[n]);  out = sum_n softmax(s)[n] * latent[n]
 * 16-bit products on the matrix pipe with FP32 sums, the probabilities rounded to q's type for the value product, the
 * softmax in FP32. A row's positions are cut into pieces of `piece` positions (a multiple of 32), piece i to partition
 * i mod partitions; partials [n_rows * columns][heads][partitions] x (rank floats, a maximum, a sum) are merged in
 * partition order, the sink logit (sinks [heads], natural log, -inf: none) folded in last; lse [tokens][heads] the
 * natural log-sum-exp (the sink counted). cache_dtype: 0 BF16, 1 FP16 (q in the same type), 2 E4M3 with `scales`
 * [pages][page][scales_per_row] FP32 (2: the latent's and the rotary key's, 1: one for the row) and BF16 or FP16 q.
 * rank is a power of two from 16 to 1024 and rope one from 16 to 256, as the reference's module takes them (anything
 * else: CRIT_PKV_E_GEOMETRY); ranks from 64 with widths from 32 are read on the matrix pipe, the smaller ones by plain
 * vector arithmetic. phases:
 * 0 both launches, 1 the partitions only, 2 the merge only.
 * tile_rows: the query rows a workgroup holds, which decides the kernel and with it a token's bits. 16: tiles of 16 rows
 * (two a workgroup from 32 rows on), every geometry, the fastest for a few batch rows. 128: 128 rows a workgroup on
 * 32 x 32 matrix tiles, the cache rows by DMA into LDS, one workgroup a compute unit (caches of (512, 64) only, pages a
 * multiple of 16 positions; anything else: CRIT_PKV_E_GEOMETRY), about twice the throughput of the other from a few
 * dozen batch rows of 128 heads on and slower below ten; with fewer heads a tile takes 128 / heads columns of a window,
 * which is how prompt chunks fill it. 0: 128 where it is allowed and the heads are a multiple of 128, else 16. The
 * partials of the two are laid out differently: with 128 they take ceil(columns * heads / 128) * 128 rows a batch row
 * (partial_max and partial_sum as always), and phases 1 and 2 of one call take the same tile_rows. */
typedef struct crit_pkv_latent_params {
    const void* q;
    const void* cache;
    const float* scales;
    const int32_t* tables;
    const void* rows;               /* int32, or int64 with rows_are_64 */
    const int32_t* starts;
    const int32_t* counts;          /* optional */
    const int64_t* firsts;
    float* partial_out;
    float* partial_max;
    float* partial_sum;
    void* out;
    float* lse;                     /* optional */
    const float* sinks;             /* optional */
    int64_t q_stride_t, q_stride_h, out_stride_t, out_stride_h, table_stride;
    int32_t table_width, n_rows, columns, heads, rank, rope, page, cache_dtype, q_dtype, out_dtype, scales_per_row,
        partitions, piece, rows_are_64, phases, tile_rows;
    float scale;
} crit_pkv_latent_params;

int crit_pkv_latent_attend(const crit_pkv_latent_params* p, void* stream);

/* ---- append to a latent cache ----------------------------------------------------------------------------------------
 * Replaces write() of the latent-attention kernels module (latent_attention/__init__.py:74-97, torch indexing there):
 * token t's latent [rank] and rotary key [rope_width] (in_dtype: CRIT_PKV_F32, _BF16 or _F16; rows latent_stride and
 * rope_stride elements apart, each contiguous) go side by side into row slots[t] of cache [slots][rank + rope_width];
 * a slot below 0 is skipped. cache_dtype 0 BF16 / 1 FP16: values rounded to nearest even. cache_dtype 2 E4M3: each of
 * the two parts coded at its own scale, scale = max(max|x| / 448, 1e-30), code = e4m3(clamp(x / scale, -448, 448)) with
 * IEEE divisions, the scales stored at scales[slot][0] (latent) and [slot][1] (rotary key). One launch. */
typedef struct crit_pkv_latent_write_params {
    const void* latent;
    const void* rope;
    const int64_t* slots;           /* [tokens] */
    void* cache;
    float* scales;                  /* [slots][2] FP32, cache_dtype 2; else NULL */
    int64_t tokens, latent_stride, rope_stride;
    int32_t rank, rope_width, in_dtype, cache_dtype;
} crit_pkv_latent_write_params;

int crit_pkv_latent_write(const crit_pkv_latent_write_params* p, void* stream);

/* ---- sparse index selection ---------------------------------------------------------------------------------------
 * Replaces scores() and topk() of crit's sparse-indexer kernels module (kernels/techniques/attention/sparse-indexer/
 * torch-ext/sparse_indexer/__init__.py:83-139 and its score_kernel / topk_kernel / cuda_select.cu; the operation:
 * inference/attention-state/code/sparse_index.py): for each query token a score over every compressed key it may see,
 *   out[t][s] = sum_h weights[t][h] * scale * max(0, q[t][h] . keys[s])   for s < ends[t], -inf at or past it,
 * 16-bit products on the matrix pipe with FP32 sums, ReLU, the head's factor and the sum over the heads (a fixed tree)
 * in FP32. q [tokens][heads][dim] BF16 or FP16 (heads up to 128, dim 64, 128 or 256); keys [rows][dim] in q's type
 * (key_dtype 0 BF16, 1 FP16) or E4M3 codes (2) with key_scales FP32 [rows], a key's value its code times its scale;
 * key_stride in elements. slots (optional, int32 or int64 [groups][n], slots_stride apart): key j of token t is row
 * slots[t / group][j] of keys (keys read in place where a pool stores them; group = tokens a group); without slots key
 * j is row j. A token's bits are its own. */
typedef struct crit_pkv_index_scores_params {
    const void* q;
    const void* keys;
    const float* key_scales;        /* E4M3 keys */
    const float* weights;           /* [tokens][weights_stride >= heads] */
    const int32_t* ends;            /* [tokens] */
    const void* slots;              /* optional */
    float* out;                     /* [tokens][out_stride >= n] */
    int64_t q_stride_t, q_stride_h, key_stride, weights_stride, out_stride, slots_stride;
    int32_t tokens, n, group, heads, dim, key_dtype, q_dtype, slots_are_64;
    float scale;
} crit_pkv_index_scores_params;

int crit_pkv_index_scores(const crit_pkv_index_scores_params* p, void* stream);

/* out[t][0 .. k - 1] (int32) = the positions of token t's k largest scores below ends[t], ascending, then -1 (all of
 * them where ends[t] <= k): ties to the lower position, -0 = +0, a NaN below every number (sparse_index.py:24-40). One
 * workgroup a token: an 8-bit radix select for the k-th score, then the positions in order. */
typedef struct crit_pkv_index_topk_params {
    const float* scores;            /* [tokens][scores_stride >= n] */
    const int32_t* ends;
    int32_t* out;                   /* [tokens][out_stride >= k] */
    void* work;                     /* optional: crit_pkv_index_topk_work_bytes() bytes of device memory (16-aligned) */
    int64_t scores_stride, out_stride, work_bytes;
    int32_t tokens, n, k;
} crit_pkv_index_topk_params;

int crit_pkv_index_topk(const crit_pkv_index_topk_params* p, void* stream);

/* Rows past 32,768 positions select faster in slices (each slice's k best in parallel, then the k best of those: the
 * same picks, sparse_indexer/__init__.py:152-170): the bytes of `work` a call of this shape takes, 0 where one pass a
 * row is the way (rows a workgroup holds, or candidates past 512 MiB). Without `work` (or with less) the call selects
 * in one pass a row. */
int64_t crit_pkv_index_topk_work_bytes(int32_t tokens, int32_t n, int32_t k);

/* ---- rows read back ----------------------------------------------------------------------------------------------
 * Replaces the index_select, cast and multiply of KVPool.gather and KVPool.rows_at (pages.py:455-493): row i of the
 * output is the pool's row at slots[i], or, with a page table instead (exactly one of slots, table, table64), at
 * table[i / page] * page + i % page (a sequence's first n positions); value = float(stored) * scale in FP32 (the
 * layer's multiplier, or the row's scale), rounded once to out_dtype. A negative slot reads as zeros. out_keys
 * [n][kv_heads][head_dim], out_values [n][kv_heads][value_dim], contiguous; value_pages / out_values NULL: keys only.
 * Head widths are multiples of 8. */
typedef struct crit_pkv_read_params {
    const void* key_pages;
    const void* value_pages;
    const float* key_scales;        /* kinds FP8_ROW and INT8 */
    const float* value_scales;
    const float* head_multipliers;  /* optional [2][kv_heads], kind FP8 */
    const int64_t* slots;           /* [n] */
    const int32_t* table;           /* [ceil(n / page)] */
    const int64_t* table64;
    void* out_keys;
    void* out_values;
    int64_t n;
    int64_t pool_slots;             /* slots a layer holds: a slot at or past it reads as zeros, like a negative one
                                       (the reference's index_select would raise); 0: not checked */
    int32_t kv_heads, head_dim, value_dim, page, kind, page_dtype, out_dtype;
    float key_multiplier, value_multiplier;
} crit_pkv_read_params;

int crit_pkv_read_rows(const crit_pkv_read_params* p, void* stream);

/* ---- housekeeping ------------------------------------------------------------------------------------------------- */
int crit_pkv_abi_version(void);
/* sizeof() of the parameter structs as the library was compiled, for the host's mirror to cross-check
 * (which: 0 write, 1 attend, 2 merge, 3 prefill, 4 slots_at, 5 compact, 6 copy_pages, 7 read_rows, 8 round, 9 step_buffers, 10 latent_attend, 11 index_scores, 12 index_topk, 13 latent_write), as crit_cw_params_size() does (cuda_window.cu:1502). */
int crit_pkv_params_size(int which);
const char* crit_pkv_error(int code);
/* *id = the id of the capture `stream` is recording into (never 0), or 0 when it is not capturing; returns 0 or a HIP
 * error code. For hosts that key a launch's counters (crit_pkv_attend_params.launch_state) by capture, so that a
 * replaying graph never shares them with an eager launch. No counterpart in the reference. */
int crit_pkv_stream_capture(void* stream, unsigned long long* id);
/* A streaming-read probe: sums `bytes` (a multiple of 16) of device memory into sink[0..63]; the achievable-HBM-read
 * yardstick the benchmark prints beside the nominal peak. No counterpart in the reference. */
int crit_pkv_stream_read(const void* data, int64_t bytes, float* sink, void* stream);

#ifdef __cplusplus
}
#endif
#endif
