"""crit_amd.sparse_indexer against the float64 oracle, the cases of the reference's own tests (kernels/techniques/
attention/sparse-indexer/tests/test_sparse_indexer.py): scores over 16-bit and E4M3 keys at the head counts and widths
it takes, causal ends; picks with ties, fewer valid keys than k, empty rows, NaN and -inf; a token's bits the same alone
and beside other tokens; select in groups the same as one call; keys read in place; a captured call; what it refuses."""
import numpy as np
import pytest
import torch

from crit_amd import sparse_indexer as si
from oracle import indexer as ref

pytestmark = pytest.mark.gpu
dev = torch.device("cuda")


def problem(t, h, d, n, seed=0, fp8=False, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(t, h, d, generator=g) * 0.5).to(dev).to(dtype)
    keys = (torch.randn(n, d, generator=g) * 0.5).to(dev).to(dtype)
    w = (torch.randn(t, h, generator=g) * h ** -0.5).to(dev)
    ends = torch.randint(0, n + 1, (t,), generator=g).to(torch.int32).to(dev)
    ends[0] = n
    scales, values = None, keys.float()
    if fp8:
        scales = (keys.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        keys = (keys.float() / scales[:, None]).to(torch.float8_e4m3fn)
        values = keys.float() * scales[:, None]
    return q, keys, scales, values, w, ends


def oracle_scores(q, values, w, ends, scale):
    return ref.sparse_scores(q.double().cpu().numpy(), values.double().cpu().numpy(), w.double().cpu().numpy(),
                             ends.cpu().numpy(), scale)


def oracle_index(s, ends, k):
    return torch.from_numpy(ref.sparse_index(s.double().cpu().numpy(), ends.cpu().numpy(), k))


@pytest.mark.parametrize("h,d", [(64, 128), (32, 64), (16, 256), (8, 128), (128, 256), (1, 64)])
@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_scores_match_the_oracle(h, d, fp8, dtype):
    q, keys, scales, values, w, ends = problem(37, h, d, 1000, seed=h + d, fp8=fp8, dtype=dtype)
    got = si.scores(q, keys, w, ends, key_scales=scales).cpu().numpy()
    want = oracle_scores(q, values, w, ends, d ** -0.5)
    # FP32 sums of exact 16-bit products: 1e-4 of the sum of magnitudes (the reference's own bound)
    bound = oracle_scores(q.abs(), values.abs(), w.abs(), ends, d ** -0.5) * 1e-4 + 1e-6
    finite = np.isfinite(want)
    assert np.array_equal(finite, np.isfinite(got))
    assert (got[~finite] == -np.inf).all()
    assert (np.abs(got.astype(np.float64)[finite] - want[finite]) <= bound[finite]).all()


def test_a_tokens_scores_are_its_own():
    for h, d, fp8, n in ((64, 128, False, 700), (8, 64, True, 900), (128, 256, False, 900), (1, 64, False, 333)):
        q, keys, scales, _, w, ends = problem(33, h, d, n, seed=3 + h, fp8=fp8)
        all_rows = si.scores(q, keys, w, ends, key_scales=scales)
        for t in (0, 1, 16, 32):
            alone = si.scores(q[t:t + 1], keys, w[t:t + 1], ends[t:t + 1], key_scales=scales)
            assert torch.equal(alone[0].view(torch.int32), all_rows[t].view(torch.int32)), (h, t)
        again = si.scores(q, keys, w, ends, key_scales=scales)
        assert torch.equal(again.view(torch.int32), all_rows.view(torch.int32))
        # the block of keys a workgroup takes follows the launch's size: many tokens, the same bits
        many = si.scores(q.repeat(40, 1, 1), keys, w.repeat(40, 1), ends.repeat(40), key_scales=scales)
        assert torch.equal(many[33 * 7:33 * 8].view(torch.int32), all_rows.view(torch.int32))


def test_scores_into_a_wider_out_and_strided_queries():
    q, keys, _, values, w, ends = problem(6, 16, 128, 250, seed=21)
    wide = torch.full((8, 300), 7.0, device=dev)
    si.scores(q, keys, w, ends, out=wide)
    want = si.scores(q, keys, w, ends)
    assert torch.equal(wide[:6, :250], want) and bool((wide[:, 250:] == 7.0).all()) and bool((wide[6:] == 7.0).all())
    big = torch.zeros(6, 16, 256, dtype=q.dtype, device=dev)
    big[:, :, :128] = q
    assert torch.equal(si.scores(big[:, :, :128], keys, w, ends), want)


@pytest.mark.parametrize("n,k", [(5000, 512), (700, 64), (300, 512), (1, 1), (4097, 2048)])
def test_topk_picks_the_oracles_positions(n, k):
    g = torch.Generator().manual_seed(n + k)
    t = 9
    s = torch.randn(t, n, generator=g)
    s[:, torch.randint(0, n, (n // 3,), generator=g)] = 0.0          # many ties
    s[2] = 1.0                                                        # one row all ties
    s = s.to(dev)
    ends = torch.tensor([n, n - 1, n, k // 2, 0, max(1, n - 300), k, n, 1], dtype=torch.int32, device=dev).clamp(0, n)
    got = si.topk(s, ends, k)
    assert torch.equal(got.long().cpu(), oracle_index(s, ends, k))


def test_a_nan_ranks_below_every_number():
    s = torch.tensor([[1.0, float("nan"), float("-inf"), 2.0, float("nan")]], device=dev)
    end = torch.tensor([5], dtype=torch.int32, device=dev)
    assert si.topk(s, end, 4).tolist() == [[0, 1, 2, 3]]   # 2, 1, -inf, then the first NaN
    assert si.topk(s, end, 3).tolist() == [[0, 2, 3]]
    z = torch.tensor([[0.0, -0.0, 0.0, -0.0, -1.0]], device=dev)
    assert si.topk(z, end, 2).tolist() == [[0, 1]]          # the zeros tie


# (rows of 9,000, 13,000, 20,000 and 30,000: each of the element counts a thread of the kernel that holds a row is built
# for; 128 rows or more of up to 64,512: a workgroup holds such a row whole)
@pytest.mark.parametrize("n,k,t", [(200000, 512, 1), (60000, 4096, 2), (8192, 512, 3), (5, 512, 1), (33000, 16, 4),
                                   (4096, 1, 2), (9000, 2048, 2), (13000, 64, 2), (20000, 2048, 2), (30000, 300, 2),
                                   (50000, 2048, 2), (36000, 2048, 130), (50000, 2048, 130), (57000, 100, 128),
                                   (64512, 2048, 129), (64513, 700, 128)])
def test_long_rows_with_ties_nans_and_rows_cut_short(n, k, t):
    g = torch.Generator().manual_seed(n * 7 + k)
    s = torch.randn(t, n, generator=g)
    s[:, torch.randint(0, n, (n // 3,), generator=g)] = 0.0
    s[:, torch.randint(0, n, (max(1, n // 50),), generator=g)] = float("nan")
    s[:, torch.randint(0, n, (max(1, n // 40),), generator=g)] = float("-inf")
    s[-1, : n // 2] = 2.5   # more ties at the threshold than k
    s = s.to(dev)
    for cut in (0, 1, 3, n // 2, n):
        ends = torch.full((t,), n, dtype=torch.int32, device=dev)
        ends[0] = max(0, n - cut)
        got = si.topk(s, ends, k)
        assert torch.equal(got.long().cpu(), oracle_index(s, ends, k)), (n, k, t, cut)


def test_rows_of_a_batch_pick_what_they_pick_alone():
    n, k = 20000, 2048
    g = torch.Generator().manual_seed(n)
    s = torch.randn(200, n, generator=g)
    s[:, torch.randint(0, n, (n // 4,), generator=g)] = 0.0
    s[1, 100:] = 0.5
    s = s.to(dev)
    ends = torch.full((200,), n, dtype=torch.int32, device=dev)
    ends[2], ends[3] = n - 777, k + 5
    batch = si.topk(s, ends, k)
    for t in range(4):
        alone = si.topk(s[t:t + 1].contiguous(), ends[t:t + 1], k)
        assert torch.equal(alone[0], batch[t]), t
    assert torch.equal(batch[:4].long().cpu(), oracle_index(s[:4], ends[:4], k))


def test_select_in_groups_is_one_call_and_matches_the_oracle():
    q, keys, scales, values, w, ends = problem(50, 64, 128, 3000, seed=9, fp8=True)
    whole = si.select(q, keys, w, ends, 256, key_scales=scales, workspace_bytes=1 << 30)
    grouped = si.select(q, keys, w, ends, 256, key_scales=scales, workspace=torch.empty(7 * 3000, device=dev))
    assert torch.equal(whole, grouped)
    want = oracle_scores(q, values, w, ends, 128 ** -0.5)
    picked = ref.sparse_index(want, ends.cpu().numpy(), 256)
    got_scores = si.scores(q, keys, w, ends, key_scales=scales)
    assert torch.equal(si.topk(got_scores, ends, 256), whole)
    # where the exact and the kernel's picks differ, the kernel's picks score within the products' error of the k-th
    for t in range(q.shape[0]):
        a, b = set(whole[t].tolist()) - {-1}, set(picked[t].tolist()) - {-1}
        if a != b:
            kth = want[t][list(b)].min()
            assert float(want[t][list(a - b)].min()) >= float(kth) - 1e-3, t


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("kind", [torch.int32, torch.int64])
def test_keys_read_in_place_score_as_their_gathered_copy(fp8, kind):
    rows, each, n = 3, 4, 700
    q, _, _, _, w, ends = problem(rows * each, 64, 128, n, seed=11)
    g = torch.Generator().manual_seed(5)
    store = (torch.randn(5000, 128, generator=g) * 0.5).to(dev).to(torch.bfloat16)
    scales = None
    if fp8:
        scales = (store.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        store = (store.float() / scales[:, None]).to(torch.float8_e4m3fn)
    slots = torch.stack([torch.randperm(5000, generator=g)[:n] for _ in range(rows)]).to(dev).to(kind)
    got = si.scores(q, store, w, ends, key_scales=scales, slots=slots)
    for r in range(rows):
        span = slice(r * each, (r + 1) * each)
        keys = store[slots[r].long()]
        want = si.scores(q[span], keys, w[span], ends[span], key_scales=None if scales is None else scales[slots[r].long()])
        assert torch.equal(got[span], want), r
    one = si.scores(q[:each], store, w[:each], ends[:each], key_scales=scales, slots=slots[0])
    assert torch.equal(one, got[:each])                                   # [n]: one sequence
    picked = si.select(q[:each], store, w[:each], ends[:each], 16, key_scales=scales, slots=slots[0])
    assert torch.equal(picked, si.topk(got[:each], ends[:each], 16))
    with pytest.raises(ValueError):
        si.scores(q[:5], store, w[:5], ends[:5], key_scales=scales, slots=slots)   # 5 tokens are not 3 groups
    with pytest.raises(ValueError):
        si.scores(q, store, w, ends, key_scales=scales, slots=slots.float())


def test_one_list_for_many_tokens_takes_the_shared_kernel_whatever_their_count():
    # One slot list [n] for every token (a prompt chunk of one sequence): 19 or 21 tokens fill no whole workgroups of 4
    # or 8, and share their keys through LDS all the same; every token scores as it does alone.
    n = 900
    g = torch.Generator().manual_seed(15)
    store = (torch.randn(4000, 128, generator=g) * 0.5).to(dev).to(torch.bfloat16)
    slots = torch.randperm(4000, generator=g)[:n].to(dev)
    for tokens in (19, 21):
        q, _, _, _, w, ends = problem(tokens, 64, 128, n, seed=16 + tokens)
        got = si.scores(q, store, w, ends, slots=slots)
        assert torch.equal(got, si.scores(q, store[slots], w, ends))
        for t in (0, 7, tokens - 1):
            assert torch.equal(got[t], si.scores(q[t:t + 1], store, w[t:t + 1], ends[t:t + 1], slots=slots)[0]), t


@pytest.mark.parametrize("fp8", [False, True])
@pytest.mark.parametrize("each", [16, 12])
def test_a_rounds_rows_share_their_keys_in_place(fp8, each):
    # Many tokens in groups (a round's rows, each a sequence with its own slots): groups of 16 fill the workgroups that
    # share keys through LDS, groups of 12 do not and go a token a workgroup; either way the gathered keys' bits.
    rows, n = 4, 900
    q, _, _, _, w, ends = problem(rows * each, 64, 128, n, seed=13)
    g = torch.Generator().manual_seed(6)
    store = (torch.randn(4000, 128, generator=g) * 0.5).to(dev).to(torch.bfloat16)
    scales = None
    if fp8:
        scales = (store.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        store = (store.float() / scales[:, None]).to(torch.float8_e4m3fn)
    slots = torch.stack([torch.randperm(4000, generator=g)[:n] for _ in range(rows)]).to(dev)
    got = si.scores(q, store, w, ends, key_scales=scales, slots=slots)
    for r in range(rows):
        span = slice(r * each, (r + 1) * each)
        want = si.scores(q[span], store[slots[r]], w[span], ends[span], key_scales=None if scales is None else scales[slots[r]])
        assert torch.equal(got[span].view(torch.int32), want.view(torch.int32)), r
        alone = si.scores(q[span][:1], store, w[span][:1], ends[span][:1], key_scales=scales, slots=slots[r].to(torch.int32))
        assert torch.equal(alone[0].view(torch.int32), got[span][0].view(torch.int32)), r


def test_calls_past_a_launchs_tokens_go_in_runs(monkeypatch):
    monkeypatch.setattr(si, "_LAUNCH_TOKENS", 40)
    q, keys, _, _, w, ends = problem(100, 8, 64, 300, seed=17)
    runs = si.scores(q, keys, w, ends)
    g = torch.Generator().manual_seed(7)
    slots = torch.stack([torch.randperm(300, generator=g)[:200] for _ in range(5)]).to(dev)      # 5 groups of 20
    ends2 = ends.clamp(max=200)
    grouped = si.scores(q, keys, w, ends2, slots=slots)
    wide = si.scores(q, keys, w, ends2, slots=slots[:2].repeat_interleave(1, 0)[:2])            # 2 groups of 50: past 40 each
    monkeypatch.setattr(si, "_LAUNCH_TOKENS", 65535)
    assert torch.equal(runs, si.scores(q, keys, w, ends))
    assert torch.equal(grouped, si.scores(q, keys, w, ends2, slots=slots))
    assert torch.equal(wide, si.scores(q, keys, w, ends2, slots=slots[:2]))


def test_graphs_capture_a_select():
    q, keys, scales, _, w, ends = problem(4, 64, 128, 2048, seed=4)
    out = torch.empty(4, 512, dtype=torch.int32, device=dev)
    space = torch.empty(4 * 2048, device=dev)
    si.select(q, keys, w, ends, 512, out=out, workspace=space)
    want = out.clone()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        si.select(q, keys, w, ends, 512, out=out, workspace=space)
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_it_refuses_what_it_does_not_take():
    q, keys, scales, _, w, ends = problem(2, 64, 128, 10)
    with pytest.raises(ValueError):
        si.scores(q.float(), keys, w, ends)
    with pytest.raises(ValueError):
        si.scores(q, keys.half(), w, ends)
    with pytest.raises(ValueError):
        si.scores(q, keys.to(torch.float8_e4m3fn), w, ends)              # E4M3 keys without scales
    with pytest.raises(ValueError):
        si.scores(q, keys, w, ends.long())
    with pytest.raises(ValueError):
        si.scores(q[:, :48], keys, w[:, :48], ends)                      # heads not a power of two
    with pytest.raises(ValueError):
        si.topk(torch.zeros(2, 10, device=dev), ends, 0)
    with pytest.raises(ValueError):
        si.scores(q.cpu(), keys.cpu(), w.cpu(), ends.cpu())              # there is no CPU path


@pytest.mark.parametrize("kind,fp8_keys", [("bf16", False), ("fp8", True)])
def test_a_sparse_decode_step_reads_the_blocks_the_index_selects(kind, fp8_keys):
    # What the reference's sparse reader does with the two modules (inference/attention-state/code/sparse_index.py, then
    # paged_kv_attention.attend(blocks=)): four decode tokens of one sequence of 4,000 positions, one index key per
    # block of 64 positions; each token scores the blocks it may see, its 8 best become its block list, and the
    # attention reads those blocks only. The picks against the oracle's, the attention against float64 attention over
    # the listed blocks.
    from tests.support import Cache, rand_q
    block, n_pos, k = 64, 4000, 8
    n_blocks = -(-n_pos // block)
    cache = Cache(kind, 2, 128, 128, 16, [n_pos])
    q, keys, scales, values, w, _ = problem(4, 16, 64, n_blocks, seed=21, fp8=fp8_keys)
    firsts = n_pos - 4
    ends = torch.tensor([(firsts + t) // block + 1 for t in range(4)], dtype=torch.int32, device=dev)   # the blocks a token may see
    picked = si.select(q, keys, w, ends, k, key_scales=scales)
    assert picked.dtype == torch.int32 and picked.shape == (4, k)
    want_scores = oracle_scores(q, values, w, ends, 64 ** -0.5)
    exact = ref.sparse_index(want_scores, ends.cpu().numpy(), k)
    for t in range(4):
        a, b = set(picked[t].tolist()), set(exact[t].tolist())
        if a != b:      # a pick that differs scores within the products' error of the k-th
            assert float(want_scores[t][list(a - b)].min()) >= float(want_scores[t][list(b)].min()) - 1e-3, t
    qa = rand_q(4, 8, 128, 5)
    lse = torch.empty(4, 8, device=dev)
    zero = torch.zeros(1, dtype=torch.int32, device=dev)
    at = torch.tensor([firsts], dtype=torch.int64, device=dev)
    out = cache.attend(qa, zero, zero, at, 4, blocks=picked, block_size=block, lse=lse, partitions=4)
    want, want_lse = cache.want(qa.to(torch.bfloat16), 0, firsts, 4, blocks=picked.cpu(), block_size=block)
    torch.testing.assert_close(out.double().cpu(), want, atol=8e-3, rtol=2e-2)
    torch.testing.assert_close(lse.double().cpu(), want_lse, atol=1e-3, rtol=1e-4)
    # the same step as one captured graph: no host work between the index and the attention
    graph = torch.cuda.CUDAGraph()
    again, picked_again = torch.empty_like(out), torch.empty_like(picked)
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        si.select(q, keys, w, ends, k, key_scales=scales, out=picked_again)
        cache.attend(qa, zero, zero, at, 4, blocks=picked_again, block_size=block, partitions=4, out=again)
        torch.cuda.synchronize()
        picked_again.fill_(-1), again.zero_()
        with torch.cuda.graph(graph, stream=stream):
            si.select(q, keys, w, ends, k, key_scales=scales, out=picked_again)
            cache.attend(qa, zero, zero, at, 4, blocks=picked_again, block_size=block, partitions=4, out=again)
    for _ in range(2):
        picked_again.fill_(-1), again.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(picked_again, picked) and torch.equal(again, out)


@pytest.mark.parametrize("fp8", [False, True])
def test_a_decode_steps_sequences_score_their_own_keys_in_place(fp8):
    # 64 sequences of one token, each over its own 50,000 keys where a store holds them (pages of 64 rows at random
    # places): blocks of thousands of keys a workgroup, the launch whose wavefronts keep three tiles of key rows in
    # flight. A sequence's scores are bit for bit those of the sequence alone over a gathered copy of its keys.
    groups, n, page = 64, 50000, 64
    q, _, _, _, w, _ = problem(groups, 64, 128, 8, seed=31)
    g = torch.Generator(device=dev).manual_seed(6)
    rows = groups * (n // page + 1) * page
    store = (torch.randn(rows, 128, device=dev, generator=g) * 0.5).to(torch.bfloat16)
    scales = None
    if fp8:
        scales = (store.float().abs().amax(1) / 448.0).clamp_min(1e-30)
        store = (store.float() / scales[:, None]).to(torch.float8_e4m3fn)
    pages = torch.randperm(rows // page, device=dev, generator=g).view(groups, -1)
    slots = (pages[:, :, None] * page + torch.arange(page, device=dev)[None, None, :]).reshape(groups, -1)[:, :n]
    slots = slots.to(torch.int32).contiguous()
    ends = torch.randint(n - 5000, n + 1, (groups,), generator=torch.Generator().manual_seed(2)).to(torch.int32).to(dev)
    ends[0], ends[1], ends[2], ends[3] = n, 0, 17, 4160
    got = si.scores(q, store, w, ends, key_scales=scales, slots=slots)
    assert bool((got[1] == float("-inf")).all())
    for s in (0, 2, 3, 4, 33, 63):
        keys = store[slots[s].long()]
        alone = si.scores(q[s:s + 1], keys, w[s:s + 1], ends[s:s + 1], key_scales=None if scales is None else scales[slots[s].long()])
        assert torch.equal(got[s], alone[0]), s
        seen = int(ends[s])
        assert bool(torch.isfinite(got[s, :seen]).all()) and bool((got[s, seen:] == float("-inf")).all())
    picked = si.topk(got, ends, 64)
    assert torch.equal(picked[0], oracle_index(got[:1], ends[:1], 64)[0].to(dev))
