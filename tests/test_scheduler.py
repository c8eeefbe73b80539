"""Invariants of the tile scheduler, checked on the host mirror (distca_ca_schedule_host runs
the same cost functions and the same bin sort as the device builder).

The reference has no GPU-side scheduler to compare with; what is fixed is the mathematics:
the items must tile every task exactly once, each item's extent must cover exactly the keys
(or query blocks) the causal mask with KV-prefix offset lk - lq makes visible, and the order
must be longest first."""
import heapq

import numpy as np
import pytest

from distca_amd import scheduler, workloads
from oracle.attention import causal_pairs

HQ, HKV = 32, 8
G = HQ // HKV


def _cu(lens):
    return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)


CASES = [
    ([1], [1]),
    ([5, 0, 300], [5, 7, 300]),
    ([128, 64, 33], [128 + 512, 64, 33 + 1000]),          # KV prefixes (context-parallel shards)
    ([31, 32, 33, 1000], [31, 32, 33, 1000]),
    ([17, 600], [10, 600]),                               # lk < lq: the first tokens see nothing
]


# Batches of short tasks (fewer than 2048 query tokens per task on average) have the forward and dQ lists made of
# merged items: item i of a task is its blocks i m .. (i + 1) m - 1, with m = 128 // (KV tiles of the task's last block),
# between 1 and 8, so that a work item has about 128 tiles to stream whatever the task's length.
MERGE_MEAN_TOKENS, MERGE_TILES, MAX_MERGE = 2048, 128, 8


@pytest.mark.parametrize("lq,lk", CASES + [([4096, 2100], [4096, 5000]), ([1024] * 6, [1024] * 6), ([700, 2500, 90], [900, 2500, 4000])])
@pytest.mark.parametrize("causal", [True, False])
def test_forward_items_tile_each_task_once_and_cover_visible_keys(lq, lk, causal):
    rows, kv = scheduler.tile_shape(scheduler.FWD, HQ, HKV)
    items = scheduler.build_schedule(scheduler.FWD, _cu(lq), _cu(lk), HQ, HKV, causal=causal)
    seen = {}
    for t, b, c, w in items.tolist():
        assert (t, b) not in seen and w == 1 << 16          # forward items are never cut
        seen[(t, b)] = c
    merged = sum(lq) < MERGE_MEAN_TOKENS * len(lq)
    some_merged = False
    for t, (a, k) in enumerate(zip(lq, lk)):
        nblk = -(-a * G // rows)
        costs = []
        for b in range(nblk):
            last_tok = min(a, -(-(b + 1) * rows // G)) - 1           # last token with a row in the block
            vis = min(k, max(0, last_tok + 1 + (k - a))) if causal else k
            costs.append(-(-vis // kv))                                # KV tiles the block streams
        m = min(MAX_MERGE, max(1, MERGE_TILES // max(1, costs[-1]))) if merged and nblk > 1 else 1
        some_merged |= m > 1
        nitems = -(-nblk // m)
        assert sorted(b for (tt, b) in seen if tt == t) == list(range(nitems))
        for i in range(nitems):
            assert seen[(t, i)] == sum(costs[i * m:(i + 1) * m])
    if not merged:
        assert not some_merged
    costs = items[:, 2]
    assert (np.diff(costs) <= 0).all()


@pytest.mark.parametrize("lq,lk", CASES)
@pytest.mark.parametrize("causal", [True, False])
def test_backward_items_cover_every_query_block_that_sees_the_key_block(lq, lk, causal):
    rows, kv = scheduler.tile_shape(scheduler.BWD, HQ, HKV)
    items = scheduler.build_schedule(scheduler.BWD, _cu(lq), _cu(lk), HQ, HKV, causal=causal)
    whole = scheduler.whole_items(items)
    seen = {(t, b): c for t, b, c in whole.tolist()}
    assert len(seen) == len(whole)
    # these batches are small, so expensive key blocks come in pieces: piece j of k, each once, of
    # consecutive query blocks counted from the last block down (cost n: blocks [n j / k, n (j+1) / k))
    pieces = {}
    for t, b, c, w in items.tolist():
        pieces.setdefault((t, b), []).append((scheduler.item_piece(w), scheduler.item_pieces(w), c))
    for (t, b), ps in pieces.items():
        k = ps[0][1]
        assert sorted(j for j, _, _ in ps) == list(range(k)) and all(kk == k for _, kk, _ in ps)
        n = seen[(t, b)]
        assert all(c == n * (j + 1) // k - n * j // k for j, _, c in ps)
    det = scheduler.build_schedule(scheduler.BWD, _cu(lq), _cu(lk), HQ, HKV, causal=causal, deterministic=True)
    assert ((det[:, 3] & ~np.int32(scheduler.WALK_UP)) == 1 << 16).all() and sorted(map(tuple, det[:, :3].tolist())) == sorted(map(tuple, whole.tolist()))
    for t, (a, k) in enumerate(zip(lq, lk)):
        nkb = -(-k // kv) if a > 0 else 0
        assert sorted(b for (tt, b) in seen if tt == t) == list(range(nkb))
        nmb = -(-a * G // rows)
        for n in range(nkb):
            # brute force: query blocks holding a token that sees a key of block n
            keys = np.arange(n * kv, min(k, (n + 1) * kv))
            toks = np.arange(a)
            vis_tok = toks[(toks + (k - a) >= keys.min())] if causal else toks
            first = (int(vis_tok.min()) * G) // rows if len(vis_tok) else nmb
            # the kernel walks m-blocks [nmb - cost, nmb): it must include `first`; it may start
            # at most one block early (first-token rounding), never late
            start = nmb - seen[(t, n)]
            assert start <= first
            assert first - start <= 1
    assert (np.diff(items[:, 2]) <= 0).all()


def test_forward_cost_totals_match_the_causal_pair_count():
    """Sum of item costs x tile area bounds the exact pair count from above by at most the
    diagonal tiles' slack (one KV tile and one row block per item)."""
    b = workloads.config2_llama8b_128k()
    rows, kv = scheduler.tile_shape(scheduler.FWD, HQ, HKV)
    items = scheduler.build_schedule(scheduler.FWD, b.cu_seqlens_q, b.cu_seqlens_k, HQ, HKV)
    lq, lk = np.diff(b.cu_seqlens_q), np.diff(b.cu_seqlens_k)
    pairs = sum(causal_pairs(int(a), int(k)) for a, k in zip(lq, lk)) * G   # (row, key) pairs per kv head
    covered = int(items[:, 2].astype(np.int64).sum()) * rows * kv
    assert pairs <= covered <= pairs + len(items) * rows * kv + int(lq.sum()) * G * kv


@pytest.mark.parametrize("kind", [scheduler.FWD, scheduler.BWD])
def test_sorted_dispatch_balances_a_skewed_batch(kind):
    """In-order dispatch of the sorted list onto free slots (what the hardware does with
    workgroup ids) ends within a few percent of the mean load; unsorted order does not."""
    b = workloads.config2_llama8b_128k()
    items = scheduler.build_schedule(kind, b.cu_seqlens_q, b.cu_seqlens_k, HQ, HKV)
    slots = 256 * 2 // HKV            # workgroup slots of the chip per kv head

    def makespan(costs):
        heap = [0] * slots
        for c in costs:
            heapq.heappush(heap, heapq.heappop(heap) + int(c) + 1)
        return max(heap)

    costs = items[:, 2]
    ideal = (costs.sum() + len(costs)) / slots
    assert makespan(costs) <= 1.05 * ideal + costs.max()
    rng = np.random.default_rng(0)
    assert makespan(costs) <= makespan(rng.permutation(costs))


def test_empty_batch_and_empty_tasks():
    assert scheduler.build_schedule(scheduler.FWD, [0], [0], HQ, HKV).shape == (0, 4)
    items = scheduler.build_schedule(scheduler.FWD, _cu([0, 0, 4]), _cu([9, 0, 4]), HQ, HKV)
    assert set(items[:, 0].tolist()) == {2}
    items = scheduler.build_schedule(scheduler.BWD, _cu([0, 4]), _cu([700, 4]), HQ, HKV)
    assert set(items[:, 0].tolist()) == {1}       # keys nobody queries receive no work item (their grads are the zero fill)


def test_group_sizes():
    for hq, hkv in [(8, 8), (16, 8), (64, 8), (28, 4)]:
        rows, kv = scheduler.tile_shape(scheduler.FWD, hq, hkv)
        # (tasks long enough that their blocks are not merged into larger work items: one item per block)
        items = scheduler.build_schedule(scheduler.FWD, _cu([4100, 2037]), _cu([4100, 2037]), hq, hkv)
        g = hq // hkv
        assert len(items) == -(-4100 * g // rows) + -(-2037 * g // rows)


def _check_capacity_and_tiling(lq, lk, hq, hkv, total_k=None):
    cu_q, cu_k = _cu(lq), _cu(lk)
    items = scheduler.build_schedule(scheduler.BWD, cu_q, cu_k, hq, hkv, total_k=total_k)
    cap = scheduler.schedule_capacity(scheduler.BWD, cu_q, cu_k, hq, hkv, total_k=total_k)
    assert len(items) <= cap, f"lq={lq} lk={lk} heads {hq}/{hkv}: {len(items)} items for a list of {cap}"
    return items


@pytest.mark.parametrize("hq,hkv", [(8, 8), (32, 8), (64, 8), (128, 8), (4, 1), (8, 2), (16, 4)])
def test_backward_list_always_has_room_for_the_pieces(hq, hkv):
    """The list is sized on the host as (bound on key blocks) + (pieces aimed for); the builder drops what does
    not fit, so the piece size must be such that the count never exceeds it.  (With the piece size rounded down,
    one document of 989 tokens at 128/8 heads, or of 1345 at 64/8, made one piece more than the list holds.)
    Every document length up to the point where cutting stops, then a coarser sweep beyond."""
    rows, kv = scheduler.tile_shape(scheduler.BWD, hq, hkv)
    g = hq // hkv
    lengths = list(range(1, 3000)) + list(range(3000, 16001, 37))
    for n in lengths:
        items = _check_capacity_and_tiling([n], [n], hq, hkv)
        if n in (989, 1345, 1364, 2999) or n % 500 == 0:
            # the pieces of every key block tile the query blocks that see it: [first block, nmb)
            nmb = -(-n * g // rows)
            got = {}
            for t, b, c, w in items.tolist():
                got.setdefault(b, []).append((scheduler.item_piece(w), scheduler.item_pieces(w), c))
            assert sorted(got) == list(range(-(-n // kv)))
            for b, ps in got.items():
                k = ps[0][1]
                assert sorted(j for j, _, _ in ps) == list(range(k))
                first = ((b * kv) * g) // rows
                assert sum(c for _, _, c in ps) == nmb - first


def test_backward_list_has_room_for_batches_and_shared_prefixes():
    rng = np.random.default_rng(7)
    for trial in range(300):
        hq, hkv = [(32, 8), (64, 8), (8, 8), (4, 1), (128, 8)][trial % 5]
        n = int(rng.integers(1, 9))
        lq = rng.integers(0, 700, size=n)
        extra = rng.integers(0, 900, size=n) * (rng.random(n) < 0.5)
        lk = lq + extra
        _check_capacity_and_tiling(lq.tolist(), lk.tolist(), hq, hkv)
        # the same tasks over stored prefixes: fewer K/V rows than the lengths add up to
        _check_capacity_and_tiling(lq.tolist(), lk.tolist(), hq, hkv, total_k=int(lk.max()))


@pytest.mark.parametrize("hq,hkv", [(32, 8), (16, 16), (4, 1)])
def test_walk_flags_alternate_by_rounds_of_the_list(hq, hkv):
    """Bit 31 of a backward item's fourth word: set for the items whose rank in the list lies in an odd round of
    (compute units / kv heads) items; forward lists carry none.  Without a device the mirror assumes 256 units."""
    rng = np.random.default_rng(3)
    lq = rng.integers(1, 9000, size=9)
    lk = lq + rng.integers(0, 3000, size=9) * (rng.random(9) < 0.5)
    items = scheduler.build_schedule(scheduler.BWD, _cu(lq), _cu(lk), hq, hkv, deterministic=True)
    n = len(items)
    up = items[:, 3] < 0
    rounds = sorted({r for r in (256 // hkv,) if np.array_equal(up, ((np.arange(n) // r) & 1).astype(bool))} |
                    {r for r in range(1, 1025) if np.array_equal(up, ((np.arange(n) // r) & 1).astype(bool))})
    assert rounds, "flags do not alternate by rounds of any size"
    assert (scheduler.item_pieces(items[:, 3]) == 1).all() and (scheduler.item_piece(items[:, 3]) == 0).all()
    fwd = scheduler.build_schedule(scheduler.FWD, _cu(lq), _cu(lk), hq, hkv)
    assert (fwd[:, 3] == 1 << 16).all()


def test_walk_flags_of_a_bin_too_large_to_rank():
    """Entries of one cost bin are ranked among themselves only up to 64 of them; a hundred documents of one length
    put a hundred entries into every bin, and all of them take the mark that the bin's first entry would get."""
    items = scheduler.build_schedule(scheduler.BWD, _cu([1536] * 100), _cu([1536] * 100), 8, 8, deterministic=True)
    costs, up = items[:, 2], items[:, 3] < 0
    rnd = 256 // 8
    for c in np.unique(costs):
        idx = np.flatnonzero(costs == c)
        assert len(idx) == 100 and (up[idx] == bool((idx[0] // rnd) & 1)).all()
