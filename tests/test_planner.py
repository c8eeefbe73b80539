"""The attention-work planner (distca_amd.planner), on the CPU: plans are valid shard plans, the
work per rank they claim is the work counted from the plan, ranks end within the tolerance of the
mean up to one layer's granularity, and a case small enough to do by hand."""
import numpy as np
import pytest

from distca_amd.compute_metadata import from_planner_output
from distca_amd.planner import PlannerConfig, causal_cost, plan_cost_per_rank, plan_documents


def test_causal_cost():
    assert causal_cost(4, 4) == 10 and causal_cost(1, 7) == 7 and causal_cost(3, 10) == 10 + 9 + 8
    assert causal_cost(5, 5) + causal_cost(3, 8) == causal_cost(8, 8)


def test_by_hand():
    """One document of 8 tokens (36 pairs) on rank 0, nothing on rank 1: the mean is 18, a layer costs
    9 per token pair, so two tokens either side of the middle go to rank 1 as one shard [2, 6)."""
    plan, load = plan_documents([[8], []], PlannerConfig(tolerance=0.0))
    assert [(s.rid, s.dispatch_rid, s.logical_sid, s.shard_len) for s in plan[0]] == [(0, 0, 0, 2), (0, 1, 1, 4), (0, 0, 2, 2)]
    assert load == [18, 18] and plan_cost_per_rank(plan, 2) == [18, 18]


def test_layers_nest_from_the_middle():
    """Three ranks, one long document: two layers are peeled; the first (inner) goes to the first
    recipient, and position order is outer | second layer | first layer | second layer | outer."""
    plan, load = plan_documents([[600], [], []], PlannerConfig(tolerance=0.0))
    doc = plan[0]
    assert sum(s.shard_len for s in doc) == 600 and [s.logical_sid for s in doc] == list(range(len(doc)))
    servers = [s.dispatch_rid for s in doc]
    assert servers[0] == 0 and servers[-1] == 0 and len(doc) == 5 and servers[1] == servers[3] != servers[2]
    assert doc[1].shard_len == doc[3].shard_len and doc[0].shard_len == doc[4].shard_len
    mean = 600 * 601 / 2 / 3
    assert max(abs(x - mean) for x in load) <= 601


@pytest.mark.parametrize("seed,world", [(0, 2), (1, 4), (2, 8), (3, 3)])
def test_random_batches(seed, world):
    rng = np.random.default_rng(seed)
    docs = [[int(x) for x in np.clip(rng.lognormal(6.5, 1.3, size=rng.integers(1, 6)), 2, 20000)] for _ in range(world)]
    cfg = PlannerConfig(tolerance=0.05)
    plan, load = plan_documents(docs, cfg)
    flat = [n for lens in docs for n in lens]
    owners = [r for r, lens in enumerate(docs) for _ in lens]
    assert len(plan) == len(flat)
    for doc, n, owner in zip(plan, flat, owners):
        assert sum(s.shard_len for s in doc) == n and all(s.shard_len > 0 for s in doc)
        assert [s.logical_sid for s in doc] == list(range(len(doc))) and all(s.rid == owner for s in doc)
        assert all(a.dispatch_rid != b.dispatch_rid for a, b in zip(doc, doc[1:])), "neighbours on one server are merged"
    assert plan_cost_per_rank(plan, world) == load
    assert sum(load) == sum(n * (n + 1) // 2 for n in flat)
    mean = sum(load) / world
    before = [sum(n * (n + 1) // 2 for n in lens) for lens in docs]
    # within tolerance of the mean, up to the cost of one token pair of the longest document
    assert max(load) <= mean * (1 + cfg.tolerance) + max(flat) + 2
    assert min(load) >= mean * (1 - cfg.tolerance) - (max(flat) + 2)
    assert max(load) <= max(before)
    # the plan is what the metadata generator takes
    fwd, bwd, out_fwd, out_grad, attn = from_planner_output(world, plan, 64, 16, 0, 2, is_pipeline_tick=False)
    assert int(fwd.fa2a_metadata[1].sum()) > 0
    for r in range(world):
        assert int(fwd.seq_lens[0].send_seqlens[r].sum()) == sum(docs[r])


def test_balanced_input_is_left_alone():
    plan, load = plan_documents([[100, 50], [100, 50]])
    assert all(len(doc) == 1 and doc[0].dispatch_rid == doc[0].rid for doc in plan) and load[0] == load[1]


def test_rejects_empty_documents():
    with pytest.raises(ValueError):
        plan_documents([[10, 0]])


# ---------------------------------------------------------------------------------------------
# The reference's item surface.  Expected values below are the ones its own tests hold
# (tests/test_planner.py:399-452 span lengths per rank, :455-566 placed items, :569-616 piece lists).
# ---------------------------------------------------------------------------------------------
import collections
import random
from types import SimpleNamespace

import torch

from distca_amd.planner import (Item, Planner, batch_to_items_general, batch_to_items_with_dummy, cp_list_to_mlp_list,
                                get_flops)

K = 1024


def _model_config():
    return SimpleNamespace(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, num_hidden_layers=32)


def _planner(world=4, tolerance=0.1, tp=1, pp=1):
    return Planner(world_size=world, parallel_config=SimpleNamespace(tensor_model_parallel_size=tp, pipeline_model_parallel_size=pp),
                   model_config=_model_config(), tolerance_factor=tolerance)


def _dicts(items):
    return [d for it in items for d in it.to_dicts()]


def check_layout(originals, replans):
    """tests/test_planner.py:20-99: for every document some of whose spans were handed to another
    server, the spans still hold all its query tokens, and the handed-over spans, ordered by where
    they end, lie end to start (kv_i - kv_{i-1} == q_i)."""
    q_of = collections.Counter()
    for d in originals:
        q_of[d["seqid"]] += d["q"]
    by_doc = collections.defaultdict(list)
    for d in replans:
        by_doc[d["seqid"]].append(d)
    checked = 0
    for seqid, spans in by_doc.items():
        moved = sorted((d for d in spans if not d["is_original"]), key=lambda d: d["kv"])
        if not moved:
            continue
        checked += 1
        assert sum(d["q"] for d in spans) == q_of[seqid], f"document {seqid} lost or gained query tokens"
        for a, b in zip(moved, moved[1:]):
            assert b["kv"] - a["kv"] == b["q"], f"document {seqid}: handed-over spans {a} and {b} are not adjacent"
    return checked


def check_flops_and_balance(originals, replans, tolerance):
    """tests/test_planner.py:101-184: no pair is lost, and every server that appears ends within
    `tolerance` of the mean."""
    total = sum(get_flops(**d) for d in originals)
    assert total == sum(get_flops(**d) for d in replans)
    per_gpu = collections.Counter()
    for d in replans:
        per_gpu[d["gpuid"]] += get_flops(**d)
    mean = total / len(per_gpu)
    for gpu, flops in per_gpu.items():
        assert mean * (1 - tolerance) <= flops <= mean * (1 + tolerance), f"server {gpu}: {flops} against a mean of {mean}"
    return per_gpu


def test_get_flops_is_the_sum_it_abbreviates():
    for q, kv in [(1, 1), (5, 5), (3, 10), (7, 7), (16, 40)]:
        assert get_flops(q=q, kv=kv, gpuid=3) == sum(kv - i for i in range(q))
    it = Item(None, 40, 0, 0, 0, {"q": 4, "kv": 4}, {"q": 6, "kv": 40})
    assert it.get_flops() == sum(range(1, 5)) + sum(range(35, 41)) == it.total_flops


def test_cp_planner_classical_batch():
    """tests/test_planner.py:345-397: four ranks of 16K tokens holding 1, 2, 4 and 8 documents."""
    planner = _planner()
    batch = [[16 * K], [8 * K] * 2, [4 * K] * 4, [2 * K] * 8]
    initial = batch_to_items_general(batch, 16 * K, 4, _model_config())
    assert [it.src_gpuid for it in initial] == [0] + [1] * 2 + [2] * 4 + [3] * 8 and all(it.complete for it in initial)
    snapshot = repr(initial)
    planned = planner.plan_items(initial)
    assert repr(initial) == snapshot, "the input is not changed"
    assert check_layout(_dicts(initial), _dicts(planned)) >= 1
    per_gpu = check_flops_and_balance(_dicts(initial), _dicts(planned), 0.1)
    assert sorted(per_gpu) == [0, 1, 2, 3]
    before = collections.Counter()
    for it in initial:
        before[it.gpuid] += it.total_flops
    assert max(before.values()) > 1.5 * sum(before.values()) / 4, "the batch was unbalanced to begin with"


@pytest.mark.parametrize("seed", range(6))
def test_cp_planner_random_dp_batches(seed):
    """The reference's commented-out random case (tests/test_planner.py:364-365): every rank holds a
    random number of documents of even length that fill its 16K tokens."""
    random.seed(seed)
    world = random.choice([2, 4, 8])
    batch = []
    for _ in range(world):
        n = random.randint(1, 4)
        cuts = sorted(random.sample(range(1, 8 * K), n - 1))
        batch.append([2 * (b - a) for a, b in zip([0] + cuts, cuts + [8 * K])])
    planner = _planner(world)
    initial = batch_to_items_general(batch, 16 * K, world, _model_config())
    planned = planner.plan_items(initial)
    check_layout(_dicts(initial), _dicts(planned))
    check_flops_and_balance(_dicts(initial), _dicts(planned), 0.1)
    plan = planner.items_to_shardinfo(initial)
    assert [sum(s.shard_len for s in doc) for doc in plan] == [n for lens in batch for n in lens]
    assert plan_cost_per_rank(plan, world) == [sum(get_flops(**d) for d in _dicts(planned) if d["gpuid"] == r) for r in range(world)]


@pytest.mark.parametrize("seed", range(4))
def test_cp_planner_documents_that_span_ranks(seed):
    """Documents longer than a rank (lengths odd and even): the placed items and the planned ones
    both tile every document, pairs are conserved, servers end within the tolerance, and the plan is
    one the metadata generator takes."""
    rng = np.random.default_rng(100 + seed)
    world, budget = 4, 4096
    lens = []
    left = world * budget
    while left > 0:
        n = int(min(left, rng.integers(1, 9000)))
        lens.append(n)
        left -= n
    planner = _planner(world)
    initial = batch_to_items_general([lens], budget, world, _model_config())
    held = collections.Counter()
    for it in initial:
        held[it.src_gpuid] += sum(d["q"] for d in it.items)
    assert [held[r] for r in range(world)] == [budget] * world
    assert sum(it.total_flops for it in initial) == sum(n * (n + 1) // 2 for n in lens)
    planned = planner.plan_items(initial)
    check_flops_and_balance(_dicts(initial), _dicts(planned), 0.1)
    plan = planner.items_to_shardinfo(initial)            # postprocess_items checks that spans tile each document
    assert [sum(s.shard_len for s in doc) for doc in plan] == lens
    for r in range(world):
        assert sum(s.shard_len for doc in plan for s in doc if s.rid == r) == budget, "tokens stay on their linear rank"
    fwd, _, _, _, attn = from_planner_output(world, plan, 64, 16, 0, 2, is_pipeline_tick=False)
    for r in range(world):
        assert int(fwd.seq_lens[0].send_seqlens[r].sum()) == budget


def test_split_item_contract():
    """planner.py:404-494: whole move, partial move of inner layers, nothing to move."""
    mc = _model_config()
    it = Item(mc, 100, 7, 0, 0, {"q": 100, "kv": 100})
    new, moved = it.split_item(50, 1)                      # less than one token pair (101 pairs)
    assert new is None and moved == 0 and it.complete and it.gpuid == 0
    new, moved = it.split_item(3 * 101 + 50, 1)
    assert moved == 3 * 101 == new.total_flops and not it.complete
    assert (new.head, new.tail) == ({"q": 3, "kv": 50}, {"q": 3, "kv": 53}) and new.gpuid == 1 and not new.is_original and new.src_gpuid == 0
    assert (it.head, it.tail) == ({"q": 47, "kv": 47}, {"q": 47, "kv": 100}) and it.is_original
    assert it.total_flops == 5050 - 303
    new2, moved2 = it.split_item(10 ** 9, 2)
    assert new2 is None and moved2 == 5050 - 303 and it.gpuid == 2 and not it.is_original
    with pytest.raises(AssertionError):
        Item(mc, 10, 0, 0, 0)
    with pytest.raises(AssertionError):
        Item(mc, 10, 0, 0, 0, {"q": 10})


def test_mlp_seq_len_expected_by_the_reference():
    planner = _planner()
    items = batch_to_items_general([[256, 256], [128, 384], [512], [10, 502]], 512, 4, _model_config())
    lens, ranges = planner.items_to_mlp_doc_len(items, device="cpu")
    assert [x.tolist() for x in lens] == [[256, 256], [128, 384], [512], [10, 502]] and lens[0].dtype == torch.int32
    assert ranges[3].tolist() == [[0, 10], [0, 502]]
    items = batch_to_items_general([[256, 1024], [256], [128, 384]], 512, 4, _model_config())
    lens, ranges = planner.items_to_mlp_doc_len(items, device="cpu")
    assert [x.tolist() for x in lens] == [[256, 128, 128], [256, 256], [128, 128, 256], [128, 384]]
    assert ranges[0].tolist() == [[0, 256], [0, 128], [896, 1024]] and ranges[1].tolist() == [[128, 384], [640, 896]]
    assert ranges[2].tolist() == [[384, 512], [512, 640], [0, 256]]


def test_batch_to_items_with_dummy_expected_by_the_reference():
    mc = _model_config()

    def rows(items):
        return [(it.seq_len, it.seqid, it.gpuid, it.src_gpuid, [(d["q"], d["kv"]) for d in it.items], it.is_original) for it in items]

    def whole(n, seqid, rank):
        return (n, seqid, rank, rank, [(n, n)], True)

    got = batch_to_items_with_dummy([[256, 256], [128, 384], [512], [10, 502]], 512, 8, mc)
    assert rows(got) == [whole(256, 0, 0), whole(256, 1, 0), whole(128, 2, 1), whole(384, 3, 1), whole(512, 4, 2), whole(10, 5, 3),
                         whole(502, 6, 3)]
    got = batch_to_items_with_dummy([[8], [8], [8], [8], [256, 256], [128, 384], [512], [10, 502]], 512, 8, mc)
    assert rows(got) == [whole(8, 0, 0), whole(8, 1, 1), whole(8, 2, 2), whole(8, 3, 3), whole(256, 4, 4), whole(256, 5, 4),
                         whole(128, 6, 5), whole(384, 7, 5), whole(512, 8, 6), whole(10, 9, 7), whole(502, 10, 7)]
    got = batch_to_items_with_dummy([[8], [8], [8], [8], [256, 768], [512, 10, 502]], 512, 8, mc)
    assert rows(got) == [whole(8, 0, 0), whole(8, 1, 1), whole(8, 2, 2), whole(8, 3, 3), whole(256, 4, 4),
                         (768, 5, 4, 4, [(128, 128), (128, 768)], True), (768, 5, 5, 5, [(256, 384), (256, 640)], False),
                         whole(512, 6, 6), whole(10, 7, 7), whole(502, 8, 7)]
    got = batch_to_items_with_dummy([[256, 768], [512, 10, 502], [8], [8], [8], [8]], 512, 8, mc)
    assert rows(got) == [whole(256, 0, 0), (768, 1, 0, 0, [(128, 128), (128, 768)], True),
                         (768, 1, 1, 1, [(256, 384), (256, 640)], False), whole(512, 2, 2), whole(10, 3, 3), whole(502, 4, 3),
                         whole(8, 5, 4), whole(8, 6, 5), whole(8, 7, 6), whole(8, 8, 7)]
    assert repr(got[0]) == "<Item seqid=0 src_gpuid = 0 gpuid=0 complete=q=256 kv=256>"
    assert repr(got[1]) == "<Item seqid=1 src_gpuid = 0 gpuid=0 split=head(q=128, kv=128) tail(q=128, kv=768)>"
    with pytest.raises(ValueError, match="Not enough space"):
        batch_to_items_general([[600]], 256, 2, mc)


def test_cp_list_to_mlp_list_expected_by_the_reference():
    assert cp_list_to_mlp_list([[512, 512], [512, 512], [1], [1]], 4, 1024) == [[512, 512], [512, 512], [1], [1]]
    assert cp_list_to_mlp_list([[1], [1], [1376, 672]], 4, 1024) == [[1], [1], [512, 512], [176, 176, 672]]
    assert cp_list_to_mlp_list([[256, 1024, 768]] + [[8]] * 8, 12, 512) == \
        [[256, 128, 128], [256, 256], [128, 128, 128, 128], [256, 256]] + [[8]] * 8
    big = [[1376, 336, 336], [1024, 1024], [680, 680, 344, 344], [800, 800, 224, 224], [1024, 1024], [440, 440, 584, 584],
           [1024, 1024], [1024, 1024]]
    assert cp_list_to_mlp_list([[8]] * 8 + [[1376, 4080, 2288, 3376, 5264]], 16, 2048) == [[8]] * 8 + big
    assert cp_list_to_mlp_list([[1376, 4080, 2288, 3376, 5264]] + [[8]] * 8, 16, 2048) == big + [[8]] * 8
    assert cp_list_to_mlp_list([[100]], 3, 128) == [[100], [], []]


def test_planner_plan_returns_metadata_for_a_step():
    """Planner.plan (planner.py:567-608): metadata of the four all-to-alls, attention arguments per
    server, span lengths and ranges per linear rank."""
    planner = _planner(world=4, tolerance=0.05)
    items = batch_to_items_general([[2048], [512, 512, 1024], [1024, 1024], [2048]], 2048, 4, _model_config())
    fa2a, attn, lens, ranges = planner.plan(items, is_resend_qkv=True, device="cpu")
    assert len(fa2a) == 4 and len(attn) == 4 and [int(x.sum()) for x in lens] == [2048] * 4
    assert all(int(r[:, 1].max()) <= 2048 for r in ranges)
    plan = planner.items_to_shardinfo(items)
    load = plan_cost_per_rank(plan, 4)
    assert max(load) <= 1.05 * sum(load) / 4 + 2049
    p8 = Planner.from_individual_params(tp_size=8, pp_size=2, dp_size=4, world_size=64, hidden_size_q=512, hidden_size_k=128)
    assert p8.attention_server_world_size == 8 and p8._hidden_sizes() == (512, 128)
