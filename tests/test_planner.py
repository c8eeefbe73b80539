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
