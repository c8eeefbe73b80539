"""One layer step of several ranks, played on one GPU: every rank's pack / unpack and CA-server
tick runs through the library on that rank's own buffers, and the transport is replaced by
copying the byte ranges the all-to-all metadata names (what the reference's tests do in
tests/test_fa2a_metadata.py:160-175).  Documents are cut into shards that live on one rank for
the linear layers and are attended on another; a K/V shard may be needed on several ranks (the
replicated pack) and several times on one rank (aliased receive offsets, duplicate-gradient sum).
Checked against the oracle's attention over whole documents."""
import math

import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, make_qkv
from oracle.attention import ca_reference_bwd, ca_reference_fwd

pytestmark = pytest.mark.gpu


def _plan(seed, world, docs, max_shards, lo, hi):
    from distca_amd.compute_metadata import ShardInfo
    rng = np.random.default_rng(seed)
    plan = []
    for _ in range(docs):
        n = int(rng.integers(1, max_shards + 1))
        plan.append([ShardInfo(int(rng.integers(world)), int(rng.integers(world)), i, int(rng.integers(lo, hi + 1))) for i in range(n)])
    return plan


@pytest.mark.parametrize("seed,world,docs,max_shards,lo,hi", [(11, 3, 5, 4, 40, 300), (12, 4, 6, 5, 1, 130), (13, 2, 3, 3, 500, 1500)])
def test_layer_step_of_several_ranks(cuda, seed, world, docs, max_shards, lo, hi):
    _layer_step(cuda, world, _plan(seed, world, docs, max_shards, lo, hi), seed, replicas=True)


def _planner_for_the_test(world, tolerance):
    from types import SimpleNamespace
    from distca_amd.planner import Planner
    return Planner(world_size=world, tolerance_factor=tolerance,
                   parallel_config=SimpleNamespace(tensor_model_parallel_size=1, pipeline_model_parallel_size=1),
                   model_config=SimpleNamespace(hidden_size=8 * 128, num_attention_heads=8, num_key_value_heads=2))


def test_layer_step_of_a_planned_batch(cuda):
    """The plan comes from the planner's item surface (Item -> Planner.items_to_shardinfo): four
    ranks, one of them with a long document whose middle layers are handed to the others."""
    from distca_amd.planner import Item, plan_cost_per_rank
    docs = [[2600, 300], [420], [150, 90, 64], [700]]
    planner = _planner_for_the_test(4, 0.02)
    items = []
    for r, lens in enumerate(docs):
        for n in lens:
            items.append(Item(planner.model_config, n, len(items), r, r, {"q": n, "kv": n}))
    plan = planner.items_to_shardinfo(items)
    load = plan_cost_per_rank(plan, 4)
    assert sum(load) == sum(n * (n + 1) // 2 for lens in docs for n in lens) and max(load) < 1.1 * sum(load) / 4
    assert len(plan[0]) >= 5, "the long document is cut into nested layers"
    _layer_step(cuda, 4, plan, 14, replicas=True)


def test_layer_step_of_a_planned_batch_whose_documents_span_ranks(cuda):
    """Context-parallel placement (batch_to_items_general): ranks of 1024 tokens, a document of 2200
    tokens lies on three of them as head and tail spans; the planner then balances the servers."""
    from distca_amd.planner import batch_to_items_general, plan_cost_per_rank
    planner = _planner_for_the_test(4, 0.05)
    lens = [2200, 500, 372, 1024]
    items = batch_to_items_general([lens], 1024, 4, planner.model_config)
    assert sum(1 for it in items if it.seqid == 0) == 3
    plan = planner.items_to_shardinfo(items)
    assert [sum(s.shard_len for s in doc) for doc in plan] == lens and len({s.rid for s in plan[0]}) == 3
    load = plan_cost_per_rank(plan, 4)
    assert max(load) < 1.1 * sum(load) / 4 + 2201
    _layer_step(cuda, 4, plan, 16, replicas=True)


def test_layer_step_with_an_idle_server_and_an_empty_owner(cuda):
    """Rank 2 holds tokens but serves no attention; rank 3 serves attention but holds no tokens."""
    from distca_amd.compute_metadata import ShardInfo
    plan = [[ShardInfo(0, 0, 0, 100), ShardInfo(1, 3, 1, 50), ShardInfo(1, 0, 2, 30)], [ShardInfo(2, 1, 0, 70)]]
    _layer_step(cuda, 4, plan, 15, replicas=False, every_rank_serves=False)


def _layer_step(cuda, world, plan, seed, replicas, every_rank_serves=True):
    from distca_amd.compute_metadata import from_planner_output, simulate_fa2a, step_params
    from distca_amd.dispatch_fn import pre_all2all_layout_transfer, pre_all2all_layout_transfer_backward
    from distca_amd.fused_comm_attn import (FlashAttnArgs, fused_comm_attn_backward, fused_comm_attn_forward,
                                            post_a2a_attn_out_with_lse, post_a2a_attn_out_with_lse_backward)
    hq, hkv, d = 8, 2, 128
    lse_elems = math.ceil(hq * 4 / 16) * 16 // 2
    md = from_planner_output(world, plan, hq * d, hkv * d, lse_elems, 2, is_pipeline_tick=False, is_resend_qkv=True)
    qkv_fwd, qkv_grad, out_fwd, request, attn = md
    if every_rank_serves:
        assert all(a["max_seqlen_q"] > 0 for a in attn), "every rank of this plan serves attention"
    if replicas:
        assert qkv_fwd.max_cp_degree > 1, "some K/V shard of this plan is needed on several ranks"
        assert any(int(x.num_copies.sum()) > 0 for x in qkv_grad.kv_grad_send_dedup), "some shard is needed twice on one rank"
    steps = [step_params(r, md, cuda) for r in range(world)]
    fa_args = FlashAttnArgs(hq, hkv, d)

    # whole documents and their oracle
    doc_len = [sum(s.shard_len for s in doc) for doc in plan]
    cu_doc = np.concatenate([[0], np.cumsum(doc_len)]).astype(np.int32)
    T = int(cu_doc[-1])
    q, k, v, do = make_qkv(T, T, hq, hkv, d, seed)
    ref_out, ref_lse = ca_reference_fwd(q, k, v, cu_doc, cu_doc)
    rows = [[] for _ in range(world)]              # global token rows each linear rank holds, in its shard order
    for di, doc in enumerate(plan):
        start = int(cu_doc[di])
        for s in doc:
            rows[s.rid] += list(range(start, start + s.shard_len))
            start += s.shard_len
    rows = [torch.tensor(r, dtype=torch.int64) for r in rows]
    flat = lambda x, r: x[rows[r]].reshape(len(rows[r]), x.shape[1] * x.shape[2]).to(cuda)
    bufs = lambda sizes: [torch.full((int(n),), 0x5A, dtype=torch.uint8, device=cuda) for n in sizes]

    def exchange(m, send):
        recv = bufs(m.fa2a_metadata[3].sum(dim=1))
        simulate_fa2a(send, recv, m.fa2a_metadata)
        return recv

    # ---- forward ---------------------------------------------------------------------------------------
    send = bufs(qkv_fwd.fa2a_metadata[1].sum(dim=1))
    for r in range(world):
        print(f"rank {r}: pack q/k/v, {len(rows[r])} tokens", flush=True)
        pre_all2all_layout_transfer(flat(q, r), flat(k, r), flat(v, r), steps[r].qkv_fwd_metadata, buffer=send[r])
    recv = exchange(qkv_fwd, send)
    out_send = bufs(out_fwd.fa2a_metadata[1].sum(dim=1))
    for a in range(world):
        print(f"rank {a}: server forward, cu_q {attn[a]['cu_seqlens_q'].tolist()}", flush=True)
        fused_comm_attn_forward(recv[a], out_send[a], steps[a], fa_args)
    out_recv = exchange(out_fwd, out_send)
    outs, lses = [], []
    for r in range(world):
        attn_out, lse_bytes = post_a2a_attn_out_with_lse(out_recv[r], flat(q, r), hq, steps[r].attn_out_fwd_metadata)
        torch.cuda.synchronize()
        n = len(rows[r])
        assert_close_bf16(attn_out.reshape(n, hq, d), ref_out[rows[r]], f"out of rank {r}")
        lse = lse_bytes.contiguous().view(torch.float32)
        assert lse.shape == (n, hq)
        assert n == 0 or (lse.cpu() - ref_lse.T[rows[r]]).abs().max().item() <= 2e-3
        outs.append(attn_out)
        lses.append(lse_bytes.contiguous())

    # ---- backward --------------------------------------------------------------------------------------
    out_all = torch.empty((T, hq, d), dtype=torch.bfloat16)
    lse_all = torch.empty((hq, T), dtype=torch.float32)
    for r in range(world):
        out_all[rows[r]] = outs[r].reshape(-1, hq, d).cpu()
        lse_all[:, rows[r]] = lses[r].view(torch.float32).T.cpu()
    ref_dq, ref_dk, ref_dv = ca_reference_bwd(do, q, k, v, cu_doc, cu_doc, out=out_all, softmax_lse=lse_all)
    send = bufs(request.fa2a_metadata[1].sum(dim=1))
    for r in range(world):
        post_a2a_attn_out_with_lse_backward(send[r], flat(do, r), outs[r], lses[r], flat(q, r), flat(k, r), flat(v, r),
                                            steps[r].attn_out_bwd_metadata)
    recv = exchange(request, send)
    grad_send = bufs(qkv_grad.fa2a_metadata[1].sum(dim=1))
    for a in range(world):
        print(f"rank {a}: server backward", flush=True)
        fused_comm_attn_backward(recv[a], grad_send[a], steps[a], fa_args)
    grad_recv = exchange(qkv_grad, grad_send)
    for r in range(world):
        dq, dk, dv = pre_all2all_layout_transfer_backward(steps[r].qkv_bwd_metadata, torch.bfloat16, buffer=grad_recv[r])
        torch.cuda.synchronize()
        n = len(rows[r])
        assert_close_bf16(dq.reshape(n, hq, d), ref_dq[rows[r]], f"dq of rank {r}")
        # a shard's gradient is a bf16 sum of one bf16 gradient per task that read it (up to max_shards): 4e-2 / 3e-3
        assert_close_bf16(dk.reshape(n, hkv, d), ref_dk[rows[r]], f"dk of rank {r}", max_abs=4e-2, mean_rel=3e-3)
        assert_close_bf16(dv.reshape(n, hkv, d), ref_dv[rows[r]], f"dv of rank {r}", max_abs=4e-2, mean_rel=3e-3)
