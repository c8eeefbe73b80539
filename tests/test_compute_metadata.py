"""Multi-rank all-to-all metadata from a shard plan (distca_amd.compute_metadata), on the CPU.

What pins it: a case small enough to lay out by hand; and, on random plans, the properties the
reference's own test of this generator checks (tests/test_shard_info_to_fa2a.py:199-308) with the
byte copies done by the oracle's restatement of the pack/unpack kernels: every query shard
arrives at its attention rank in task order, every task finds its document prefix as K/V,
gradients of all K/V copies on all ranks sum into the owner's shard, and attention outputs and
backward requests travel to where the plan says.  The expected tensors are built from the plan
directly, not from the generator's layout."""
import math

import numpy as np
import pytest
import torch

from distca_amd.compute_metadata import (ShardInfo, backward_from_planner_output, from_planner_output, get_fa2a_metadata,
                                         get_per_token_bytes, simulate_fa2a)
from oracle import fa2a as O


def random_plan(seed, world, num_docs, max_shards, max_len):
    rng = np.random.default_rng(seed)
    plan = []
    for _ in range(num_docs):
        n = int(rng.integers(1, max_shards + 1))
        plan.append([ShardInfo(int(rng.integers(world)), int(rng.integers(world)), i, int(rng.integers(1, max_len + 1)))
                     for i in range(n)])
    return plan


def test_per_token_bytes():
    # Llama-3-8B head geometry, bf16: q 4096 elements, k/v 1024, lse 32 heads x fp32 = 64 bf16 elements
    assert get_per_token_bytes(4096, 1024, 64, 2, False, False) == (8192, 2048, 8192)
    assert get_per_token_bytes(4096, 1024, 64, 2, False, True) == (8192, 2048, 8192 + 128)
    assert get_per_token_bytes(4096, 1024, 64, 2, True, False) == (3 * 8192 + 128, 2048, 8192)
    # padding to 16 bytes: 3 heads of 2 elements -> 3*6*2 + 6*2... use odd sizes
    q, k, o = get_per_token_bytes(12, 8, 3, 2, True, False)
    assert q == 80 and q % 16 == 0 and k == 16 and o == 32
    with pytest.raises(AssertionError):
        get_per_token_bytes(8, 8, 2, 2, True, True)


def test_fa2a_metadata_by_hand():
    send = torch.tensor([[192, 96], [0, 144]])
    sd, ssz, rd, rsz = get_fa2a_metadata(send)
    assert sd.tolist() == [[0, 192], [0, 0]] and ssz.tolist() == send.tolist()
    assert rsz.tolist() == [[192, 0], [96, 144]] and rd.tolist() == [[0, 0], [192, 96]]


def test_layout_by_hand():
    plan = [[ShardInfo(0, 1, 0, 2), ShardInfo(1, 1, 1, 3)], [ShardInfo(0, 0, 0, 4)]]
    fwd, bwd, out_fwd, out_grad, attn = from_planner_output(2, plan, 8, 8, 0, 2, is_pipeline_tick=False)
    assert fwd.fa2a_metadata[1].tolist() == [[192, 96], [0, 144]]
    assert fwd.fa2a_metadata[0].tolist() == [[0, 192], [0, 0]] and fwd.fa2a_metadata[2].tolist() == [[0, 0], [192, 96]]
    q_s, k_s, v_s = fwd.send_memcpy_metadata
    assert q_s[0].tolist() == [192, 0] and k_s[0].tolist() == [[224, 64]] and v_s[0].tolist() == [[256, 128]]
    assert q_s[1].tolist() == [0] and k_s[1].tolist() == [[48]] and v_s[1].tolist() == [[96]]
    q_r, k_r, v_r = fwd.recv_memcpy_metadata
    assert q_r[0].tolist() == [0] and k_r[0].tolist() == [64] and v_r[0].tolist() == [128]
    assert q_r[1].tolist() == [0, 96] and k_r[1].tolist() == [32, 32, 144] and v_r[1].tolist() == [64, 64, 192]
    assert fwd.seq_lens[1].recv_seqlens[1].tolist() == [2, 2, 3] and fwd.seq_lens[0].recv_seqlens[1].tolist() == [2, 3]
    assert fwd.tensor_shape[1].send_shape[0] == torch.Size((1, 6, 8)) and fwd.tensor_shape[1].recv_shape[1] == torch.Size((7, 8))
    assert [m.tolist() for m in fwd.kv_replica_mask] == [[[1], [1]], [[1]]]
    assert fwd.my_rank_send_sz == [192, 144] and fwd.my_rank_send_offset == [0, 0] and fwd.my_rank_recv_offset == [0, 96]
    d = bwd.kv_grad_send_dedup[1]
    assert d.num_copies.tolist() == [1, 0, 0] and d.copy_start_id[0, 0].item() == 2 and d.main_copy_mask.tolist() == [1, 0, 1]
    assert bwd.fa2a_metadata[0].tolist() == [[0, 192], [0, 96]] and bwd.fa2a_metadata[1].tolist() == [[192, 0], [96, 144]]
    assert attn[1]["cu_seqlens_q"].tolist() == [0, 2, 5] and attn[1]["cu_seqlens_kv"].tolist() == [0, 2, 7]
    assert attn[0]["max_seqlen_kv"] == 4 and attn[1]["max_seqlen_kv"] == 5
    # attention output: 16-byte tokens, q shards only
    assert out_grad.fa2a_metadata[1].tolist() == [[64, 32], [0, 48]]
    assert out_fwd.send_memcpy_metadata[0][1].tolist() == [0, 32] and out_fwd.recv_memcpy_metadata[0][0].tolist() == [64, 0]


def test_replica_numbering_by_hand():
    """A K/V shard needed on two attention ranks is sent twice from its owner, replica 0 to the
    rank that needs it first in (document, shard) order."""
    plan = [[ShardInfo(0, 1, 0, 2), ShardInfo(0, 0, 1, 2), ShardInfo(0, 1, 2, 2)]]
    fwd, *_ = from_planner_output(2, plan, 8, 8, 0, 2, is_pipeline_tick=False)
    assert fwd.kv_replica_mask[0].tolist() == [[1, 1], [1, 1], [1, 0]]
    # regions from rank 0: to rank 0 = q(0,1) 32 | k(0,0) k(0,1) 64 | v 64 = 160; to rank 1 = q 64 | k(0,0),(0,1),(0,2) 96 | v 96
    assert fwd.fa2a_metadata[1][0].tolist() == [160, 256]
    k_s = fwd.send_memcpy_metadata[1][0]
    assert k_s.tolist() == [[160 + 64, 32 + 32, 160 + 64 + 64], [32, 160 + 64 + 32, -1]]


def _tokens(plan, world):
    """Per linear rank the (document, position) ids of its tokens in order, and per attention rank
    the ids of its query rows and K/V rows, straight from the plan."""
    base = np.cumsum([0] + [sum(s.shard_len for s in doc) for doc in plan])
    lin = [[] for _ in range(world)]
    aq = [[] for _ in range(world)]
    ak = [[] for _ in range(world)]
    tasks = [[] for _ in range(world)]
    for d, doc in enumerate(plan):
        start = 0
        for sh in doc:
            ids = list(range(base[d] + start, base[d] + start + sh.shard_len))
            lin[sh.rid] += ids
            aq[sh.dispatch_rid] += ids
            ak[sh.dispatch_rid] += list(range(base[d], base[d] + start + sh.shard_len))
            tasks[sh.dispatch_rid].append((sh.shard_len, start + sh.shard_len))
            start += sh.shard_len
    return [np.array(x, dtype=np.int64) for x in lin], [np.array(x, dtype=np.int64) for x in aq], \
        [np.array(x, dtype=np.int64) for x in ak], tasks, int(base[-1])


def _payload(ids, hidden, salt):
    return (ids[:, None] * 64 + np.arange(hidden)[None, :] + salt).astype(np.int32)


def _exchange(md, send_bufs):
    recv = [np.zeros(int(md.fa2a_metadata[3][r].sum()), np.uint8) for r in range(len(send_bufs))]
    simulate_fa2a(send_bufs, recv, md.fa2a_metadata)
    return recv


@pytest.mark.parametrize("seed,world,docs,max_shards,max_len", [(0, 2, 4, 2, 9), (1, 3, 6, 4, 17), (2, 4, 9, 5, 8), (3, 1, 3, 3, 5),
                                                               (4, 4, 2, 6, 12)])
def test_round_trip_on_random_plans(seed, world, docs, max_shards, max_len):
    plan = random_plan(seed, world, docs, max_shards, max_len)
    hq, hk, esz = 8, 4, 4                       # int32 "elements": q tokens 32 bytes, k tokens 16 bytes
    fwd, bwd, out_fwd, out_grad, attn = from_planner_output(world, plan, hq, hk, 0, esz, is_pipeline_tick=False)
    lin, aq, ak, tasks, _ = _tokens(plan, world)

    # transfer sizes agree on both sides; receive regions of a rank tile its buffer without overlap
    sd, ssz, rd, rsz = fwd.fa2a_metadata
    assert torch.equal(ssz.t(), rsz)
    for r in range(world):
        spans = sorted((int(rd[s, r]), int(rd[s, r]) + int(ssz[s, r])) for s in range(world))
        assert spans[0][0] == 0 and all(a[1] == b[0] for a, b in zip(spans, spans[1:]))

    # ---- forward: q, k, v to the attention ranks -------------------------------------------------------
    send = []
    for r in range(world):
        m = fwd.get_slice(r)
        buf = np.full(int(ssz[r].sum()), 0xEE, np.uint8)
        q, k, v = _payload(lin[r], hq, 0), _payload(lin[r], hk, 1 << 20), _payload(lin[r], hk, 1 << 21)
        assert tuple(m.tensor_shape[0].send_shape) == q.shape and tuple(m.tensor_shape[1].send_shape[1:]) == k.shape
        O.copy_non_cp(q, buf, m.send_memcpy_metadata[0], m.seq_lens[0].send_seqlens)
        O.copy_cp(k, buf, m.kv_replica_mask, m.send_memcpy_metadata[1], m.seq_lens[1].send_seqlens)
        O.copy_cp(v, buf, m.kv_replica_mask, m.send_memcpy_metadata[2], m.seq_lens[1].send_seqlens)
        send.append(buf)
    recv = _exchange(fwd, send)
    for a in range(world):
        m = fwd.get_slice(a)
        q = np.zeros(tuple(m.tensor_shape[0].recv_shape), np.int32)
        k = np.zeros(tuple(m.tensor_shape[1].recv_shape), np.int32)
        v = np.zeros_like(k)
        O.copy_non_cp(q, recv[a], m.recv_memcpy_metadata[0], m.seq_lens[0].recv_seqlens, to_buffer=False)
        O.copy_non_cp(k, recv[a], m.recv_memcpy_metadata[1], m.seq_lens[1].recv_seqlens, to_buffer=False)
        O.copy_non_cp(v, recv[a], m.recv_memcpy_metadata[2], m.seq_lens[1].recv_seqlens, to_buffer=False)
        assert np.array_equal(q, _payload(aq[a], hq, 0))
        assert np.array_equal(k, _payload(ak[a], hk, 1 << 20)) and np.array_equal(v, _payload(ak[a], hk, 1 << 21))
        cu_q = np.cumsum([0] + [t[0] for t in tasks[a]])
        cu_k = np.cumsum([0] + [t[1] for t in tasks[a]])
        assert attn[a]["cu_seqlens_q"].tolist() == cu_q.tolist() and attn[a]["cu_seqlens_kv"].tolist() == cu_k.tolist()

    # ---- backward: gradients of every copy sum into the owner's shard ----------------------------------
    rng = np.random.default_rng(seed + 100)
    total = sum(len(x) for x in lin)
    want_dk = np.zeros((total, hk), np.float32)
    send = []
    for a in range(world):
        m = bwd.get_slice(a)
        dq = _payload(aq[a], hq, 7).astype(np.float32)
        dk = rng.integers(-8, 9, size=(len(ak[a]), hk)).astype(np.float32)
        np.add.at(want_dk, ak[a], dk)
        d = m.kv_grad_send_dedup
        dk_t = torch.from_numpy(dk.copy())
        O.grad_sum(dk_t, d.num_copies, d.copy_start_id, m.seq_lens[1].send_seqlens)
        buf = np.full(int(bwd.fa2a_metadata[1][a].sum()), 0xEE, np.uint8)
        O.copy_non_cp(dq, buf, m.send_memcpy_metadata[0], m.seq_lens[0].send_seqlens)
        for off in m.send_memcpy_metadata[1:]:
            O.copy_non_cp(dk_t.numpy(), buf, off, m.seq_lens[1].send_seqlens, copy_seq_mask=d.main_copy_mask)
        send.append(buf)
    recv = _exchange(bwd, send)
    for r in range(world):
        m = bwd.get_slice(r)
        dq = np.zeros(tuple(m.tensor_shape[0].recv_shape), np.float32)
        O.copy_non_cp(dq, recv[r], m.recv_memcpy_metadata[0], m.seq_lens[0].recv_seqlens, to_buffer=False)
        assert np.array_equal(dq, _payload(lin[r], hq, 7).astype(np.float32))
        for off in m.recv_memcpy_metadata[1:]:
            planes = np.zeros(tuple(m.tensor_shape[1].recv_shape), np.float32)
            O.copy_cp(planes, recv[r], m.kv_replica_mask, off, m.seq_lens[1].recv_seqlens, to_buffer=False)
            assert np.array_equal(planes.sum(0), want_dk[lin[r]])

    # ---- attention output back to the linear ranks, and its gradient out again -------------------------
    send = []
    for a in range(world):
        m = out_fwd.get_slice(a)
        buf = np.zeros(int(out_fwd.fa2a_metadata[1][a].sum()), np.uint8)
        O.copy_non_cp(_payload(aq[a], hq, 3), buf, m.send_memcpy_metadata[0], m.seq_lens[0].send_seqlens)
        send.append(buf)
    recv = _exchange(out_fwd, send)
    send = []
    for r in range(world):
        m = out_fwd.get_slice(r)
        out = np.zeros(tuple(m.tensor_shape[0].recv_shape), np.int32)
        O.copy_non_cp(out, recv[r], m.recv_memcpy_metadata[0], m.seq_lens[0].recv_seqlens, to_buffer=False)
        assert np.array_equal(out, _payload(lin[r], hq, 3))
        g = out_grad.get_slice(r)
        buf = np.zeros(int(out_grad.fa2a_metadata[1][r].sum()), np.uint8)
        O.copy_non_cp(out, buf, g.send_memcpy_metadata[0], g.seq_lens[0].send_seqlens)
        send.append(buf)
    recv = _exchange(out_grad, send)
    for a in range(world):
        g = out_grad.get_slice(a)
        got = np.zeros(tuple(g.tensor_shape[0].recv_shape), np.int32)
        O.copy_non_cp(got, recv[a], g.recv_memcpy_metadata[0], g.seq_lens[0].recv_seqlens, to_buffer=False)
        assert np.array_equal(got, _payload(aq[a], hq, 3))


def test_resend_metadata_token_sizes():
    """The step with q/k/v sent again in backward: the reply carries [out | lse], the request
    [dO | O | lse | q] + k + v, the gradients plain q/k/v tokens; same shard order throughout."""
    plan = random_plan(5, 3, 5, 3, 11)
    heads, d = 4, 8
    hq, hk, esz = heads * d, 2 * d, 2
    lse = math.ceil(heads * 4 / 16) * 16 // esz
    fwd, grad, out_fwd, request, attn = from_planner_output(3, plan, hq, hk, lse, esz, is_pipeline_tick=False, is_resend_qkv=True)
    request2, grad2, attn2 = backward_from_planner_output(3, plan, hq, hk, lse, esz)
    qb, kb, ob = hq * esz, hk * esz, (hq + lse) * esz
    mq = (3 * hq + lse) * esz
    for r in range(3):
        f, g, o, q = fwd.get_slice(r), grad.get_slice(r), out_fwd.get_slice(r), request.get_slice(r)
        assert f.tensor_shape[0].send_shape[1] * esz == qb and q.tensor_shape[0].send_shape[1] * esz == mq
        assert o.tensor_shape[0].recv_shape[1] * esz == ob and g.tensor_shape[0].send_shape[1] * esz == qb
        assert torch.equal(f.seq_lens[0].send_seqlens, q.seq_lens[0].send_seqlens)
        assert torch.equal(q.kv_replica_mask, f.kv_replica_mask)
        assert torch.equal(request2.get_slice(r).send_memcpy_metadata[1], q.send_memcpy_metadata[1])
        assert torch.equal(grad2.get_slice(r).fa2a_metadata[1], g.fa2a_metadata[1])
        assert attn2[r]["cu_seqlens_kv"].tolist() == attn[r]["cu_seqlens_kv"].tolist()
    tokens_q = sum(s.shard_len for doc in plan for s in doc)
    assert int(out_fwd.fa2a_metadata[1].sum()) == tokens_q * ob
    assert int(request.fa2a_metadata[1].sum()) - int(fwd.fa2a_metadata[1].sum()) == tokens_q * (mq - qb)
    tick = from_planner_output(3, plan, hq, hk, lse, esz, is_pipeline_tick=True)
    assert tick[1] is None and tick[3] is None and tick[2].tensor_shape[0].recv_shape[0][1] * esz == ob
    with pytest.raises(AssertionError):
        from_planner_output(3, plan, hq, hk, lse, esz, is_pipeline_tick=True, is_resend_qkv=True)


def test_rank_without_attention_work():
    plan = [[ShardInfo(0, 0, 0, 3), ShardInfo(1, 0, 1, 2)]]
    fwd, bwd, _, _, attn = from_planner_output(2, plan, 8, 8, 0, 2, is_pipeline_tick=False)
    assert attn[1]["cu_seqlens_q"].tolist() == [0] and fwd.seq_lens[0].recv_seqlens[1].numel() == 0
    assert fwd.fa2a_metadata[3][1].tolist() == [0, 0] and bwd.kv_grad_send_dedup[1].num_copies.numel() == 0
