"""The metadata types and the single-rank plan against the hand-derived example of one
document cut into shards a | b | c (compute_metadata.py:404-459,202-273,277-323 of the
reference, world size 1): tasks Lq = [a, b, c], Lk = [a, a+b, a+b+c]; K/V entries
[k0 | k0 k1 | k0 k1 k2]; main copies are the first occurrences; duplicates are summed into them."""
import warnings

import numpy as np
import pytest
import torch

from distca_amd import metadata
from oracle import fa2a


def test_worked_example_single_document():
    a, b, c = 5, 3, 7
    p = metadata.single_rank_plan([[a, b, c]], 4, 2)
    assert p.q_seqlens.tolist() == [a, b, c]
    assert p.kv_seqlens.tolist() == [a, a + b, a + b + c]
    assert p.kv_entry_tokens.tolist() == [a, a, b, a, b, c]
    assert p.dedup.main_copy_mask.tolist() == [1, 0, 1, 0, 0, 1]
    assert p.dedup.num_copies.tolist() == [2, 0, 1, 0, 0, 0]
    assert p.dedup.copy_start_id[0].tolist() == [a, 2 * a + b]
    assert p.dedup.copy_start_id[2, 0].item() == 3 * a + b
    m = metadata.get_attn_metadata(p.q_seqlens, p.kv_seqlens)
    assert m["cu_seqlens_q"].tolist() == [0, a, a + b, a + b + c]
    assert m["cu_seqlens_kv"].tolist() == [0, a, 2 * a + b, 3 * a + 2 * b + c]
    assert (m["max_seqlen_q"], m["max_seqlen_kv"]) == (max(a, b, c), a + b + c)


def test_normalize_dtypes():
    d = metadata.DedupGradSumMetadata(torch.tensor([1, 0]), torch.tensor([[3], [0]], dtype=torch.int32),
                                      torch.tensor([1, 0])).normalize("cpu")
    assert (d.num_copies.dtype, d.copy_start_id.dtype, d.main_copy_mask.dtype) == (torch.int32, torch.int64, torch.int8)
    s = metadata.SeqLens(torch.tensor([1, 2], dtype=torch.int32), torch.tensor([3], dtype=torch.int32)).normalize("cpu")
    assert s.send_seqlens.dtype == torch.int64 and s.recv_seqlens.dtype == torch.int64
    s2 = metadata.SeqLens((torch.tensor([1]),), (torch.tensor([2]),)).normalize("cpu")
    assert isinstance(s2.send_seqlens, tuple)


def test_layouts_tile_the_buffers_and_alias_duplicates():
    p = metadata.single_rank_plan([[4, 2, 3], [6]], 6, 2)
    assert p.out_lse_bytes == 1568 and p.merged_q_bytes % 16 == 0
    for backward in (False, True):
        q_off, k_off, v_off, total = p.request_layout(backward)
        qb = p.merged_q_bytes if backward else p.q_bytes
        # distinct regions tile [0, total) exactly once
        regions = [(int(o), int(n) * qb) for o, n in zip(q_off, p.q_seqlens)]
        seen = set()
        for off_list in (k_off, v_off):
            for e, o in enumerate(off_list.tolist()):
                if (o, id(off_list)) not in seen and p.dedup.main_copy_mask[e]:
                    regions.append((o, int(p.kv_entry_tokens[e]) * p.k_bytes))
        regions.sort()
        cur = 0
        for o, n in regions:
            assert o == cur
            cur += n
        assert cur == total
        # every duplicate entry reads its main copy's bytes
        for e, s in enumerate(p.kv_entry_shard.tolist()):
            main = p.kv_entry_shard.tolist().index(s)
            assert k_off[e] == k_off[main] and v_off[e] == v_off[main]


def test_plan_drives_the_oracle_round_trip():
    """Unpacking a request laid out by the plan materialises each task's prefix; the masked pack of
    the summed gradients sends every stored shard once."""
    p = metadata.single_rank_plan([[3, 2], [4]], 2, 1, head_dim=8)
    rng = np.random.default_rng(0)
    stored = p.stored_shard_tokens.numpy()
    k = rng.integers(0, 255, size=(int(stored.sum()), p.k_bytes), dtype=np.uint8)
    q_off, k_off, v_off, total = p.request_layout(False)
    buf = np.zeros(total, np.uint8)
    st = np.concatenate([[0], np.cumsum(stored)])
    for s in range(len(stored)):                                  # the sender writes each stored shard once
        o = int(k_off[p.kv_entry_shard.tolist().index(s)])
        buf[o:o + stored[s] * p.k_bytes] = k[st[s]:st[s + 1]].reshape(-1)
    recv_k = np.zeros((p.num_kv_tokens, p.k_bytes), np.uint8)
    fa2a.copy_non_cp(recv_k, buf, k_off.numpy(), p.kv_entry_tokens.numpy(), None, False)
    want = np.concatenate([k[st[s]:st[s + 1]] for s in p.kv_entry_shard.tolist()])
    assert np.array_equal(recv_k, want)                            # [k0 | k0 k1 | k2]
    g = torch.arange(p.num_kv_tokens * 4, dtype=torch.float32).reshape(-1, 4)
    summed = g.clone()
    fa2a.grad_sum(summed, p.dedup.num_copies.numpy(), p.dedup.copy_start_id.numpy(), p.kv_entry_tokens.numpy())
    assert torch.equal(summed[0:3], g[0:3] + g[3:6])              # k0's copy in task 1 folded into the main copy


def test_single_rank_step_params_are_consistent():
    """The four AlltoAllMetadata of a step agree with each other: what one side sends is what the
    other receives, sizes tile the buffers, normalize() yields the dtypes the kernels read."""
    p = metadata.single_rank_plan([[4, 2, 3], [6]], 6, 2)
    step = metadata.single_rank_step_params(p)
    for md in (step.qkv_fwd_metadata, step.qkv_bwd_metadata, step.attn_out_fwd_metadata, step.attn_out_bwd_metadata):
        assert md.fa2a_metadata[1].item() == md.my_rank_send_sz == md.fa2a_metadata[3].item()
        n = md.normalize("cpu")
        assert all(t.dtype == torch.uint64 for t in n.fa2a_metadata)
        assert all(t.dtype == torch.int64 for t in n.send_memcpy_metadata + n.recv_memcpy_metadata)
    fwd, grad = step.qkv_fwd_metadata, step.qkv_bwd_metadata
    assert fwd.seq_lens[1].send_seqlens.tolist() == [4, 2, 3, 6]                  # stored shards
    assert fwd.seq_lens[1].recv_seqlens.tolist() == [4, 4, 2, 4, 2, 3, 6]        # prefix entries per task
    assert fwd.send_memcpy_metadata[1].shape == (1, 4) and fwd.kv_replica_mask.shape == (4, 1)
    # every entry of a stored shard unpacks from the bytes its single copy was packed to
    sent = fwd.send_memcpy_metadata[1][0]
    for e, s_ in enumerate(p.kv_entry_shard.tolist()):
        assert fwd.recv_memcpy_metadata[1][e] == sent[s_]
    # gradients: the server sends entries (masked to main copies), the linear side receives stored shards
    assert grad.seq_lens[1].send_seqlens.tolist() == fwd.seq_lens[1].recv_seqlens.tolist()
    assert grad.kv_grad_send_dedup.main_copy_mask.tolist() == [1, 0, 1, 0, 0, 1, 1]
    dev = step.to_device("cpu")
    assert dev.cu_seqlens_q.dtype == torch.int32 and dev.bwd_packed_seq_params.cu_seqlens_kv.dtype == torch.int32


def test_alltoall_metadata_get_slice():
    two = metadata.AlltoAllMetadata(
        tuple(torch.arange(4).reshape(2, 2) + i for i in range(4)), (torch.arange(6).reshape(2, 3),), (torch.arange(6).reshape(2, 3) * 2,),
        [0, 10], [0, 20], [5, 6], (metadata.SeqLens(torch.ones(2, 3), torch.ones(2, 3) * 2),),
        (metadata.LogicalShape([torch.Size((3, 8)), torch.Size((4, 8))], [torch.Size((5, 8)), torch.Size((6, 8))]),))
    r1 = two.get_slice(1)
    assert r1.my_rank_send_offset == 10 and r1.my_rank_send_sz == 6
    assert r1.send_memcpy_metadata[0].tolist() == [3, 4, 5] and r1.recv_memcpy_metadata[0].tolist() == [6, 8, 10]
    assert r1.seq_lens[0].recv_seqlens.tolist() == [2, 2, 2] and r1.tensor_shape[0].recv_shape == torch.Size((6, 8))


def test_shared_kv_layout_keeps_one_copy_per_shard_and_documents_contiguous():
    """Tasks listed in any order; every task's prefix must be one run of store rows starting at its document."""
    from distca_amd.metadata import shared_kv_layout
    # documents A = shards (3, 5, 2), B = (4,), C = (6, 1); stored shard ids 0..5; tasks: (A,1) (C,0) (A,0) (B,0) (A,2) (C,1)
    tasks = [[0, 1], [4], [0], [3], [0, 1, 2], [4, 5]]
    tokens = {0: 3, 1: 5, 2: 2, 3: 4, 4: 6, 5: 1}
    entry_key = [s for t in tasks for s in t]
    entry_tokens = [tokens[s] for s in entry_key]
    lens = [sum(tokens[s] for s in t) for t in tasks]
    lay = shared_kv_layout(lens, entry_tokens, entry_key)
    assert lay.num_rows == sum(tokens.values())
    # order of first appearance of the documents: A, C, B; shards of a document in document order
    assert lay.store_tokens.tolist() == [3, 5, 2, 6, 1, 4]
    starts = dict(zip([0, 1, 2, 4, 5, 3], np.concatenate([[0], np.cumsum(lay.store_tokens.numpy())[:-1]]).tolist()))
    assert lay.kv_task_offsets.tolist() == [starts[t[0]] for t in tasks]
    assert [entry_key[e] for e in lay.entry_of_stored.tolist()] == [0, 1, 2, 4, 5, 3]
    assert all(entry_key.index(entry_key[e]) == e for e in lay.entry_of_stored.tolist())   # the first of its aliases
    # an empty task and zero-length entries are tolerated
    lay = shared_kv_layout([3, 0, 8], [3, 0, 3, 5], [0, 9, 0, 1])
    assert lay.store_tokens.tolist() == [3, 5] and lay.kv_task_offsets.tolist() == [0, 0, 0]
    # tasks that do not read nested prefixes (the second skips shard 1): no shared layout
    assert shared_kv_layout([8, 5], [3, 5, 3, 2], [0, 1, 0, 2]) is None
    # entries that do not add up to the task lengths
    assert shared_kv_layout([4], [3], [0]) is None


def test_a_step_without_nested_prefixes_says_that_it_keeps_a_copy_per_task(monkeypatch):
    """When the K/V shards of a step's tasks are not nested prefixes of one stored sequence per document, the one-copy
    layout does not exist: the step carries none (the ticks then take the reference's layout) and says so once."""
    p = metadata.single_rank_plan([[3, 5], [4]], 4, 2)
    step = metadata.single_rank_step_params(p)
    with warnings.catch_warnings():
        warnings.simplefilter("error")
        dev = step.to_device("cpu")          # nested prefixes: no warning, both layouts present
    assert dev.shared_kv_fwd is not None and dev.shared_kv_bwd is not None
    monkeypatch.setattr(metadata, "shared_kv_layout", lambda *a, **k: None)
    with pytest.warns(RuntimeWarning, match="one K/V copy per task"):
        dev = step.to_device("cpu")
    assert dev.shared_kv_fwd is None and dev.shared_kv_bwd is None
    with pytest.warns(RuntimeWarning, match="one K/V copy per task"):
        _, fwd, bwd, _ = metadata.server_metas(p, device="cpu")
    assert fwd.shared_kv is None and bwd.shared_kv is None
