"""The metadata types and the single-rank plan against the hand-derived example of one
document cut into shards a | b | c (compute_metadata.py:404-459,202-273,277-323 of the
reference, world size 1): tasks Lq = [a, b, c], Lk = [a, a+b, a+b+c]; K/V entries
[k0 | k0 k1 | k0 k1 k2]; main copies are the first occurrences; duplicates are summed into them."""
import numpy as np
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
