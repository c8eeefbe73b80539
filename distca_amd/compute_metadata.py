"""From a shard plan to the all-to-all metadata of one layer step, for any number of ranks.

A plan is a list of documents, each a list of `ShardInfo` in document order: `rid` is the
rank that holds the shard's tokens for the linear layers, `dispatch_rid` the rank whose CA
server computes its attention.  The layouts produced here follow what the reference derives
in distca/runtime/compute_metadata.py:368-639 (`_from_planner_output`):

  * linear layout of rank r: its shards in (document, shard) order;
  * attention layout of rank a: its query shards in the same order, and for the query shard
    (doc, i) the K/V entries (doc, 0) .. (doc, i): one task per query shard with the document
    prefix as keys;
  * a K/V shard travels once per (linear rank, attention rank) pair however many entries need
    it there (the first entry is the main copy, the others alias its bytes), and the set of
    attention ranks that need it numbers its replicas in order of first need;
  * between a pair of ranks the buffer region holds the q shards, then the de-duplicated k
    shards, then the v shards; regions are laid out per peer by exclusive prefix sums on both
    sides (`get_fa2a_metadata`, :78-89);
  * the gradient direction is the forward direction reversed (`compute_reverse_a2a_layout_metadata`,
    runtime/metadata.py:239-279) plus the duplicate-gradient metadata of every attention rank.

Only the single-GPU part of this build runs the result: `simulate_fa2a` stands in for the
transport by copying the byte ranges the metadata names between per-rank buffers.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch
from torch import Tensor

from .fused_comm_attn import PackedSeqParams
from .metadata import (AlltoAllMetadata, DedupGradSumMetadata, LogicalShape, PingPangSingleStepPackedSeqParams, SeqLens,
                       get_attn_metadata)
from .utils import exclusive_cumsum, size_pad_by_int4


@dataclass
class ShardInfo:
    """One shard of a document (distca/runtime/shard_info.py:9-23)."""
    rid: int           # rank of the linear layers for these tokens
    dispatch_rid: int  # rank of the CA server for these tokens
    logical_sid: int   # position of the shard in its document
    shard_len: int


def get_per_token_bytes(hidden_size_q: int, hidden_size_kv: int, lse_size_in_hidden_dtype: int, element_size: int,
                        is_resend_qkv_in_bwd: bool, is_send_lse_in_fwd: bool) -> Tuple[int, int, int]:
    """(q token, k token, attention-output token) in bytes, q-side tokens padded to 16 bytes
    (compute_metadata.py:49-75): the backward request carries [dO | O | lse | q], the forward
    reply [out | lse]."""
    assert not (is_send_lse_in_fwd and is_resend_qkv_in_bwd)
    q_elems = hidden_size_q * 3 + lse_size_in_hidden_dtype if is_resend_qkv_in_bwd else hidden_size_q
    q_bytes = size_pad_by_int4(element_size * q_elems, 1)[0]
    k_bytes = element_size * hidden_size_kv
    assert k_bytes % 16 == 0, "K/V tokens must be a multiple of 16 bytes"
    out_elems = hidden_size_q + lse_size_in_hidden_dtype if is_send_lse_in_fwd else hidden_size_q
    out_bytes = size_pad_by_int4(element_size * out_elems, 1)[0]
    return q_bytes, k_bytes, out_bytes


def get_fa2a_metadata(send_bytes: Tensor):
    """send_bytes[i, j] = bytes rank i sends to rank j -> (sender_send_offset, sender_transfer_sz,
    sender_recv_offset, recver_transfer_sz), each [world, world]."""
    recver_transfer_sz = send_bytes.t().contiguous()
    return (exclusive_cumsum(send_bytes, dim=1), send_bytes, exclusive_cumsum(recver_transfer_sz, dim=1).t().contiguous(),
            recver_transfer_sz)


def reverse_a2a_metadata(fwd: AlltoAllMetadata) -> AlltoAllMetadata:
    """The way back: every byte returns to where it came from (stacked per-rank form)."""
    send_disp, send_sz, recv_disp, recv_sz = fwd.fa2a_metadata
    fa2a = (recv_disp.t().contiguous(), recv_sz, send_disp.t().contiguous(), send_sz)
    diag = lambda t: torch.diagonal(t).tolist()
    return AlltoAllMetadata(
        fa2a, fwd.recv_memcpy_metadata, fwd.send_memcpy_metadata, diag(fa2a[0]), diag(fa2a[2]), diag(fa2a[1]),
        tuple(SeqLens(s.recv_seqlens, s.send_seqlens) for s in fwd.seq_lens),
        tuple(LogicalShape(t.recv_shape, t.send_shape) for t in fwd.tensor_shape), kv_replica_mask=fwd.kv_replica_mask)


@dataclass
class _Layout:
    """Who holds what, derived once from the plan."""
    linear: List[List[Tuple[int, int]]]           # per rank: (doc, shard) in linear order
    attn_q: List[List[Tuple[int, int]]]           # per rank: query shards in attention order
    attn_k: List[List[Tuple[int, int]]]           # per rank: K/V entries in attention order
    attn_q_lens: List[List[int]]
    attn_kv_lens: List[List[int]]                 # per task: prefix length
    pos_linear: Dict[Tuple[int, int], int]        # (doc, shard) -> index on its linear rank
    q_pairs: List[List[List[Tuple[int, int]]]]    # [l][a] -> (index on l, index on a) of q shards
    k_pairs: List[List[List[Tuple[int, int, int, int]]]]  # [l][a] -> (index on l, entry on a, replica, main entry on a)
    num_dst: List[List[int]]                      # per linear rank, per shard: attention ranks that need its K/V


def _layout(world_size: int, plan: Sequence[Sequence[ShardInfo]]) -> _Layout:
    lay = _Layout([[] for _ in range(world_size)], [[] for _ in range(world_size)], [[] for _ in range(world_size)],
                  [[] for _ in range(world_size)], [[] for _ in range(world_size)], {},
                  [[[] for _ in range(world_size)] for _ in range(world_size)],
                  [[[] for _ in range(world_size)] for _ in range(world_size)], [])
    dsts: Dict[Tuple[int, int], List[int]] = {}
    first_entry: Dict[Tuple[int, int, int], int] = {}       # (doc, shard, attention rank) -> main entry on that rank
    for d, doc in enumerate(plan):
        context = 0
        for i, sh in enumerate(doc):
            assert sh.logical_sid == i, "shards of a document must be listed in order"
            l, a = sh.rid, sh.dispatch_rid
            lay.pos_linear[(d, i)] = len(lay.linear[l])
            lay.linear[l].append((d, i))
            lay.q_pairs[l][a].append((lay.pos_linear[(d, i)], len(lay.attn_q[a])))
            lay.attn_q[a].append((d, i))
            context += sh.shard_len
            lay.attn_q_lens[a].append(sh.shard_len)
            lay.attn_kv_lens[a].append(context)
            for j in range(i + 1):
                kl = doc[j].rid
                entry = len(lay.attn_k[a])
                lay.attn_k[a].append((d, j))
                need = dsts.setdefault((d, j), [])
                if a not in need:
                    need.append(a)
                main = first_entry.setdefault((d, j, a), entry)
                lay.k_pairs[kl][a].append((lay.pos_linear[(d, j)], entry, need.index(a), main))
    lay.num_dst = [[len(dsts.get(s, [])) for s in lay.linear[r]] for r in range(world_size)]
    return lay


def _dedup_metadata(entry_lens: Tensor, pairs_into_rank: Sequence[Sequence[Tuple[int, int, int, int]]]) -> DedupGradSumMetadata:
    n = entry_lens.shape[0]
    starts = exclusive_cumsum(entry_lens.to(torch.int64), dim=0).tolist() if n else []
    copies: List[List[int]] = [[] for _ in range(n)]
    main_mask = torch.zeros(n, dtype=torch.int8)
    for pair in pairs_into_rank:
        for _, entry, _, main in pair:
            if entry == main:
                main_mask[entry] = 1
            else:
                copies[main].append(starts[entry])
    width = max([len(c) for c in copies] + [1])
    copy_start = torch.zeros((n, width), dtype=torch.int64)
    for e, c in enumerate(copies):
        if c:
            copy_start[e, :len(c)] = torch.tensor(c, dtype=torch.int64)
    return DedupGradSumMetadata(torch.tensor([len(c) for c in copies], dtype=torch.int32), copy_start, main_mask)


def _assign(lay: _Layout, plan, fa2a, token_bytes: int, pair_lists, n_send, n_recv):
    """Offsets of plain (non-replicated) shards inside each pair's region, starting at the
    region's start: (send offsets per linear rank, receive offsets per attention rank)."""
    W = len(n_send)
    send = [torch.zeros(n, dtype=torch.int64) for n in n_send]
    recv = [torch.zeros(n, dtype=torch.int64) for n in n_recv]
    cursor = torch.zeros((W, W), dtype=torch.int64)
    for l in range(W):
        for a in range(W):
            used = 0
            for i, j in pair_lists[l][a]:
                send[l][i] = int(fa2a[0][l, a]) + used
                recv[a][j] = int(fa2a[2][l, a]) + used
                d, sid = lay.linear[l][i]
                used += plan[d][sid].shard_len * token_bytes
            cursor[l, a] = used
    return send, recv, cursor


def _from_planner_output(world_size: int, plan: Sequence[Sequence[ShardInfo]], q_bytes: int, k_bytes: int, element_size: int,
                         compute_attn_out_metadata: bool, attn_out_bytes: Optional[int]):
    """(qkv linear->attention, its reverse with the duplicate-gradient metadata, [attention output
    attention->linear, its gradient linear->attention,] attention cu_seqlens per rank), each
    stacked over ranks (compute_metadata.py:368-639)."""
    lay = _layout(world_size, plan)
    W = world_size
    length = lambda s: plan[s[0]][s[1]].shard_len
    lens = lambda shards: torch.tensor([length(s) for s in shards], dtype=torch.int64)
    n_lin = [len(x) for x in lay.linear]
    n_q = [len(x) for x in lay.attn_q]

    q_tokens = torch.zeros((W, W), dtype=torch.int64)
    k_tokens = torch.zeros((W, W), dtype=torch.int64)
    for l in range(W):
        for a in range(W):
            q_tokens[l, a] = sum(length(lay.linear[l][i]) for i, _ in lay.q_pairs[l][a])
            k_tokens[l, a] = sum(length(lay.linear[l][i]) for i, e, _, m in lay.k_pairs[l][a] if e == m)
    fa2a = get_fa2a_metadata(q_tokens * q_bytes + 2 * k_tokens * k_bytes)

    q_send, q_recv, cursor = _assign(lay, plan, fa2a, q_bytes, lay.q_pairs, n_lin, n_q)
    max_cp = max([max(nd + [1]) for nd in lay.num_dst] + [1])     # one replica count for all ranks, as stacked tensors need
    k_send = [torch.full((max_cp, n), -1, dtype=torch.int64) for n in n_lin]
    v_send = [t.clone() for t in k_send]
    mask = [torch.zeros((n, max_cp), dtype=torch.int8) for n in n_lin]
    k_recv = [torch.zeros(len(x), dtype=torch.int64) for x in lay.attn_k]
    v_recv = [t.clone() for t in k_recv]
    for l in range(W):
        for s, nd in enumerate(lay.num_dst[l]):
            mask[l][s, :nd] = 1
        for a in range(W):
            used = int(cursor[l, a])
            for send, recv in ((k_send, k_recv), (v_send, v_recv)):
                for i, e, rep, m in lay.k_pairs[l][a]:
                    if e != m:
                        continue
                    send[l][rep, i] = int(fa2a[0][l, a]) + used
                    recv[a][e] = int(fa2a[2][l, a]) + used
                    used += length(lay.linear[l][i]) * k_bytes
                for i, e, rep, m in lay.k_pairs[l][a]:
                    if e != m:
                        recv[a][e] = recv[a][m]          # a duplicate entry reads its main copy's bytes
            assert used == int(fa2a[1][l, a])

    lin_lens = [lens(x) for x in lay.linear]
    attn_q_lens = [lens(x) for x in lay.attn_q]
    attn_k_lens = [lens(x) for x in lay.attn_k]
    tok = lambda t: int(t.sum())
    q_hidden, k_hidden = q_bytes // element_size, k_bytes // element_size
    q_shape = LogicalShape([torch.Size((tok(lin_lens[r]), q_hidden)) for r in range(W)],
                           [torch.Size((tok(attn_q_lens[r]), q_hidden)) for r in range(W)])
    k_shape = LogicalShape([torch.Size((max_cp, tok(lin_lens[r]), k_hidden)) for r in range(W)],
                           [torch.Size((tok(attn_k_lens[r]), k_hidden)) for r in range(W)])
    diag = lambda t: torch.diagonal(t).tolist()
    qkv_fwd = AlltoAllMetadata(fa2a, (tuple(q_send), tuple(k_send), tuple(v_send)), (tuple(q_recv), tuple(k_recv), tuple(v_recv)),
                               diag(fa2a[0]), diag(fa2a[2]), diag(fa2a[1]),
                               (SeqLens(lin_lens, attn_q_lens), SeqLens(lin_lens, attn_k_lens)), (q_shape, k_shape),
                               kv_replica_mask=tuple(mask), max_cp_degree=max_cp)
    qkv_bwd = reverse_a2a_metadata(qkv_fwd)
    qkv_bwd.kv_grad_send_dedup = [_dedup_metadata(attn_k_lens[a], [lay.k_pairs[l][a] for l in range(W)]) for a in range(W)]

    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    attn = [dict(cu_seqlens_q=torch.zeros(1, dtype=torch.int32), cu_seqlens_kv=torch.zeros(1, dtype=torch.int32),
                 max_seqlen_q=0, max_seqlen_kv=0) if not lay.attn_q_lens[a] else
            get_attn_metadata(i32(lay.attn_q_lens[a]), i32(lay.attn_kv_lens[a])) for a in range(W)]
    if not compute_attn_out_metadata:
        return qkv_fwd, qkv_bwd, attn

    # attention output: built in the gradient direction (linear -> attention), the forward reply is its reverse
    out_fa2a = get_fa2a_metadata(q_tokens * attn_out_bytes)
    o_send, o_recv, _ = _assign(lay, plan, out_fa2a, attn_out_bytes, lay.q_pairs, n_lin, n_q)
    out_hidden = attn_out_bytes // element_size
    o_shape = LogicalShape([torch.Size((tok(lin_lens[r]), out_hidden)) for r in range(W)],
                           [torch.Size((tok(attn_q_lens[r]), out_hidden)) for r in range(W)])
    out_grad = AlltoAllMetadata(out_fa2a, (tuple(o_send),), (tuple(o_recv),), diag(out_fa2a[0]), diag(out_fa2a[2]), diag(out_fa2a[1]),
                                (SeqLens(lin_lens, attn_q_lens),), (o_shape,))
    return qkv_fwd, qkv_bwd, reverse_a2a_metadata(out_grad), out_grad, attn


def from_planner_output(world_size: int, scheduler_output: Sequence[Sequence[ShardInfo]], hidden_size_q: int, hidden_size_kv: int,
                        lse_size_in_hidden_dtype: int, element_size: int, is_pipeline_tick: bool, is_resend_qkv: bool = False):
    """(qkv linear->attention, qkv gradients attention->linear, attention output attention->linear,
    its gradient (or, with `is_resend_qkv`, the backward request [dO | O | lse | q] + k + v)
    linear->attention, attention cu_seqlens per rank); same flags as compute_metadata.py:642-692:
    a pipeline tick describes the forward only, and both flags make the reply carry the lse."""
    if is_resend_qkv:
        assert not is_pipeline_tick, "is_resend_qkv belongs to the non-pipelined step"
    q_bytes, k_bytes, out_bytes = get_per_token_bytes(hidden_size_q, hidden_size_kv, lse_size_in_hidden_dtype, element_size,
                                                      False, is_pipeline_tick or is_resend_qkv)
    qkv_fwd, qkv_grad, out_fwd, out_grad, attn = _from_planner_output(world_size, scheduler_output, q_bytes, k_bytes,
                                                                      element_size, True, out_bytes)
    if is_pipeline_tick:
        qkv_grad = out_grad = None
    if is_resend_qkv:
        out_grad, qkv_grad, _ = backward_from_planner_output(world_size, scheduler_output, hidden_size_q, hidden_size_kv,
                                                             lse_size_in_hidden_dtype, element_size)
    return qkv_fwd, qkv_grad, out_fwd, out_grad, attn


def backward_from_planner_output(world_size: int, scheduler_output_bwd: Sequence[Sequence[ShardInfo]], hidden_size_q: int,
                                 hidden_size_kv: int, lse_size_in_hidden_dtype: int, element_size: int):
    """(backward request linear->attention, qkv gradients attention->linear, attention cu_seqlens)
    (compute_metadata.py:695-734)."""
    q_bytes, k_bytes, _ = get_per_token_bytes(hidden_size_q, hidden_size_kv, lse_size_in_hidden_dtype, element_size, True, False)
    request, _, _ = _from_planner_output(world_size, scheduler_output_bwd, q_bytes, k_bytes, element_size, False, None)
    q_bytes, k_bytes, _ = get_per_token_bytes(hidden_size_q, hidden_size_kv, lse_size_in_hidden_dtype, element_size, False, False)
    _, qkv_grad, attn = _from_planner_output(world_size, scheduler_output_bwd, q_bytes, k_bytes, element_size, False, None)
    return request, qkv_grad, attn


def step_params(rank: int, fwd_out, device="cuda") -> PingPangSingleStepPackedSeqParams:
    """The layer-step parameters of one rank from `from_planner_output(..., is_resend_qkv=True)`."""
    qkv_fwd, qkv_grad, out_fwd, request, attn = fwd_out
    a = attn[rank]
    bwd = PackedSeqParams(cu_seqlens_q=a["cu_seqlens_q"], cu_seqlens_kv=a["cu_seqlens_kv"],
                          max_seqlen_q=a["max_seqlen_q"], max_seqlen_kv=a["max_seqlen_kv"])
    return PingPangSingleStepPackedSeqParams(
        "thd", a["cu_seqlens_q"], a["cu_seqlens_kv"], a["max_seqlen_q"], a["max_seqlen_kv"],
        qkv_fwd_metadata=qkv_fwd.get_slice(rank), qkv_bwd_metadata=qkv_grad.get_slice(rank),
        attn_out_fwd_metadata=out_fwd.get_slice(rank), attn_out_bwd_metadata=request.get_slice(rank),
        bwd_packed_seq_params=bwd).to_device(device)


def simulate_fa2a(send_buffers: Sequence[Tensor], recv_buffers: Sequence[Tensor], fa2a_metadata) -> None:
    """What the transport does, on one device: for every (source, destination) pair copy
    `sender_transfer_sz` bytes from the source's send buffer at `sender_send_offset` to the
    destination's receive buffer at `sender_recv_offset` (tests/test_fa2a_metadata.py:160-175 of
    the reference holds the same stand-in)."""
    send_disp, send_sz, recv_disp, _ = fa2a_metadata
    world = len(send_buffers)
    for src in range(world):
        for dst in range(world):
            n = int(send_sz[src, dst])
            if n:
                so, ro = int(send_disp[src, dst]), int(recv_disp[src, dst])
                recv_buffers[dst][ro:ro + n] = send_buffers[src][so:so + n]
