"""Types that carry lengths, offsets and masks into the CA-server path, and a single-rank
plan builder.

`SeqLens`, `LogicalShape` and `DedupGradSumMetadata` have the fields and the dtype
normalisation of distca/runtime/metadata.py:12-67 (lengths and offsets int64, masks int8,
num_copies int32, cu_seqlens int32 as in runtime/megatron/packed_seq_params.py:11-14).
`get_attn_metadata` follows runtime/compute_metadata.py:326-365.

`single_rank_plan` lays out what one CA server holds for a list of documents cut into
shards when linear rank and attention rank are the same GPU: the task list (shard i of a
document attends to the document's first i+1 shards, compute_metadata.py:404-448), the
K/V shard entries with their main-copy mask and duplicate-gradient metadata (:202-219,
277-323), and contiguous byte offsets for the q | k | v regions of each buffer.  The
reference derives the same quantities for any number of ranks from planner output
(_from_planner_output, :368-639); distca_amd.compute_metadata does that.
"""
from __future__ import annotations

import warnings

from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple, Union

import torch
from torch import Tensor

from .utils import exclusive_cumsum, prepend_zero_fn, size_pad_by_int4

_TensorOrList = Union[Tensor, Sequence[Tensor]]


def _dev(t: Tensor, dtype: torch.dtype, device) -> Tensor:
    return t.to(device=device, dtype=dtype).contiguous()


@dataclass
class SeqLens:
    send_seqlens: _TensorOrList
    recv_seqlens: _TensorOrList

    def get_slice(self, rank):
        return SeqLens(self.send_seqlens[rank], self.recv_seqlens[rank])

    def normalize(self, device="cuda"):
        if isinstance(self.send_seqlens, Tensor):
            return SeqLens(_dev(self.send_seqlens, torch.int64, device), _dev(self.recv_seqlens, torch.int64, device))
        return SeqLens(tuple(_dev(t, torch.int64, device) for t in self.send_seqlens),
                       tuple(_dev(t, torch.int64, device) for t in self.recv_seqlens))


@dataclass
class LogicalShape:
    """Shapes used to allocate receive tensors; a KV send shape is (cp_degree, tokens, hidden)."""
    send_shape: Union[torch.Size, Sequence[torch.Size]]
    recv_shape: Union[torch.Size, Sequence[torch.Size]]

    def get_slice(self, rank):
        return LogicalShape(self.send_shape[rank], self.recv_shape[rank])


@dataclass
class DedupGradSumMetadata:
    """A KV shard used by several query shards of a rank has several copies there; one copy
    is sent forward, and the copies' gradients are summed into the main copy before one
    gradient is sent back."""
    num_copies: Tensor       # int32 [entries]
    copy_start_id: Tensor    # int64 [entries, max_copies], token index of each duplicate
    main_copy_mask: Tensor   # int8 [entries]

    def normalize(self, device="cuda"):
        return DedupGradSumMetadata(_dev(self.num_copies, torch.int32, device),
                                    _dev(self.copy_start_id, torch.int64, device),
                                    _dev(self.main_copy_mask, torch.int8, device))


def _slice_or_none(x, rank):
    return None if x is None else x[rank]


@dataclass
class AlltoAllMetadata:
    """Everything one all-to-all of the CA path needs (fields and meaning of
    distca/runtime/metadata.py:70-100): the transport's per-peer displacements and sizes
    (`fa2a_metadata`: sender_send_offset, sender_transfer_sz, sender_recv_offset,
    recver_transfer_sz, in bytes), the byte offset of every shard in the send buffer
    (`send_memcpy_metadata`, ordered by the sender's shards; for K/V as [cp, shard]) and in the
    receive buffer (`recv_memcpy_metadata`, ordered by the receiver's shards), the shard lengths
    and tensor shapes on either side, the K/V replica mask of the sender and, for the gradient
    direction, the duplicate-gradient metadata."""
    fa2a_metadata: Tuple[Tensor, Tensor, Tensor, Tensor]
    send_memcpy_metadata: Sequence[_TensorOrList]
    recv_memcpy_metadata: Sequence[_TensorOrList]
    my_rank_send_offset: Union[int, List[int]]
    my_rank_recv_offset: Union[int, List[int]]
    my_rank_send_sz: Union[int, List[int]]
    seq_lens: Sequence[SeqLens]
    tensor_shape: Sequence[LogicalShape]
    kv_replica_mask: Optional[_TensorOrList] = None
    kv_grad_send_dedup: Optional[Union[DedupGradSumMetadata, Sequence[DedupGradSumMetadata]]] = None
    single_stream: bool = False
    send_num_seqs: Optional[Sequence[int]] = None
    recv_num_seqs: Optional[Sequence[int]] = None
    max_cp_degree: Optional[int] = None

    def get_slice(self, rank):
        """The metadata of one rank out of the stacked per-rank form (metadata.py:177-198)."""
        return AlltoAllMetadata(
            tuple(t[rank] for t in self.fa2a_metadata),
            tuple(t[rank] for t in self.send_memcpy_metadata),
            tuple(t[rank] for t in self.recv_memcpy_metadata),
            self.my_rank_send_offset[rank], self.my_rank_recv_offset[rank], self.my_rank_send_sz[rank],
            tuple(sl.get_slice(rank) for sl in self.seq_lens),
            tuple(ts.get_slice(rank) for ts in self.tensor_shape),
            kv_replica_mask=_slice_or_none(self.kv_replica_mask, rank),
            kv_grad_send_dedup=_slice_or_none(self.kv_grad_send_dedup, rank),
            single_stream=self.single_stream)

    def normalize(self, device="cuda"):
        """To device with the dtypes the kernels read (metadata.py:200-220): transport
        displacements uint64, shard offsets int64, masks int8."""
        return AlltoAllMetadata(
            tuple(_dev(t, torch.uint64, device) for t in self.fa2a_metadata),
            tuple(_dev(t, torch.int64, device) for t in self.send_memcpy_metadata),
            tuple(_dev(t, torch.int64, device) for t in self.recv_memcpy_metadata),
            self.my_rank_send_offset, self.my_rank_recv_offset, self.my_rank_send_sz,
            tuple(t.normalize(device) for t in self.seq_lens), self.tensor_shape,
            kv_replica_mask=_dev(self.kv_replica_mask, torch.int8, device) if self.kv_replica_mask is not None else None,
            kv_grad_send_dedup=self.kv_grad_send_dedup.normalize(device) if self.kv_grad_send_dedup is not None else None,
            single_stream=self.single_stream, send_num_seqs=self.send_num_seqs, recv_num_seqs=self.recv_num_seqs,
            max_cp_degree=self.max_cp_degree)


def get_attn_metadata(seqlens_q, seqlens_kv=None, get_packed_seq_params: bool = False):
    """cu_seqlens / max_seqlen of a task list (one tensor) or of one list per rank."""
    from .fused_comm_attn import PackedSeqParams
    return_list = True
    if seqlens_kv is None:
        seqlens_kv = seqlens_q
    if isinstance(seqlens_q, Tensor):
        assert isinstance(seqlens_kv, Tensor)
        seqlens_q, seqlens_kv = [seqlens_q], [seqlens_kv]
        return_list = False
    assert len(seqlens_kv) == len(seqlens_q)
    world = []
    for sq, skv in zip(seqlens_q, seqlens_kv):
        assert sq.ndim == 1 and skv.shape == sq.shape
        out = dict(cu_seqlens_q=prepend_zero_fn(sq.cumsum(dim=0)), cu_seqlens_kv=prepend_zero_fn(skv.cumsum(dim=0)),
                   max_seqlen_q=sq.max().item(), max_seqlen_kv=skv.max().item())
        if get_packed_seq_params:
            out = PackedSeqParams(qkv_format="thd", **out)
        world.append(out)
    return world if return_list else world[0]


@dataclass
class SharedKVLayout:
    """One stored copy of every K/V shard the tasks of a tick read, the shards of a document side by side
    in document order, so that every task finds its whole prefix as one run of rows (kv_task_offsets) and
    nothing is copied once per task.  The reference materialises the prefix of every task
    (compute_metadata.py:429-448: one recv entry per (task, shard), aliased in the buffer) and sums the
    gradients of the copies afterwards (inplace_grad_sum_kernel); with this layout the attention kernels
    read the one copy and leave summed dK/dV in it."""
    store_tokens: Tensor      # int64 [stored shards]: tokens of each, in store order
    entry_of_stored: Tensor   # int64 [stored shards]: the K/V entry (first of its aliases) it is unpacked from
    kv_task_offsets: Tensor   # int32 [tasks]: first store row of each task's prefix
    num_rows: int


def _warn_no_shared_layout():
    """Said once per call site that drops the one-copy layout: the ticks then still give the same results, through the
    reference's layout (a copy of the prefix per task, the duplicate-gradient sum, a masked pack), at the cost of the
    duplicated K/V rows."""
    warnings.warn("the K/V shards of this step's tasks are not nested prefixes of one stored sequence per document: "
                  "the server ticks keep one K/V copy per task (unpack, duplicate-gradient sum, masked pack) instead of "
                  "reading one stored copy in place", RuntimeWarning, stacklevel=3)


def shared_kv_layout(task_kv_lens: Sequence[int], entry_tokens: Sequence[int], entry_key: Sequence[int]) -> Optional[SharedKVLayout]:
    """Host arrays in, host tensors out.  `entry_tokens[e]` / `entry_key[e]`: length and identity (any value equal
    for aliases of one stored shard and different otherwise: the shard's byte offset in the receive buffer will
    do) of the K/V entries, listed task by task; the entries of task t add up to task_kv_lens[t].  Returns None
    when the tasks of some document do not read nested prefixes of one shard sequence (then the per-task
    unpack has to be used)."""
    entry_tokens = [int(x) for x in entry_tokens]
    entry_key = [int(x) for x in entry_key]
    tasks: List[List[int]] = []
    e = 0
    for lk in task_kv_lens:
        lk, got, mine = int(lk), 0, []
        while got < lk:
            if e >= len(entry_tokens):
                return None
            if entry_tokens[e] > 0:
                mine.append(e)
            got += entry_tokens[e]
            e += 1
        if got != lk:
            return None
        tasks.append(mine)
    # a document = the tasks whose first entry is the same stored shard; its shard sequence = its longest task's
    docs: dict = {}
    order: List[int] = []
    for t, mine in enumerate(tasks):
        if not mine:
            continue
        head = entry_key[mine[0]]
        if head not in docs:
            docs[head] = mine
            order.append(head)
        elif len(mine) > len(docs[head]):
            docs[head] = mine
    for mine in tasks:
        if mine:
            ref = docs[entry_key[mine[0]]]
            if [entry_key[x] for x in mine] != [entry_key[x] for x in ref[:len(mine)]]:
                return None
    first_entry: dict = {}
    for idx, key in enumerate(entry_key):
        if entry_tokens[idx] > 0:
            first_entry.setdefault(key, idx)
    store_tokens, entry_of_stored, doc_start, row = [], [], {}, 0
    seen = set()
    for head in order:
        doc_start[head] = row
        for x in docs[head]:
            key = entry_key[x]
            if key in seen:
                return None   # one shard in two documents' sequences: not a prefix structure
            seen.add(key)
            store_tokens.append(entry_tokens[x])
            entry_of_stored.append(first_entry[key])
            row += entry_tokens[x]
    offs = [doc_start[entry_key[mine[0]]] if mine else 0 for mine in tasks]
    return SharedKVLayout(torch.tensor(store_tokens, dtype=torch.int64), torch.tensor(entry_of_stored, dtype=torch.int64),
                          torch.tensor(offs, dtype=torch.int32), row)


@dataclass
class SingleRankPlan:
    """Everything one CA-server tick needs for `docs` (host tensors; `.to(device)` variants
    are built by server_metas)."""
    q_seqlens: Tensor            # int64 [tasks]  Lq of each task = its shard length
    kv_seqlens: Tensor           # int64 [tasks]  Lk = document tokens up to the end of the shard
    kv_entry_tokens: Tensor      # int64 [entries] K/V shard entries in task order (prefix shards per task)
    kv_entry_shard: Tensor       # int64 [entries] index of the stored shard each entry reads
    dedup: DedupGradSumMetadata
    num_heads_q: int
    num_heads_kv: int
    head_dim: int
    itemsize: int

    @property
    def num_q_tokens(self) -> int:
        return int(self.q_seqlens.sum())

    @property
    def num_kv_tokens(self) -> int:
        return int(self.kv_entry_tokens.sum())

    # -- token sizes in bytes -------------------------------------------------------------
    @property
    def q_bytes(self) -> int:
        return self.num_heads_q * self.head_dim * self.itemsize

    @property
    def k_bytes(self) -> int:
        return self.num_heads_kv * self.head_dim * self.itemsize

    @property
    def out_lse_bytes(self) -> int:
        """[out | lse fp32 per head | pad to 16] (attn_kernels/dispatch.py:209-221)."""
        return size_pad_by_int4(self.q_bytes + self.num_heads_q * 4, 1)[0]

    @property
    def merged_q_bytes(self) -> int:
        """[dO | O | lse | q | pad to 16] (attn_kernels/dispatch.py:138-158)."""
        return size_pad_by_int4(3 * self.q_bytes + self.num_heads_q * 4, 1)[0]

    def _regions(self, q_token_bytes: int) -> Tuple[Tensor, Tensor, Tensor, int]:
        """Contiguous q | k | v regions, shards in order: (q offsets per task, k and v offsets per
        stored shard, total bytes)."""
        stored = self.stored_shard_tokens
        q_off = exclusive_cumsum(self.q_seqlens * q_token_bytes)
        base = int((self.q_seqlens * q_token_bytes).sum())
        ksz = stored * self.k_bytes
        k_off = base + exclusive_cumsum(ksz)
        v_off = k_off + int(ksz.sum())
        return q_off, k_off, v_off, base + 2 * int(ksz.sum())

    @property
    def stored_shard_tokens(self) -> Tensor:
        """Tokens of each distinct K/V shard; equals q_seqlens because every shard is both a query
        shard and a K/V shard of its document."""
        return self.q_seqlens

    def request_layout(self, backward: bool):
        """(q offsets [tasks], k offsets [entries], v offsets [entries], bytes) of the receive
        buffer; entries of one stored shard alias its single copy."""
        q_off, k_off, v_off, total = self._regions(self.merged_q_bytes if backward else self.q_bytes)
        return q_off, k_off[self.kv_entry_shard], v_off[self.kv_entry_shard], total

    def reply_layout(self, backward: bool):
        """Send buffer: forward [out|lse] per task; backward dq per task and dk, dv per stored
        shard (entries that are not main copies keep their main's offset and are masked out)."""
        if not backward:
            off = exclusive_cumsum(self.q_seqlens * self.out_lse_bytes)
            return off, None, None, int((self.q_seqlens * self.out_lse_bytes).sum())
        q_off, k_off, v_off, total = self._regions(self.q_bytes)
        return q_off, k_off[self.kv_entry_shard], v_off[self.kv_entry_shard], total


def single_rank_plan(docs: Sequence[Sequence[int]], num_heads_q: int, num_heads_kv: int, head_dim: int = 128,
                     itemsize: int = 2) -> SingleRankPlan:
    """`docs[d]` = shard lengths tiling document d in order.  One task per shard."""
    q_lens: List[int] = []
    kv_lens: List[int] = []
    entry_tokens: List[int] = []
    entry_shard: List[int] = []
    shard_base = 0
    for doc in docs:
        context = 0
        for i, n in enumerate(doc):
            if n <= 0:
                raise ValueError("shard lengths must be positive")
            context += n
            q_lens.append(n)
            kv_lens.append(context)
            for j in range(i + 1):
                entry_tokens.append(doc[j])
                entry_shard.append(shard_base + j)
        shard_base += len(doc)
    entry_tokens_t = torch.tensor(entry_tokens, dtype=torch.int64)
    entry_shard_t = torch.tensor(entry_shard, dtype=torch.int64)
    starts = exclusive_cumsum(entry_tokens_t).tolist() if entry_tokens else []
    first = {}
    copies: List[List[int]] = [[] for _ in entry_tokens]
    main_mask = [0] * len(entry_tokens)
    for e, s in enumerate(entry_shard):
        if s not in first:
            first[s] = e
            main_mask[e] = 1
        else:
            copies[first[s]].append(starts[e])
    max_copies = max([len(c) for c in copies] + [1])
    copy_start = torch.zeros((len(entry_tokens), max_copies), dtype=torch.int64)
    for e, c in enumerate(copies):
        if c:
            copy_start[e, :len(c)] = torch.tensor(c, dtype=torch.int64)
    dedup = DedupGradSumMetadata(torch.tensor([len(c) for c in copies], dtype=torch.int32), copy_start,
                                 torch.tensor(main_mask, dtype=torch.int8))
    return SingleRankPlan(torch.tensor(q_lens, dtype=torch.int64), torch.tensor(kv_lens, dtype=torch.int64),
                          entry_tokens_t, entry_shard_t, dedup, num_heads_q, num_heads_kv, head_dim, itemsize)


def server_metas(plan: SingleRankPlan, device="cuda", shared_kv: bool = True):
    """(PackedSeqParams, ServerFwdMeta, ServerBwdMeta, buffer sizes) on `device` for one tick:
    sizes = (fwd receive, fwd send, bwd receive, bwd send) bytes.  With `shared_kv` the metas also carry the
    layout that keeps one copy of every K/V shard (SharedKVLayout), which the in-place ticks use."""
    from .fused_comm_attn import ServerBwdMeta, ServerFwdMeta, SharedKVOnDevice
    i64 = lambda t: _dev(t, torch.int64, device)
    attn = get_attn_metadata(plan.q_seqlens, plan.kv_seqlens, get_packed_seq_params=True)
    attn.cu_seqlens_q = _dev(attn.cu_seqlens_q, torch.int32, device)
    attn.cu_seqlens_kv = _dev(attn.cu_seqlens_kv, torch.int32, device)
    hq_d = plan.num_heads_q * plan.head_dim
    hkv_d = plan.num_heads_kv * plan.head_dim
    tq, tk = plan.num_q_tokens, plan.num_kv_tokens
    fq, fk, fv, f_recv = plan.request_layout(False)
    fo, _, _, f_send = plan.reply_layout(False)
    fwd = ServerFwdMeta(i64(plan.q_seqlens), i64(plan.kv_entry_tokens), i64(fq), i64(fk), i64(fv),
                        i64(plan.q_seqlens), i64(fo), (tq, hq_d), (tk, hkv_d))
    shared = shared_kv_layout(plan.kv_seqlens.tolist(), plan.kv_entry_tokens.tolist(), plan.kv_entry_shard.tolist()) if shared_kv else None
    if shared_kv and shared is None:
        _warn_no_shared_layout()
    if shared is not None:
        fwd.shared_kv = SharedKVOnDevice.build(shared, fk, fv, device)
    bq, bk, bv, b_recv = plan.request_layout(True)
    gq, gk, gv, b_send = plan.reply_layout(True)
    d = plan.dedup.normalize(device)
    bwd = ServerBwdMeta(i64(plan.q_seqlens), i64(plan.kv_entry_tokens), i64(bq), i64(bk), i64(bv),
                        i64(plan.q_seqlens), i64(plan.kv_entry_tokens), i64(gq), i64(gk), i64(gv),
                        d.main_copy_mask, d.num_copies, d.copy_start_id, (tq, hq_d), (tq, plan.num_heads_q), (tk, hkv_d))
    if shared is not None:
        bwd.shared_kv = SharedKVOnDevice.build(shared, bk, bv, device, gk, gv)
    return attn, fwd, bwd, (f_recv, f_send, b_recv, b_send)


@dataclass
class PingPangSingleStepPackedSeqParams:
    """What one layer step carries into the CA path (runtime/megatron/packed_seq_params.py:26-57):
    the attention-layout cu_seqlens plus the four all-to-all descriptions (q/k/v out and gradients
    back, attention output out and its gradient back) and the backward's own cu_seqlens."""
    qkv_format: str = "thd"
    cu_seqlens_q: Tensor = None
    cu_seqlens_kv: Tensor = None
    max_seqlen_q: int = None
    max_seqlen_kv: int = None
    qkv_fwd_metadata: AlltoAllMetadata = None
    qkv_bwd_metadata: AlltoAllMetadata = None
    attn_out_fwd_metadata: AlltoAllMetadata = None
    attn_out_bwd_metadata: AlltoAllMetadata = None
    bwd_packed_seq_params: object = None
    stream: object = None
    dispatcher_id: int = None
    kv_task_offsets: Optional[Tensor] = None
    # set by to_device(): the one-copy K/V layouts of the forward and backward ticks (fused_comm_attn.SharedKVOnDevice),
    # None when the tasks do not read nested prefixes
    shared_kv_fwd: object = None
    shared_kv_bwd: object = None

    def _shared_kv(self, device):
        """The SharedKVLayout of this step's tasks, from the host copies of the metadata: the K/V entries of the
        receive side are listed task by task, aliases of a shard share their byte offset."""
        from .fused_comm_attn import SharedKVOnDevice
        host = lambda t: t.detach().cpu().to(torch.int64)
        out = []
        for req, grad, cu in ((self.qkv_fwd_metadata, None, self.cu_seqlens_kv),
                              (self.attn_out_bwd_metadata, self.qkv_bwd_metadata,
                               self.bwd_packed_seq_params.cu_seqlens_kv if self.bwd_packed_seq_params is not None else None)):
            if req is None or cu is None or len(req.recv_memcpy_metadata) < 3:
                out.append(None)
                continue
            k_off, v_off = host(req.recv_memcpy_metadata[1]), host(req.recv_memcpy_metadata[2])
            if k_off.dim() != 1:
                out.append(None)
                continue
            lens = host(cu).diff().tolist()
            layout = shared_kv_layout(lens, host(req.seq_lens[1].recv_seqlens).tolist(), k_off.tolist())
            if layout is None:
                _warn_no_shared_layout()
                out.append(None)
                continue
            gk = gv = None
            if grad is not None:
                gk, gv = host(grad.send_memcpy_metadata[1]), host(grad.send_memcpy_metadata[2])
            out.append(SharedKVOnDevice.build(layout, k_off, v_off, device, gk, gv))
        return out

    def to_device(self, device="cuda"):
        to_i32 = lambda t: None if t is None else _dev(t, torch.int32, device)
        to_int = lambda x: None if x is None else int(x)
        bwd = self.bwd_packed_seq_params
        if bwd is not None:
            bwd = type(bwd)(cu_seqlens_q=to_i32(bwd.cu_seqlens_q), cu_seqlens_kv=to_i32(bwd.cu_seqlens_kv),
                            max_seqlen_q=to_int(bwd.max_seqlen_q), max_seqlen_kv=to_int(bwd.max_seqlen_kv))
        shared_fwd, shared_bwd = self._shared_kv(device)
        return PingPangSingleStepPackedSeqParams(
            self.qkv_format, to_i32(self.cu_seqlens_q), to_i32(self.cu_seqlens_kv), to_int(self.max_seqlen_q),
            to_int(self.max_seqlen_kv), self.qkv_fwd_metadata.normalize(device), self.qkv_bwd_metadata.normalize(device),
            self.attn_out_fwd_metadata.normalize(device), self.attn_out_bwd_metadata.normalize(device), bwd, self.stream,
            self.dispatcher_id, to_i32(self.kv_task_offsets), shared_fwd, shared_bwd)


def single_rank_step_params(plan: SingleRankPlan) -> PingPangSingleStepPackedSeqParams:
    """The four AlltoAllMetadata of one layer step when the linear rank and the attention rank are
    the same GPU (world size 1: the transport moves `my_rank_send_sz` bytes from the send buffer's
    offset 0 to the receive buffer's offset 0).  Host tensors; call to_device() before use."""
    from .fused_comm_attn import PackedSeqParams
    t64 = lambda x: torch.tensor([[x]], dtype=torch.int64)
    tq, tkv = plan.num_q_tokens, plan.num_kv_tokens
    stored = plan.stored_shard_tokens
    hq_d, hkv_d = plan.num_heads_q * plan.head_dim, plan.num_heads_kv * plan.head_dim
    first = torch.tensor([plan.kv_entry_shard.tolist().index(s) for s in range(len(stored))], dtype=torch.int64)

    def qkv_md(backward_request: bool):
        q_off, k_off, v_off, total = plan.request_layout(backward_request)
        qb = plan.merged_q_bytes if backward_request else plan.q_bytes * 1
        send = (q_off, k_off[first].unsqueeze(0), v_off[first].unsqueeze(0))      # K/V as [cp = 1, shard]
        recv = (q_off, k_off, v_off)
        seq = (SeqLens(plan.q_seqlens, plan.q_seqlens), SeqLens(stored, plan.kv_entry_tokens))
        q_cols = qb // plan.itemsize
        shape = (LogicalShape(torch.Size((tq, q_cols)), torch.Size((tq, q_cols))),
                 LogicalShape(torch.Size((1, int(stored.sum()), hkv_d)), torch.Size((tkv, hkv_d))))
        return AlltoAllMetadata((t64(0), t64(total), t64(0), t64(total)), send, recv, 0, 0, total, seq, shape,
                                kv_replica_mask=torch.ones((len(stored), 1), dtype=torch.int8))

    def grad_md():
        q_off, k_off, v_off, total = plan.reply_layout(True)
        send = (q_off, k_off, v_off)                                               # ordered by the server's entries
        recv = (q_off, k_off[first].unsqueeze(0), v_off[first].unsqueeze(0))
        seq = (SeqLens(plan.q_seqlens, plan.q_seqlens), SeqLens(plan.kv_entry_tokens, stored))
        shape = (LogicalShape(torch.Size((tq, hq_d)), torch.Size((tq, hq_d))),
                 LogicalShape(torch.Size((tkv, hkv_d)), torch.Size((1, int(stored.sum()), hkv_d))))
        return AlltoAllMetadata((t64(0), t64(total), t64(0), t64(total)), send, recv, 0, 0, total, seq, shape,
                                kv_replica_mask=torch.ones((len(stored), 1), dtype=torch.int8), kv_grad_send_dedup=plan.dedup)

    def out_md():
        off, _, _, total = plan.reply_layout(False)
        seq = (SeqLens(plan.q_seqlens, plan.q_seqlens),)
        cols = plan.out_lse_bytes // plan.itemsize
        shape = (LogicalShape(torch.Size((tq, cols)), torch.Size((tq, cols))),)
        return AlltoAllMetadata((t64(0), t64(total), t64(0), t64(total)), (off,), (off,), 0, 0, total, seq, shape)

    attn = get_attn_metadata(plan.q_seqlens, plan.kv_seqlens)
    bwd = PackedSeqParams(cu_seqlens_q=attn["cu_seqlens_q"], cu_seqlens_kv=attn["cu_seqlens_kv"],
                          max_seqlen_q=attn["max_seqlen_q"], max_seqlen_kv=attn["max_seqlen_kv"])
    return PingPangSingleStepPackedSeqParams(
        "thd", attn["cu_seqlens_q"], attn["cu_seqlens_kv"], attn["max_seqlen_q"], attn["max_seqlen_kv"],
        qkv_fwd_metadata=qkv_md(False), qkv_bwd_metadata=grad_md(), attn_out_fwd_metadata=out_md(),
        attn_out_bwd_metadata=qkv_md(True), bwd_packed_seq_params=bwd)
