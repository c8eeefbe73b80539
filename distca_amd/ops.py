"""Shard pack / unpack / duplicate-gradient ops of the CA server.

Same names, argument order and error behaviour as the reference's Python wrappers
(distca/runtime/attn_kernels/ops.py:153-215), bound to the HIP kernels through the C ABI
instead of torch.ops.dispatch_kernels.  The transport buffer is either an explicit device
tensor (the reference's `buffer=` form, csrc/bindings/all_to_all.cpp:102-113,243-254) or, as
in the reference's normal mode, the send / receive buffer of the `DispatcherWrapper` instance
`instance_id` names.  The transport between ranks is not part of this package: the
dispatcher's buffers are ordinary device memory and `fast_a2a` covers a world of one rank.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from . import _lib

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _check_tensor(ndim: int, x: torch.Tensor, name: str) -> None:
    # mirrors _CHECK_TENSOR, csrc/bindings/all_to_all.cpp:18-21
    if x.dim() != ndim:
        raise RuntimeError(f"tensor {name} must have {ndim} dimensions")
    if not x.is_cuda:
        raise RuntimeError(f"tensor {name} must be on CUDA")
    if not x.is_contiguous():
        raise RuntimeError(f"tensor {name} must be contiguous")


def _check_dtype(x: torch.Tensor, dtype: torch.dtype, name: str) -> None:
    # the reference reads metadata through const_data_ptr<T>(), which throws on a mismatch
    if x.dtype != dtype:
        raise RuntimeError(f"expected scalar type {dtype} but found {x.dtype} for {name}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class DispatcherWrapper:
    """Who owns the transport buffers (distca/runtime/attn_kernels/ops.py:67-150).  Two instances,
    for the two halves of a ping-pong step; each holds a send and a receive buffer of
    `buffer_size` bytes.  `acquire` / `release` keep the reference's bookkeeping (a receive buffer
    is acquired by the all-to-all that fills it and released by the op that has unpacked it, and
    the memcpy ops check that order) without the cross-rank signal behind it."""
    instance: Optional[List["DispatcherWrapper"]] = None
    is_acquired: List[bool] = [False, False]
    cur_instance: int = 0

    def __init__(self, buffer_size: int, device):
        self.buffer_size = int(buffer_size)
        self.device = torch.device(device)
        self.send_buffer = torch.zeros(self.buffer_size, dtype=torch.uint8, device=self.device)
        self.recv_buffer = torch.zeros(self.buffer_size, dtype=torch.uint8, device=self.device)

    @staticmethod
    def init(rank: int = 0, local_rank: int = 0, world_size: int = 1, buffer_size: int = 0, uid=None, device="cuda"):
        if world_size != 1:
            raise NotImplementedError("the transport between ranks is not part of this package: world_size must be 1")
        DispatcherWrapper.instance = [DispatcherWrapper(buffer_size, device) for _ in range(2)]
        DispatcherWrapper.is_acquired = [False, False]
        DispatcherWrapper.cur_instance = 0

    @staticmethod
    def get_instance(instance_id: Optional[int] = None) -> "DispatcherWrapper":
        if DispatcherWrapper.instance is None:
            raise AssertionError("DispatcherWrapper not initialized")
        return DispatcherWrapper.instance[DispatcherWrapper.cur_instance if instance_id is None else instance_id]

    @staticmethod
    def switch_buffer():
        DispatcherWrapper.cur_instance = (DispatcherWrapper.cur_instance + 1) % 2

    @staticmethod
    def update_buffer_size(buffer_size: int):
        """Grow both instances to `buffer_size` bytes; contents are not kept."""
        torch.cuda.synchronize()
        for i, inst in enumerate(DispatcherWrapper.instance):
            assert not DispatcherWrapper.is_acquired[i]
            if inst.buffer_size < buffer_size:
                DispatcherWrapper.instance[i] = DispatcherWrapper(buffer_size, inst.device)

    @staticmethod
    def acquire(instance_id: int):
        assert not DispatcherWrapper.is_acquired[instance_id]
        DispatcherWrapper.is_acquired[instance_id] = True

    @staticmethod
    def release(instance_id: int):
        assert DispatcherWrapper.is_acquired[instance_id]
        DispatcherWrapper.is_acquired[instance_id] = False


def _transport_buffer(buffer: Optional[torch.Tensor], instance_id: Optional[int], to_nvshmem: bool) -> torch.Tensor:
    """The explicit buffer, or the dispatcher's (ops.py:160-181 of the reference: with an instance
    id, packing needs the instance released and unpacking needs it acquired)."""
    if buffer is not None:
        return buffer
    if instance_id is not None:
        if to_nvshmem:
            assert not DispatcherWrapper.is_acquired[instance_id], "pack into a dispatcher whose receive buffer is not released"
        else:
            assert DispatcherWrapper.is_acquired[instance_id], "unpack from a dispatcher no all-to-all has filled"
    inst = DispatcherWrapper.get_instance(instance_id)
    return inst.send_buffer if to_nvshmem else inst.recv_buffer


def fast_a2a(sender_send_disp: torch.Tensor, sender_transfer_sz: torch.Tensor, sender_recv_disp: torch.Tensor,
             recver_transfer_sz: torch.Tensor, my_rank_send_offset: int, my_rank_recv_offset: int, my_rank_send_sz: int,
             instance_id: Optional[int] = None):
    """The all-to-all of a world of one rank (ops.py:217-262 of the reference): what a rank sends to
    itself goes from the send buffer to the receive buffer as one device copy, and the receive buffer
    counts as acquired from then on.  More ranks need a transport, which this package does not hold."""
    if sender_send_disp.numel() != 1:
        raise NotImplementedError("fast_a2a: the transport between ranks is not part of this package")
    if instance_id is not None:
        DispatcherWrapper.acquire(instance_id)
    inst = DispatcherWrapper.get_instance(instance_id)
    n = int(my_rank_send_sz)
    if my_rank_send_offset + n > inst.buffer_size or my_rank_recv_offset + n > inst.buffer_size:
        raise RuntimeError(f"fast_a2a: {n} bytes do not fit the dispatcher's buffers of {inst.buffer_size} bytes")
    inst.recv_buffer[my_rank_recv_offset:my_rank_recv_offset + n].copy_(inst.send_buffer[my_rank_send_offset:my_rank_send_offset + n])


def a2a_memcpy_non_cp(
    tensor: torch.Tensor, nvshmem_offset: torch.Tensor,
    shard_tokens: torch.Tensor, to_nvshmem: bool,
    shard_do_copy_mask: Optional[torch.Tensor] = None,
    buffer: Optional[torch.Tensor] = None, instance_id: Optional[int] = None,
):
    """Pack (`to_nvshmem=True`) rows of `tensor` [T, hidden] into `buffer`, or unpack them.

    Shard s covers rows excl_cumsum(shard_tokens)[s].. and buffer bytes nvshmem_offset[s]..
    `shard_do_copy_mask` (int8, packing only) skips shards whose entry is 0.
    """
    if shard_do_copy_mask is not None and buffer is None:
        assert to_nvshmem
    buffer = _transport_buffer(buffer, instance_id, to_nvshmem)
    _check_tensor(2, tensor, "tensor")
    _check_tensor(1, nvshmem_offset, "seq_nvshmem_offset")
    _check_dtype(nvshmem_offset, torch.int64, "seq_nvshmem_offset")
    _check_dtype(shard_tokens, torch.int64, "seq_tokens")
    num_seq = nvshmem_offset.size(0)
    mask_ptr = None
    if shard_do_copy_mask is not None:
        _check_tensor(1, shard_do_copy_mask, "copy_seq_mask")
        if shard_do_copy_mask.size(0) != num_seq:
            raise RuntimeError("copy_seq_mask must be of shape (num_sequence,)")
        _check_dtype(shard_do_copy_mask, torch.int8, "copy_seq_mask")
        mask_ptr = shard_do_copy_mask.data_ptr()
    if not buffer.is_cuda:
        raise RuntimeError("tensor buffer must be on CUDA")
    token_bytes = tensor.size(1) * tensor.element_size()
    with torch.cuda.device(tensor.device):
        rc = _lib.load().distca_memcpy_non_cp(
            tensor.data_ptr(), buffer.data_ptr(), nvshmem_offset.data_ptr(), shard_tokens.data_ptr(),
            mask_ptr, num_seq, token_bytes, tensor.size(0), 1 if to_nvshmem else 0, _stream())
    _lib.check(rc, "a2a_memcpy_non_cp")
    return None


def a2a_memcpy_non_cp_multi(tensors, nvshmem_offsets, shard_tokens, to_nvshmem: bool, shard_do_copy_masks=None, *,
                            buffer: Optional[torch.Tensor] = None, instance_id: Optional[int] = None):
    """Several a2a_memcpy_non_cp calls against one buffer as a single launch: tensors[i] with nvshmem_offsets[i],
    shard_tokens[i] and (packing only) shard_do_copy_masks[i].  What the reference does with consecutive calls for
    the q, k and v of a tick (distca/runtime/attn_kernels/dispatch.py:39-56,60-94); the result is the same bytes."""
    n = len(tensors)
    if not (len(nvshmem_offsets) == len(shard_tokens) == n) or (shard_do_copy_masks is not None and len(shard_do_copy_masks) != n):
        raise RuntimeError("a2a_memcpy_non_cp_multi: one offset tensor, one length tensor and at most one mask per tensor")
    if n > _lib.PACK_MAX_JOBS:
        raise RuntimeError(f"a2a_memcpy_non_cp_multi: at most {_lib.PACK_MAX_JOBS} tensors per launch")
    if n == 0:
        return None
    buffer = _transport_buffer(buffer, instance_id, to_nvshmem)
    if not buffer.is_cuda:
        raise RuntimeError("tensor buffer must be on CUDA")
    jobs = (_lib.PackJob * n)()
    for i in range(n):
        t, off, tok = tensors[i], nvshmem_offsets[i], shard_tokens[i]
        _check_tensor(2, t, "tensor")
        _check_tensor(1, off, "seq_nvshmem_offset")
        _check_tensor(1, tok, "seq_tokens")
        _check_dtype(off, torch.int64, "seq_nvshmem_offset")
        _check_dtype(tok, torch.int64, "seq_tokens")
        if tok.size(0) != off.size(0):
            raise RuntimeError("seq_tokens must be of shape (num_sequence,)")
        mask = shard_do_copy_masks[i] if shard_do_copy_masks is not None else None
        if mask is not None:
            _check_tensor(1, mask, "copy_seq_mask")
            _check_dtype(mask, torch.int8, "copy_seq_mask")
            if mask.size(0) != off.size(0):
                raise RuntimeError("copy_seq_mask must be of shape (num_sequence,)")
        jobs[i] = _lib.PackJob(t.data_ptr(), off.data_ptr(), tok.data_ptr(), mask.data_ptr() if mask is not None else None,
                               off.size(0), t.size(1) * t.element_size(), t.size(0))
    with torch.cuda.device(buffer.device):
        rc = _lib.load().distca_memcpy_non_cp_multi(jobs, n, buffer.data_ptr(), 1 if to_nvshmem else 0, _stream())
    _lib.check(rc, "a2a_memcpy_non_cp_multi")
    return None


def a2a_memcpy_cp(
    tensor: torch.Tensor, do_shard: torch.Tensor,
    nvshmem_offset: torch.Tensor, shard_tokens: torch.Tensor,
    to_nvshmem: bool, buffer: Optional[torch.Tensor] = None,
    instance_id: Optional[int] = None,
):
    """Replicating pack of `tensor` [T, hidden] to every live (shard, replica) slot of
    `buffer`, or unpack into `tensor` [max_cp, T, hidden] (which the caller pre-zeroes)."""
    buffer = _transport_buffer(buffer, instance_id, to_nvshmem)
    _check_tensor(2 if to_nvshmem else 3, tensor, "tensor")
    if nvshmem_offset.dim() != 2:
        raise RuntimeError("tensor seq_nvshmem_offset must have 2 dimensions")
    num_seq = nvshmem_offset.size(1)
    cp_degree = nvshmem_offset.size(0)
    _check_tensor(1, shard_tokens, "seq_tokens")
    if shard_tokens.size(0) != num_seq:
        raise RuntimeError("seq_tokens must be of dimension (num_sequence)")
    _check_tensor(2, do_shard, "do_shard")
    if do_shard.size(0) != num_seq or do_shard.size(1) != cp_degree:
        raise RuntimeError("do_shard must be of dimension (num_sequence, cp_degree)")
    _check_dtype(do_shard, torch.int8, "do_shard")
    _check_dtype(nvshmem_offset, torch.int64, "seq_nvshmem_offset")
    _check_dtype(shard_tokens, torch.int64, "seq_tokens")
    if not nvshmem_offset.is_contiguous():
        raise RuntimeError("tensor seq_nvshmem_offset must be contiguous")
    hidden_dim = 1 if to_nvshmem else 2
    token_bytes = tensor.size(hidden_dim) * tensor.element_size()
    num_tokens = tensor.size(0) if to_nvshmem else tensor.size(1)
    with torch.cuda.device(tensor.device):
        rc = _lib.load().distca_memcpy_cp(
            tensor.data_ptr(), buffer.data_ptr(), do_shard.data_ptr(), nvshmem_offset.data_ptr(),
            shard_tokens.data_ptr(), token_bytes, num_tokens, cp_degree, num_seq,
            1 if to_nvshmem else 0, _stream())
    _lib.check(rc, "a2a_memcpy_cp")
    return None


def pre_a2a_grad_acc(
    tensor: torch.Tensor, num_copies: torch.Tensor,
    copy_start_id: torch.Tensor, shard_tokens: torch.Tensor,
):
    """Sums the gradient rows of every duplicate KV copy into its main copy, in place, so
    that only one gradient per shard has to be sent back."""
    _check_tensor(2, tensor, "tensor")
    _check_tensor(1, num_copies, "num_copies")
    _check_tensor(1, shard_tokens, "seq_lens")
    _check_tensor(2, copy_start_id, "copy_start_id")
    num_seqs = num_copies.size(0)
    if shard_tokens.size(0) != num_seqs:
        raise RuntimeError("seq_lens must be of shape (num_sequence,)")
    if copy_start_id.size(0) != num_seqs:
        raise RuntimeError("copy_start_id must be of shape (num_sequence, max_num_copies)")
    _check_dtype(num_copies, torch.int32, "num_copies")
    _check_dtype(copy_start_id, torch.int64, "copy_start_id")
    _check_dtype(shard_tokens, torch.int64, "seq_lens")
    if tensor.dtype not in _DTYPE_CODE:
        raise RuntimeError("Only fp32, fp16 and bf16 inputs are supported")
    with torch.cuda.device(tensor.device):
        rc = _lib.load().distca_grad_sum(
            tensor.data_ptr(), _DTYPE_CODE[tensor.dtype], num_copies.data_ptr(), copy_start_id.data_ptr(),
            shard_tokens.data_ptr(), tensor.size(0), tensor.size(1), num_seqs, copy_start_id.size(1), _stream())
    _lib.check(rc, "pre_a2a_grad_acc")
    return tensor
