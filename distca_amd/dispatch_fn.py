"""The layout transfers either side of the all-to-all, driven by AlltoAllMetadata, on explicit
buffers.

The reference wraps these in autograd functions that talk to an NVSHMEM dispatcher
(distca/runtime/dispatch_fn.py:28-224: pre_all2all_layout_transfer, post_all2all_layout_transfer).
Here the forward and backward halves are plain functions of the same name (+ `_backward`): the
caller owns the send and receive buffers and passes the one in play as `buffer=`.
"""
from __future__ import annotations

import torch
from torch import Tensor

from .dispatch import post_a2a_attn_out, post_a2a_qkv, pre_a2a_attn_out, pre_a2a_qkv
from .metadata import AlltoAllMetadata


def pre_all2all_layout_transfer(q: Tensor, k: Tensor, v: Tensor, metadata: AlltoAllMetadata, is_qkv: bool = True, *,
                                buffer: Tensor) -> None:
    """Sender packs its shards into the send buffer (dispatch_fn.py:31-70): q plainly, k and v
    once per destination replica; an attention output (is_qkv False) like q."""
    if is_qkv:
        pre_a2a_qkv(q.contiguous(), k.contiguous(), v.contiguous(), metadata.kv_replica_mask,
                    metadata.seq_lens[0].send_seqlens, metadata.seq_lens[1].send_seqlens, *metadata.send_memcpy_metadata,
                    is_fwd=True, buffer=buffer)
    else:
        assert k is None and v is None
        pre_a2a_attn_out(q.contiguous(), metadata.seq_lens[0].send_seqlens, *metadata.send_memcpy_metadata, buffer=buffer)


def pre_all2all_layout_transfer_backward(bwd_metadata: AlltoAllMetadata, dtype: torch.dtype, is_qkv: bool = True, *,
                                         buffer: Tensor):
    """The original sender unpacks the gradients that came back (dispatch_fn.py:72-107): dq
    plainly; dk and dv land in one plane per replica, planes nobody wrote stay zero, and the sum
    over planes is the shard's gradient.  Returns (dq, dk, dv) or (d_attn_out,)."""
    dev = buffer.device
    grad_q = torch.empty(tuple(bwd_metadata.tensor_shape[0].recv_shape), dtype=dtype, device=dev)
    if not is_qkv:
        post_a2a_attn_out(grad_q, bwd_metadata.seq_lens[0].recv_seqlens, *bwd_metadata.recv_memcpy_metadata, buffer=buffer)
        return (grad_q,)
    grad_k = torch.zeros(tuple(bwd_metadata.tensor_shape[1].recv_shape), dtype=dtype, device=dev)
    grad_v = torch.zeros_like(grad_k)
    post_a2a_qkv(grad_q, grad_k, grad_v, bwd_metadata.kv_replica_mask, bwd_metadata.seq_lens[0].recv_seqlens,
                 bwd_metadata.seq_lens[1].recv_seqlens, *bwd_metadata.recv_memcpy_metadata, is_fwd=False, buffer=buffer)
    return grad_q, grad_k.sum(dim=0), grad_v.sum(dim=0)


def post_all2all_layout_transfer(metadata: AlltoAllMetadata, dtype: torch.dtype, is_qkv: bool = True, *, buffer: Tensor):
    """Receiver unpacks what arrived (dispatch_fn.py:143-191): (q, k, v) in the attention layout,
    K/V shards once per task that reads them; or the attention output in the linear layout."""
    dev = buffer.device
    recv_q = torch.empty(tuple(metadata.tensor_shape[0].recv_shape), dtype=dtype, device=dev)
    if not is_qkv:
        post_a2a_attn_out(recv_q, metadata.seq_lens[0].recv_seqlens, *metadata.recv_memcpy_metadata, buffer=buffer)
        return (recv_q,)
    recv_k = torch.empty(tuple(metadata.tensor_shape[1].recv_shape), dtype=dtype, device=dev)
    recv_v = torch.empty_like(recv_k)
    post_a2a_qkv(recv_q, recv_k, recv_v, None, metadata.seq_lens[0].recv_seqlens, metadata.seq_lens[1].recv_seqlens,
                 *metadata.recv_memcpy_metadata, is_fwd=True, buffer=buffer)
    return recv_q, recv_k, recv_v


def post_all2all_layout_transfer_backward(grads, bwd_metadata: AlltoAllMetadata, is_qkv: bool = True, *, buffer: Tensor) -> None:
    """The receiver packs the gradients of what it unpacked (dispatch_fn.py:193-224): for q/k/v
    the copies of a K/V shard are summed into the main copy, and only main copies are sent."""
    if not is_qkv:
        (grad_q,) = grads
        pre_a2a_attn_out(grad_q.contiguous(), bwd_metadata.seq_lens[0].send_seqlens, *bwd_metadata.send_memcpy_metadata,
                         buffer=buffer)
        return
    grad_q, grad_k, grad_v = grads
    d = bwd_metadata.kv_grad_send_dedup
    assert d is not None
    kv_lens = bwd_metadata.seq_lens[1].send_seqlens
    pre_a2a_qkv(grad_q, grad_k, grad_v, bwd_metadata.kv_replica_mask, bwd_metadata.seq_lens[0].send_seqlens, kv_lens,
                *bwd_metadata.send_memcpy_metadata, is_fwd=False, kv_grad_copy_shard_mask=d.main_copy_mask,
                pre_a2a_grad_acc_args=(d.num_copies, d.copy_start_id, kv_lens), buffer=buffer)
