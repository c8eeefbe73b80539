"""The CA server's attention ops: unpack -> varlen core attention -> pack.

Mirrors distca/runtime/megatron/ops/fused_comm_attn.py: FlashAttnArgs (:80-104),
_qkv_to_attn_out_fwd (:108-201), _qkv_to_attn_out_bwd (:204-279) and the ordering of
FusedCommAttn.forward / backward (:287-461).  The flash-attn calls of the reference are
replaced by distca_ca_fwd / distca_ca_bwd of the C ABI (hand-written gfx950 kernels);
there is no other attention implementation behind these functions.
"""
from __future__ import annotations

import ctypes
import math
import os
from dataclasses import dataclass
from typing import Optional, Tuple

import torch
from torch import Tensor

from . import _lib
from .ops import DispatcherWrapper, a2a_memcpy_non_cp, a2a_memcpy_non_cp_multi, pre_a2a_grad_acc
from .utils import size_pad_by_int4
from .dispatch import (post_a2a_attn_out, post_a2a_attn_out_grad_resend_qkv, post_a2a_qkv, pre_a2a_attn_out_grad_resend_qkv,
                       pre_a2a_attn_out_with_lse, pre_a2a_qkv)


@dataclass
class PackedSeqParams:
    """The fields of megatron's PackedSeqParams the CA server reads
    (distca/runtime/megatron/packed_seq_params.py:26-57): int32 device cu_seqlens and
    Python-int max_seqlen.  `kv_task_offsets` (int32 [B], optional) gives the first KV row
    of every task so that tasks of one document can share a single KV prefix instead of
    holding one copy each; omitted, task b reads rows cu_seqlens_kv[b]..cu_seqlens_kv[b+1]."""
    cu_seqlens_q: Tensor = None
    cu_seqlens_kv: Tensor = None
    max_seqlen_q: int = None
    max_seqlen_kv: int = None
    qkv_format: str = "thd"
    kv_task_offsets: Optional[Tensor] = None


@dataclass
class FlashAttnArgs:
    num_heads_q: int
    num_heads_kv: int
    head_dim: int
    dropout_p: float = 0.0
    softmax_scale: float = None
    causal: bool = True
    window_size: Tuple[int, int] = (-1, -1)
    softcap: float = 0.0
    alibi_slopes = None
    deterministic: bool = None
    return_attn_probs: bool = False
    block_table = None

    def __post_init__(self):
        if self.deterministic is None:
            # same switch as the reference (fused_comm_attn.py:95-104)
            self.deterministic = os.getenv("NVTE_ALLOW_NONDETERMINISTIC_ALGO", "0") != "1"


# element types of the attention kernels -> DISTCA_DTYPE_* of include/distca_ca.h
_ELEM_CODE = {torch.float16: 1, torch.bfloat16: 2}
HEAD_DIM = 128   # what the kernels are built for; smaller head dimensions are zero-padded to it on the way in


def _params(num_tasks, total_q, total_k, hq, hkv, d, max_q, max_k, scale, causal, deterministic,
            dtype: torch.dtype = torch.bfloat16) -> _lib.CaParams:
    return _lib.CaParams(num_tasks, total_q, total_k, hq, hkv, d, int(max_q), int(max_k), float(scale),
                         1 if causal else 0, 1 if deterministic else 0, _ELEM_CODE[dtype])


def _pad_head_dim(t: Tensor) -> Tensor:
    """[T, H, d] -> [T, H, 128] with zeros behind the d values of every head (the reference pads to a multiple of 8,
    fused_comm_attn.py:125-129, and leaves the rest to flash-attn; here the kernels have one head dimension).
    Zero dimensions add nothing to q.k, and the output's and the gradients' padded dimensions come back as zeros."""
    d = t.shape[-1]
    if d == HEAD_DIM:
        return t
    if d > HEAD_DIM or d % 8:
        raise RuntimeError(f"head_dim={d}: must be a multiple of 8 and at most {HEAD_DIM}")
    return torch.nn.functional.pad(t, (0, HEAD_DIM - d))


def _check_qkv(q: Tensor, k: Tensor, v: Tensor, cu_q: Tensor, cu_k: Tensor, kv_off: Optional[Tensor]):
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.dim() != 3:
            raise RuntimeError(f"{name} must have shape [tokens, heads, head_dim]")
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be on CUDA")
        if t.dtype not in _ELEM_CODE or t.dtype != q.dtype:
            raise RuntimeError(f"{name} must be bfloat16 or float16, the same for q, k and v (got {t.dtype})")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
    if k.shape != v.shape:
        raise RuntimeError("k and v must have the same shape")
    if q.shape[2] != k.shape[2]:
        raise RuntimeError("q and k must have the same head_dim")
    for name, t in (("cu_seqlens_q", cu_q), ("cu_seqlens_k", cu_k)):
        if t.dtype != torch.int32 or not t.is_cuda or t.dim() != 1 or not t.is_contiguous():
            raise RuntimeError(f"{name} must be a contiguous 1-D int32 CUDA tensor")
    if cu_q.shape != cu_k.shape:
        raise RuntimeError("cu_seqlens_q and cu_seqlens_k must have the same shape")
    if kv_off is not None:
        if kv_off.dtype != torch.int32 or not kv_off.is_cuda or kv_off.shape[0] != cu_q.shape[0] - 1:
            raise RuntimeError("kv_task_offsets must be an int32 CUDA tensor of shape [num_tasks]")


def _workspace(given: Optional[Tensor], need: int, device) -> Tensor:
    if given is None:
        return torch.empty((max(need, 16),), dtype=torch.uint8, device=device)
    if given.dtype != torch.uint8 or not given.is_cuda or not given.is_contiguous() or given.numel() < need:
        raise RuntimeError(f"workspace must be a contiguous uint8 CUDA tensor of at least {need} bytes")
    return given


def ca_varlen_fwd(q: Tensor, k: Tensor, v: Tensor, cu_seqlens_q: Tensor, cu_seqlens_k: Tensor,
                  max_seqlen_q: int, max_seqlen_k: int, softmax_scale: Optional[float] = None, causal: bool = True,
                  kv_task_offsets: Optional[Tensor] = None, workspace: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """q [Tq,Hq,D], k,v [Tk,Hkv,D] bf16 or fp16 -> (out [Tq,Hq,D] in the same type, softmax_lse [Hq,Tq] fp32).
    `workspace` (uint8 CUDA tensor of at least distca_ca_fwd_workspace_bytes) is allocated
    per call when omitted.  A head dimension below 128 (multiple of 8) goes through zero-padded copies."""
    _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k, kv_task_offsets)
    scale = softmax_scale if softmax_scale is not None else q.shape[2] ** (-0.5)
    if q.shape[2] != HEAD_DIM:
        d = q.shape[2]
        out, lse = ca_varlen_fwd(_pad_head_dim(q), _pad_head_dim(k), _pad_head_dim(v), cu_seqlens_q, cu_seqlens_k, max_seqlen_q,
                                 max_seqlen_k, scale, causal, kv_task_offsets, workspace)
        return out[..., :d].contiguous(), lse
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    lib = _lib.load()
    p = _params(cu_seqlens_q.shape[0] - 1, tq, tk, hq, hkv, d, max_seqlen_q, max_seqlen_k, scale, causal, False, q.dtype)
    need = lib.distca_ca_fwd_workspace_bytes(ctypes.byref(p))
    if need < 0:
        _lib.check(int(need), "ca_varlen_fwd")
    out = torch.empty_like(q)
    lse = torch.empty((hq, tq), dtype=torch.float32, device=q.device)
    ws = _workspace(workspace, int(need), q.device)
    with torch.cuda.device(q.device):
        rc = lib.distca_ca_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(),
                               cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                               kv_task_offsets.data_ptr() if kv_task_offsets is not None else None,
                               ctypes.byref(p), ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "ca_varlen_fwd")
    return out, lse


def ca_varlen_bwd(dout: Tensor, q: Tensor, k: Tensor, v: Tensor, out: Tensor, softmax_lse: Tensor,
                  cu_seqlens_q: Tensor, cu_seqlens_k: Tensor, max_seqlen_q: int, max_seqlen_k: int,
                  softmax_scale: Optional[float] = None, causal: bool = True, deterministic: bool = False,
                  kv_task_offsets: Optional[Tensor] = None,
                  dq: Optional[Tensor] = None, dk: Optional[Tensor] = None, dv: Optional[Tensor] = None,
                  workspace: Optional[Tensor] = None):
    """Gradients (dq, dk, dv) in the type of q; written into dq/dk/dv when given (the reference's
    flash-attn backward fills caller-allocated tensors, fused_comm_attn.py:236,259-272)."""
    _check_qkv(q, k, v, cu_seqlens_q, cu_seqlens_k, kv_task_offsets)
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    for name, t in (("dout", dout), ("out", out)):
        if t.shape != q.shape or t.dtype != q.dtype or not t.is_cuda:
            raise RuntimeError(f"{name} must be a CUDA tensor with the shape and type of q")
    if d != HEAD_DIM:
        scale = softmax_scale if softmax_scale is not None else d ** (-0.5)
        grads = ca_varlen_bwd(_pad_head_dim(dout), _pad_head_dim(q), _pad_head_dim(k), _pad_head_dim(v), _pad_head_dim(out),
                              softmax_lse, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, scale, causal, deterministic,
                              kv_task_offsets, workspace=workspace)
        res = []
        for g, given in zip(grads, (dq, dk, dv)):
            g = g[..., :d]
            res.append(g.contiguous() if given is None else given.copy_(g))
        return tuple(res)
    dout = dout.contiguous()
    out = out.contiguous()
    if softmax_lse.shape != (hq, tq) or softmax_lse.dtype != torch.float32:
        raise RuntimeError(f"softmax_lse must be fp32 of shape [Hq, Tq] = {(hq, tq)}, got {tuple(softmax_lse.shape)}")
    softmax_lse = softmax_lse.contiguous()
    scale = softmax_scale if softmax_scale is not None else d ** (-0.5)
    lib = _lib.load()
    p = _params(cu_seqlens_q.shape[0] - 1, tq, tk, hq, hkv, d, max_seqlen_q, max_seqlen_k, scale, causal, deterministic, q.dtype)
    need = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(p))
    if need < 0:
        _lib.check(int(need), "ca_varlen_bwd")
    dq = torch.empty_like(q) if dq is None else dq
    dk = torch.empty_like(k) if dk is None else dk
    dv = torch.empty_like(v) if dv is None else dv
    for name, t, ref in (("dq", dq, q), ("dk", dk, k), ("dv", dv, v)):
        if t.shape != ref.shape or t.dtype != q.dtype or not t.is_contiguous() or not t.is_cuda:
            raise RuntimeError(f"{name} must be a contiguous CUDA tensor with the shape and type of its input")
    ws = _workspace(workspace, int(need), q.device)
    with torch.cuda.device(q.device):
        rc = lib.distca_ca_bwd(dout.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(),
                               softmax_lse.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
                               cu_seqlens_q.data_ptr(), cu_seqlens_k.data_ptr(),
                               kv_task_offsets.data_ptr() if kv_task_offsets is not None else None,
                               ctypes.byref(p), ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "ca_varlen_bwd")
    return dq, dk, dv


def _qkv_to_attn_out_fwd(q: Tensor, k: Tensor, v: Tensor, fa_params: PackedSeqParams, fa_args: FlashAttnArgs):
    """2-D [T, H*D] q/k/v in, (out [T, Hq*D], softmax_lse [Hq, T]) out — the contract of
    fused_comm_attn.py:108-201."""
    assert fa_args.causal
    assert fa_args.window_size == (-1, -1)
    assert fa_args.alibi_slopes is None
    assert fa_args.block_table is None
    assert fa_args.dropout_p == 0.0
    q = q.reshape(q.shape[0], fa_args.num_heads_q, fa_args.head_dim)
    k = k.reshape(k.shape[0], fa_args.num_heads_kv, fa_args.head_dim)
    v = v.reshape(v.shape[0], fa_args.num_heads_kv, fa_args.head_dim)
    softmax_scale = fa_args.softmax_scale
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    out, softmax_lse = ca_varlen_fwd(
        q.contiguous(), k.contiguous(), v.contiguous(), fa_params.cu_seqlens_q, fa_params.cu_seqlens_kv,
        fa_params.max_seqlen_q, fa_params.max_seqlen_kv, softmax_scale, causal=fa_args.causal,
        kv_task_offsets=getattr(fa_params, "kv_task_offsets", None))
    out = out.reshape(out.shape[0], fa_args.num_heads_q * fa_args.head_dim)
    return out, softmax_lse


def _qkv_to_attn_out_bwd(
    q: Tensor, k: Tensor, v: Tensor, attn_out: Tensor,
    attn_out_grad: Tensor, softmax_lse: Tensor,
    fa_args: FlashAttnArgs, cu_seqlen_q: Tensor, cu_seqlen_kv: Tensor,
    max_seqlen_q: int, max_seqlen_kv: int, kv_task_offsets: Optional[Tensor] = None,
):
    """(dq [T,Hq*D], dk, dv [Tk,Hkv*D]) — the contract of fused_comm_attn.py:204-279;
    softmax_lse is [Hq, T]."""
    hq, hkv, d = fa_args.num_heads_q, fa_args.num_heads_kv, fa_args.head_dim
    q = q.reshape(q.shape[0], hq, d).contiguous()
    k = k.reshape(k.shape[0], hkv, d).contiguous()
    v = v.reshape(v.shape[0], hkv, d).contiguous()
    out = attn_out.reshape(attn_out.shape[0], hq, d)
    dout = attn_out_grad.reshape(attn_out_grad.shape[0], hq, d)
    softmax_scale = fa_args.softmax_scale
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** (-0.5)
    dq, dk, dv = ca_varlen_bwd(dout, q, k, v, out, softmax_lse, cu_seqlen_q, cu_seqlen_kv, max_seqlen_q, max_seqlen_kv,
                               softmax_scale, fa_args.causal, fa_args.deterministic, kv_task_offsets)
    return (dq.reshape(dq.shape[0], hq * d), dk.reshape(dk.shape[0], hkv * d), dv.reshape(dv.shape[0], hkv * d))


class CoreAttention(torch.autograd.Function):
    """Differentiable varlen core attention on [T, H, D] tensors (drop-in for
    flash_attn_varlen_func(..., causal=True) on the reference's call pattern)."""

    @staticmethod
    def forward(ctx, q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, causal,
                deterministic, kv_task_offsets):
        out, lse = ca_varlen_fwd(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, causal,
                                 kv_task_offsets)
        ctx.save_for_backward(q, k, v, out, lse, cu_seqlens_q, cu_seqlens_k)
        ctx.kv_task_offsets = kv_task_offsets
        ctx.args = (max_seqlen_q, max_seqlen_k, softmax_scale, causal, deterministic)
        return out

    @staticmethod
    def backward(ctx, dout):
        q, k, v, out, lse, cu_q, cu_k = ctx.saved_tensors
        max_q, max_k, scale, causal, det = ctx.args
        dq, dk, dv = ca_varlen_bwd(dout.contiguous(), q, k, v, out, lse, cu_q, cu_k, max_q, max_k, scale, causal, det,
                                   ctx.kv_task_offsets)
        return dq, dk, dv, None, None, None, None, None, None, None, None


def core_attention(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale=None, causal=True,
                   deterministic=False, kv_task_offsets=None):
    return CoreAttention.apply(q, k, v, cu_seqlens_q, cu_seqlens_k, max_seqlen_q, max_seqlen_k, softmax_scale, causal,
                               deterministic, kv_task_offsets)


# ---------------------------------------------------------------------------------------
# The CA server tick, with explicit buffers: what FusedCommAttn.forward / backward do
# between "receive buffer holds this tick's shards" and "send buffer holds the reply".
# ---------------------------------------------------------------------------------------
@dataclass
class SharedKVOnDevice:
    """metadata.SharedKVLayout as the server tick uses it: per stored shard its tokens and the byte offsets it is
    unpacked from (and, in backward, its gradient is packed to); per task the first store row of its prefix."""
    store_tokens: Tensor          # int64 [stored shards]
    k_offset: Tensor              # int64 [stored shards] into the receive buffer
    v_offset: Tensor
    kv_task_offsets: Tensor       # int32 [tasks]
    num_rows: int
    k_grad_offset: Optional[Tensor] = None   # int64 [stored shards] into the send buffer (backward)
    v_grad_offset: Optional[Tensor] = None
    row_start: Optional[Tensor] = None       # int32 [stored shards + 1]: first store row of every shard
    task_shard: Optional[Tensor] = None      # int32 [tasks]: the stored shard that holds the first row of each task's prefix

    @classmethod
    def build(cls, layout, k_entry_offset: Tensor, v_entry_offset: Tensor, device, k_grad_entry_offset: Tensor = None,
              v_grad_entry_offset: Tensor = None) -> "SharedKVOnDevice":
        """`*_entry_offset`: host int64 tensors with one byte offset per K/V entry (aliases of a shard hold the same)."""
        pick = lambda t: None if t is None else t.cpu()[layout.entry_of_stored].to(device=device, dtype=torch.int64)
        row_start = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(layout.store_tokens.cpu(), 0)])
        task_shard = torch.searchsorted(row_start[1:].contiguous(), layout.kv_task_offsets.cpu().to(torch.int64), right=True)
        task_shard = task_shard.clamp_max(max(len(layout.store_tokens) - 1, 0))
        return cls(layout.store_tokens.to(device), pick(k_entry_offset), pick(v_entry_offset),
                   layout.kv_task_offsets.to(device=device, dtype=torch.int32), layout.num_rows,
                   pick(k_grad_entry_offset), pick(v_grad_entry_offset),
                   row_start.to(device=device, dtype=torch.int32), task_shard.to(device=device, dtype=torch.int32))

    def c_struct(self, backward: bool) -> "_lib.KvShards":
        """struct distca_kv_shards over this layout's device arrays (which must outlive the call they are passed to)."""
        ptr = lambda t: None if t is None else t.data_ptr()
        return _lib.KvShards(int(self.store_tokens.numel()), ptr(self.row_start), ptr(self.k_offset), ptr(self.v_offset),
                             ptr(self.task_shard), ptr(self.k_grad_offset) if backward else None,
                             ptr(self.v_grad_offset) if backward else None)


@dataclass
class ServerFwdMeta:
    """Receive-side layout of q/k/v shards and send-side layout of the reply."""
    q_recv_seq_tokens: Tensor      # int64 [nq_shards]
    k_recv_seq_tokens: Tensor      # int64 [nk_shards]
    q_recv_offset: Tensor          # int64 byte offsets into the receive buffer
    k_recv_offset: Tensor
    v_recv_offset: Tensor
    out_send_seq_tokens: Tensor    # int64 [nq_shards]
    out_send_offset: Tensor        # int64 byte offsets into the send buffer ([out | lse] tokens)
    recv_q_shape: Tuple[int, int]  # (Tq, Hq*D)
    recv_k_shape: Tuple[int, int]  # (Tk, Hkv*D)
    shared_kv: Optional[SharedKVOnDevice] = None   # when given, the in-place tick keeps one copy of every K/V shard


def ca_server_forward(recv_buffer: Tensor, send_buffer: Tensor, meta: ServerFwdMeta, fa_params: PackedSeqParams,
                      fa_args: FlashAttnArgs, dtype: torch.dtype = torch.bfloat16, in_place: bool = True,
                      kv_shards_in_place: bool = True):
    """fused_comm_attn.py:298-389: unpack q,k,v -> attention -> pack [out | lse].

    With `in_place` (the default) the kernel reads the query tokens where they lie in the receive
    buffer and writes the [out | lse] tokens where they belong in the send buffer.  With the one-copy
    K/V layout (`meta.shared_kv`) it also reads the K/V shards where they lie (no pack kernel runs at
    all; `kv_shards_in_place=False` unpacks every stored shard once instead); without that layout K and
    V are unpacked as in the reference, a shard read by several tasks once per task.  Returns (None, None) then.
    Without it every step is its own pass, as in the reference, and (attn_out [T,Hq*D],
    softmax_lse [Hq,T]) are returned for the caller's own use.  Both leave the same bytes in the
    send buffer."""
    dev = recv_buffer.device
    hq, hkv, d = fa_args.num_heads_q, fa_args.num_heads_kv, fa_args.head_dim
    in_place = in_place and dtype in _ELEM_CODE and d == HEAD_DIM
    shared = meta.shared_kv if in_place else None
    # with the one-copy layout the kernel reads the K/V shards where they lie in the receive buffer: nothing is unpacked
    kv_in_place = shared is not None and kv_shards_in_place and shared.row_start is not None and shared.num_rows > 0
    k_rows = shared.num_rows if shared is not None else meta.recv_k_shape[0]
    if not kv_in_place:
        recv_k = torch.empty((k_rows, meta.recv_k_shape[1]), dtype=dtype, device=dev)
        recv_v = torch.empty_like(recv_k)
    if in_place:
        kv_off = getattr(fa_params, "kv_task_offsets", None)
        if kv_in_place:
            kv_off = shared.kv_task_offsets
        elif shared is not None:
            # one copy of every K/V shard, documents contiguous: every task reads its prefix in place
            a2a_memcpy_non_cp_multi([recv_k, recv_v], [shared.k_offset, shared.v_offset], [shared.store_tokens] * 2, False,
                                    buffer=recv_buffer)
            kv_off = shared.kv_task_offsets
        else:
            a2a_memcpy_non_cp_multi([recv_k, recv_v], [meta.k_recv_offset, meta.v_recv_offset], [meta.k_recv_seq_tokens] * 2,
                                    False, buffer=recv_buffer)
        tq, tk = int(meta.recv_q_shape[0]), int(k_rows)
        scale = fa_args.softmax_scale if fa_args.softmax_scale is not None else d ** (-0.5)
        lib = _lib.load()
        cu_q, cu_k = fa_params.cu_seqlens_q, fa_params.cu_seqlens_kv
        assert fa_args.causal and fa_args.window_size == (-1, -1) and fa_args.dropout_p == 0.0
        p = _params(cu_q.shape[0] - 1, tq, tk, hq, hkv, d, fa_params.max_seqlen_q, fa_params.max_seqlen_kv, scale,
                    fa_args.causal, False, dtype)
        need = lib.distca_ca_fwd_workspace_bytes(ctypes.byref(p))
        if need < 0:
            _lib.check(int(need), "ca_server_forward")
        ws = _workspace(None, int(need), dev)
        q_tok = hq * d * 2
        out_tok = size_pad_by_int4(q_tok + hq * 4, 1)[0]
        for name, t in (("q_recv_offset", meta.q_recv_offset), ("out_send_offset", meta.out_send_offset)):
            if t.dtype != torch.int64 or not t.is_cuda or t.numel() != cu_q.shape[0] - 1:
                raise RuntimeError(f"{name} must be an int64 CUDA tensor with one entry per task")
        with torch.cuda.device(dev):
            if kv_in_place:
                shards = shared.c_struct(False)
                rc = lib.distca_ca_fwd_buffers(recv_buffer.data_ptr(), meta.q_recv_offset.data_ptr(), q_tok, recv_buffer.data_ptr(),
                                               recv_buffer.data_ptr(), ctypes.byref(shards), send_buffer.data_ptr(),
                                               meta.out_send_offset.data_ptr(), out_tok, None, cu_q.data_ptr(), cu_k.data_ptr(),
                                               kv_off.data_ptr(), ctypes.byref(p), ws.data_ptr(), ws.numel(),
                                               torch.cuda.current_stream().cuda_stream)
            else:
                rc = lib.distca_ca_fwd_tokens(recv_buffer.data_ptr(), meta.q_recv_offset.data_ptr(), q_tok, recv_k.data_ptr(),
                                              recv_v.data_ptr(), send_buffer.data_ptr(), meta.out_send_offset.data_ptr(), out_tok,
                                              None, cu_q.data_ptr(), cu_k.data_ptr(), kv_off.data_ptr() if kv_off is not None else None,
                                              ctypes.byref(p), ws.data_ptr(),
                                              ws.numel(), torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "ca_server_forward")
        return None, None
    recv_q = torch.empty(meta.recv_q_shape, dtype=dtype, device=dev)
    post_a2a_qkv(recv_q, recv_k, recv_v, None, meta.q_recv_seq_tokens, meta.k_recv_seq_tokens,
                 meta.q_recv_offset, meta.k_recv_offset, meta.v_recv_offset, is_fwd=True, buffer=recv_buffer)
    attn_out, softmax_lse = _qkv_to_attn_out_fwd(recv_q, recv_k, recv_v, fa_params, fa_args)
    lse_t = softmax_lse.T.contiguous()  # [T, Hq] for transport (fused_comm_attn.py:370-371)
    pre_a2a_attn_out_with_lse(attn_out, lse_t, meta.out_send_seq_tokens, meta.out_send_offset, buffer=send_buffer)
    return attn_out, softmax_lse


@dataclass
class ServerBwdMeta:
    q_recv_seq_tokens: Tensor      # merged [dO | O | lse | q] shards
    k_recv_seq_tokens: Tensor
    q_recv_offset: Tensor
    k_recv_offset: Tensor
    v_recv_offset: Tensor
    q_grad_send_seq_tokens: Tensor
    k_grad_send_seq_tokens: Tensor
    q_grad_send_offset: Tensor
    k_grad_send_offset: Tensor
    v_grad_send_offset: Tensor
    main_copy_mask: Tensor         # int8 [nk_shards]
    num_copies: Tensor             # int32 [nk_shards]
    copy_start_id: Tensor          # int64 [nk_shards, max_copies]
    attn_out_shape: Tuple[int, int]
    lse_shape: Tuple[int, int]     # (T, Hq)
    k_shape: Tuple[int, int]
    shared_kv: Optional[SharedKVOnDevice] = None


def ca_server_backward(recv_buffer: Tensor, send_buffer: Tensor, meta: ServerBwdMeta, fa_args: FlashAttnArgs,
                       cu_seqlens_q: Tensor, cu_seqlens_kv: Tensor, max_seqlen_q: int, max_seqlen_kv: int,
                       dtype: torch.dtype = torch.bfloat16, in_place: bool = True, kv_shards_in_place: bool = True):
    """fused_comm_attn.py:407-461: unpack merged request -> attention backward -> sum
    duplicate KV gradients -> masked pack of dq, dk, dv.

    With `in_place` (the default, for head counts that keep the q part of a request token 16-byte
    aligned) the kernels read dO, O, lse and q where they lie in the receive buffer and write dq
    where it belongs in the send buffer; K and V are unpacked (with `meta.shared_kv` every stored shard once, and
    dk / dv then come out summed over the tasks that read a shard and are packed once), dk and dv otherwise summed
With that layout and `kv_shards_in_place` (the default) the kernels also read the K/V shards where they lie
    and write the shards' dk / dv where they belong in the send buffer: no pack kernel runs, and (None, None, None)
    is returned.  Otherwise returns (None, dk, dv) when in place, else (dq, dk, dv).  dq bytes in the send buffer are
    the same in every form; dk / dv of the one-copy forms are summed in fp32 and rounded once, those of the step-by-step
    form are bf16 sums of per-task bf16 gradients, as in the reference."""
    dev = recv_buffer.device
    hq, hkv, d = fa_args.num_heads_q, fa_args.num_heads_kv, fa_args.head_dim
    in_place = in_place and (hq * 4) % 16 == 0 and dtype in _ELEM_CODE and d == HEAD_DIM
    # one copy of every K/V shard, whatever the deterministic switch says: one work item per (document, key block)
    # sums dK/dV over the document's tasks in registers
    shared = meta.shared_kv if in_place else None
    k_rows = shared.num_rows if shared is not None else meta.k_shape[0]
    kv_in_place = (shared is not None and kv_shards_in_place and shared.row_start is not None and shared.num_rows > 0
                   and shared.k_grad_offset is not None and int(cu_seqlens_q.shape[0]) > 1 and int(meta.attn_out_shape[0]) > 0)
    if kv_in_place:
        # everything where it lies: request tokens and K/V shards read from the receive buffer, dq tokens and the
        # shards' dk / dv written into the send buffer; no pack kernel runs
        tq = int(meta.attn_out_shape[0])
        scale = fa_args.softmax_scale if fa_args.softmax_scale is not None else d ** (-0.5)
        lib = _lib.load()
        p = _params(cu_seqlens_q.shape[0] - 1, tq, int(k_rows), hq, hkv, d, max_seqlen_q, max_seqlen_kv, scale, fa_args.causal,
                    fa_args.deterministic, dtype)
        need = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(p))
        if need < 0:
            _lib.check(int(need), "ca_server_backward")
        ws = _workspace(None, int(need), dev)
        row = hq * d * 2
        req_tok = size_pad_by_int4(3 * row + hq * 4, 1)[0]
        for name, t in (("q_recv_offset", meta.q_recv_offset), ("q_grad_send_offset", meta.q_grad_send_offset)):
            if t.dtype != torch.int64 or not t.is_cuda or t.numel() != cu_seqlens_q.shape[0] - 1:
                raise RuntimeError(f"{name} must be an int64 CUDA tensor with one entry per task")
        shards = shared.c_struct(True)
        with torch.cuda.device(dev):
            rc = lib.distca_ca_bwd_buffers(recv_buffer.data_ptr(), meta.q_recv_offset.data_ptr(), req_tok, recv_buffer.data_ptr(),
                                           recv_buffer.data_ptr(), ctypes.byref(shards), send_buffer.data_ptr(),
                                           meta.q_grad_send_offset.data_ptr(), row, send_buffer.data_ptr(), send_buffer.data_ptr(),
                                           cu_seqlens_q.data_ptr(), cu_seqlens_kv.data_ptr(), shared.kv_task_offsets.data_ptr(),
                                           ctypes.byref(p), ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "ca_server_backward")
        return None, None, None
    recv_k = torch.empty((k_rows, meta.k_shape[1]), dtype=dtype, device=dev)
    recv_v = torch.empty_like(recv_k)
    if in_place:
        if shared is not None:
            a2a_memcpy_non_cp_multi([recv_k, recv_v], [shared.k_offset, shared.v_offset], [shared.store_tokens] * 2, False,
                                    buffer=recv_buffer)
        else:
            a2a_memcpy_non_cp_multi([recv_k, recv_v], [meta.k_recv_offset, meta.v_recv_offset], [meta.k_recv_seq_tokens] * 2,
                                    False, buffer=recv_buffer)
        tq, tk = int(meta.attn_out_shape[0]), int(k_rows)
        scale = fa_args.softmax_scale if fa_args.softmax_scale is not None else d ** (-0.5)
        lib = _lib.load()
        p = _params(cu_seqlens_q.shape[0] - 1, tq, tk, hq, hkv, d, max_seqlen_q, max_seqlen_kv, scale, fa_args.causal,
                    fa_args.deterministic, dtype)
        need = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(p))
        if need < 0:
            _lib.check(int(need), "ca_server_backward")
        ws = _workspace(None, int(need), dev)
        row = hq * d * 2
        req_tok = size_pad_by_int4(3 * row + hq * 4, 1)[0]
        for name, t in (("q_recv_offset", meta.q_recv_offset), ("q_grad_send_offset", meta.q_grad_send_offset)):
            if t.dtype != torch.int64 or not t.is_cuda or t.numel() != cu_seqlens_q.shape[0] - 1:
                raise RuntimeError(f"{name} must be an int64 CUDA tensor with one entry per task")
        dk = torch.empty((tk, hkv * d), dtype=dtype, device=dev)
        dv = torch.empty_like(dk)
        with torch.cuda.device(dev):
            rc = lib.distca_ca_bwd_tokens(recv_buffer.data_ptr(), meta.q_recv_offset.data_ptr(), req_tok, recv_k.data_ptr(),
                                          recv_v.data_ptr(), send_buffer.data_ptr(), meta.q_grad_send_offset.data_ptr(), row,
                                          dk.data_ptr(), dv.data_ptr(), cu_seqlens_q.data_ptr(), cu_seqlens_kv.data_ptr(),
                                          shared.kv_task_offsets.data_ptr() if shared is not None else None,
                                          ctypes.byref(p), ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream)
        _lib.check(rc, "ca_server_backward")
        if shared is not None:
            # every stored shard holds the gradient summed over the tasks that read it: one pack, no duplicates to add up
            a2a_memcpy_non_cp_multi([dk, dv], [shared.k_grad_offset, shared.v_grad_offset], [shared.store_tokens] * 2, True,
                                    buffer=send_buffer)
            return None, dk, dv
        for g in (dk, dv):
            pre_a2a_grad_acc(g, meta.num_copies, meta.copy_start_id, meta.k_grad_send_seq_tokens)
        a2a_memcpy_non_cp_multi([dk, dv], [meta.k_grad_send_offset, meta.v_grad_send_offset], [meta.k_grad_send_seq_tokens] * 2,
                                True, [meta.main_copy_mask] * 2, buffer=send_buffer)
        return None, dk, dv
    (dout, out, lse, q, recv_k, recv_v) = post_a2a_attn_out_grad_resend_qkv(
        meta.attn_out_shape, meta.lse_shape, meta.attn_out_shape, torch.float32, recv_k, recv_v, None,
        meta.q_recv_seq_tokens, meta.k_recv_seq_tokens, meta.q_recv_offset, meta.k_recv_offset, meta.v_recv_offset,
        is_fwd=True, buffer=recv_buffer)
    lse = lse.T.contiguous()  # [Hq, T] (fused_comm_attn.py:440)
    dq, dk, dv = _qkv_to_attn_out_bwd(q, recv_k, recv_v, out, dout, lse, fa_args, cu_seqlens_q, cu_seqlens_kv,
                                      max_seqlen_q, max_seqlen_kv)
    dq, dk, dv = pre_a2a_qkv(
        dq, dk, dv, None, meta.q_grad_send_seq_tokens, meta.k_grad_send_seq_tokens,
        meta.q_grad_send_offset, meta.k_grad_send_offset, meta.v_grad_send_offset,
        is_fwd=False, kv_grad_copy_shard_mask=meta.main_copy_mask,
        pre_a2a_grad_acc_args=(meta.num_copies, meta.copy_start_id, meta.k_grad_send_seq_tokens), buffer=send_buffer)
    return dq, dk, dv


# ---------------------------------------------------------------------------------------
# The same tick driven by AlltoAllMetadata, and the linear side of it (what the reference's
# autograd functions do around the all-to-all): fused_comm_attn.py:287-461 and :464-526.
# ---------------------------------------------------------------------------------------
def fused_comm_attn_forward(recv_buffer: Tensor, send_buffer: Tensor, packed_seq_params, fa_args: FlashAttnArgs,
                            dtype: torch.dtype = torch.bfloat16):
    """FusedCommAttn.forward on explicit buffers: `recv_buffer` holds what the q/k/v all-to-all
    delivered (qkv_fwd_metadata.recv_memcpy_metadata), `send_buffer` receives the [out | lse] reply
    (attn_out_fwd_metadata.send_memcpy_metadata).  Returns (attn_out, softmax_lse [Hq, T])."""
    qkv, out = packed_seq_params.qkv_fwd_metadata, packed_seq_params.attn_out_fwd_metadata
    q_off, k_off, v_off = qkv.recv_memcpy_metadata
    meta = ServerFwdMeta(qkv.seq_lens[0].recv_seqlens, qkv.seq_lens[1].recv_seqlens, q_off, k_off, v_off,
                         out.seq_lens[0].send_seqlens, out.send_memcpy_metadata[0],
                         tuple(qkv.tensor_shape[0].recv_shape), tuple(qkv.tensor_shape[1].recv_shape),
                         shared_kv=getattr(packed_seq_params, "shared_kv_fwd", None))
    return ca_server_forward(recv_buffer, send_buffer, meta, packed_seq_params, fa_args, dtype)


def fused_comm_attn_backward(recv_buffer: Tensor, send_buffer: Tensor, packed_seq_params, fa_args: FlashAttnArgs,
                             dtype: torch.dtype = torch.bfloat16):
    """FusedCommAttn.backward / dummy_backward_single_sided (fused_comm_attn.py:407-461, 529-642)
    on explicit buffers: request per attn_out_bwd_metadata, gradient reply per qkv_bwd_metadata."""
    req, grad = packed_seq_params.attn_out_bwd_metadata, packed_seq_params.qkv_bwd_metadata
    bwd = packed_seq_params.bwd_packed_seq_params
    q_off, k_off, v_off = req.recv_memcpy_metadata
    gq_off, gk_off, gv_off = grad.send_memcpy_metadata
    tq = int(req.tensor_shape[0].recv_shape[0])
    hq_d = fa_args.num_heads_q * fa_args.head_dim
    d = grad.kv_grad_send_dedup
    meta = ServerBwdMeta(req.seq_lens[0].recv_seqlens, req.seq_lens[1].recv_seqlens, q_off, k_off, v_off,
                         grad.seq_lens[0].send_seqlens, grad.seq_lens[1].send_seqlens, gq_off, gk_off, gv_off,
                         d.main_copy_mask, d.num_copies, d.copy_start_id, (tq, hq_d), (tq, fa_args.num_heads_q),
                         tuple(req.tensor_shape[1].recv_shape), shared_kv=getattr(packed_seq_params, "shared_kv_bwd", None))
    return ca_server_backward(recv_buffer, send_buffer, meta, fa_args, bwd.cu_seqlens_q, bwd.cu_seqlens_kv,
                              bwd.max_seqlen_q, bwd.max_seqlen_kv, dtype)


def _server_buffers(dispatcher_id):
    """(receive buffer, send buffer) of one tick through the dispatcher, with the reference's
    bookkeeping (dispatch.py:60-94 of the reference, then :97-106): the receive buffer is the named
    instance's, or the current one's, which then stops being current; the reply goes into the
    instance that is named, or current after that switch.  The caller releases a named instance
    once its kernels are enqueued (`_server_done`)."""
    if dispatcher_id is not None:
        assert DispatcherWrapper.is_acquired[dispatcher_id], "no all-to-all has filled this dispatcher's receive buffer"
    recv = DispatcherWrapper.get_instance(dispatcher_id).recv_buffer
    if dispatcher_id is None:
        DispatcherWrapper.switch_buffer()
    return recv, DispatcherWrapper.get_instance(dispatcher_id).send_buffer


def _server_done(dispatcher_id):
    # in-place ticks read the receive buffer from inside the attention kernels, so the release
    # follows them in stream order rather than the unpack, as it does in the reference
    if dispatcher_id is not None:
        DispatcherWrapper.release(dispatcher_id)


class FusedCommAttn(torch.autograd.Function):
    """The CA server's tick as the reference's autograd function (fused_comm_attn.py:282-461), same
    arguments in the same order: unpack what the q/k/v all-to-all delivered, attention, pack the
    [out | lse] reply; its backward unpacks the request [dO | O | lse | q] + k + v, runs the attention
    backward and packs dq and the k / v gradients of the main copies.  Tensors travel through the
    `DispatcherWrapper` instance `dispatcher_id`; what autograd sees is a one-element signal."""

    @staticmethod
    def forward(ctx, signal: Tensor, fwd_qkv_metadata, bwd_qkv_metadata, fwd_attn_out_metadata, bwd_attn_out_qkv_metadata,
                fwd_fa_params, bwd_fa_params, dispatcher_id: int, flash_attn_args: FlashAttnArgs):
        qkv, out = fwd_qkv_metadata, fwd_attn_out_metadata
        q_off, k_off, v_off = qkv.recv_memcpy_metadata
        meta = ServerFwdMeta(qkv.seq_lens[0].recv_seqlens, qkv.seq_lens[1].recv_seqlens, q_off, k_off, v_off,
                             out.seq_lens[0].send_seqlens, out.send_memcpy_metadata[0],
                             tuple(qkv.tensor_shape[0].recv_shape), tuple(qkv.tensor_shape[1].recv_shape),
                             shared_kv=getattr(fwd_fa_params, "shared_kv_fwd", None))
        recv_buffer, send_buffer = _server_buffers(dispatcher_id)
        ca_server_forward(recv_buffer, send_buffer, meta, fwd_fa_params, flash_attn_args, signal.dtype)
        _server_done(dispatcher_id)

        req, grad = bwd_attn_out_qkv_metadata, bwd_qkv_metadata
        dedup = grad.kv_grad_send_dedup
        ctx.save_for_backward(
            req.seq_lens[0].recv_seqlens, req.seq_lens[1].recv_seqlens, *req.recv_memcpy_metadata,
            grad.seq_lens[0].send_seqlens, grad.seq_lens[1].send_seqlens, *grad.send_memcpy_metadata,
            dedup.main_copy_mask, dedup.num_copies, dedup.copy_start_id,
            bwd_fa_params.cu_seqlens_q, bwd_fa_params.cu_seqlens_kv)
        ctx.dispatcher_id = dispatcher_id
        ctx.fa_args = flash_attn_args
        ctx.bwd_attn_max_seqlen_q = bwd_fa_params.max_seqlen_q
        ctx.bwd_attn_max_seqlen_kv = bwd_fa_params.max_seqlen_kv
        tq = int(req.tensor_shape[0].recv_shape[0])
        ctx.bwd_q_shape = (tq, flash_attn_args.num_heads_q * flash_attn_args.head_dim)
        ctx.softmax_lse_shape = (tq, flash_attn_args.num_heads_q)
        ctx.bwd_k_shape = tuple(req.tensor_shape[1].recv_shape)
        ctx.shared_kv_bwd = getattr(fwd_fa_params, "shared_kv_bwd", None)
        return torch.empty((1,), device=signal.device, dtype=signal.dtype)

    @staticmethod
    def backward(ctx, signal_grad: Tensor):
        (q_tokens, k_tokens, q_off, k_off, v_off, gq_tokens, gk_tokens, gq_off, gk_off, gv_off,
         main_copy_mask, num_copies, copy_start_id, cu_q, cu_kv) = ctx.saved_tensors
        meta = ServerBwdMeta(q_tokens, k_tokens, q_off, k_off, v_off, gq_tokens, gk_tokens, gq_off, gk_off, gv_off,
                             main_copy_mask, num_copies, copy_start_id, ctx.bwd_q_shape, ctx.softmax_lse_shape,
                             ctx.bwd_k_shape, shared_kv=ctx.shared_kv_bwd)
        recv_buffer, send_buffer = _server_buffers(ctx.dispatcher_id)
        ca_server_backward(recv_buffer, send_buffer, meta, ctx.fa_args, cu_q, cu_kv, ctx.bwd_attn_max_seqlen_q,
                           ctx.bwd_attn_max_seqlen_kv, signal_grad.dtype)
        _server_done(ctx.dispatcher_id)
        return (torch.empty((1,), device=signal_grad.device, dtype=signal_grad.dtype),) + (None,) * 8


@torch.no_grad()
def dummy_backward_single_sided(config, packed_seq_params, dtype: torch.dtype, device, attn_out_grad_all2all: bool = True,
                                qkv_grad_all2all: bool = True):
    """The backward of FusedCommAttn with its two all-to-alls, outside autograd (fused_comm_attn.py:529-642 of the
    reference, which a pipeline stage runs for micro-batches whose forward ran elsewhere): the request all-to-all (unless
    the caller has done it), the server's backward tick, the gradient all-to-all (or, left to the caller, an event
    recorded behind the tick).  `config` gives num_attention_heads, num_query_groups, hidden_size and
    tensor_model_parallel_size; buffers are those of dispatcher `packed_seq_params.dispatcher_id`."""
    from .ops import fast_a2a
    assert packed_seq_params.bwd_packed_seq_params is not None
    tp = config.tensor_model_parallel_size
    num_heads = config.num_attention_heads // tp
    hidden = config.hidden_size // tp
    fa_args = FlashAttnArgs(num_heads_q=num_heads, num_heads_kv=config.num_query_groups // tp, head_dim=hidden // num_heads,
                            return_attn_probs=True)
    dispatcher_id = packed_seq_params.dispatcher_id
    req, grad = packed_seq_params.attn_out_bwd_metadata, packed_seq_params.qkv_bwd_metadata
    stream = getattr(packed_seq_params, "stream", None)
    if attn_out_grad_all2all:
        with torch.cuda.stream(stream):
            fast_a2a(*req.fa2a_metadata, req.my_rank_send_offset, req.my_rank_recv_offset, req.my_rank_send_sz,
                     instance_id=dispatcher_id)
        if stream is not None:
            torch.cuda.current_stream().wait_stream(stream)
    else:
        assert dispatcher_id is not None
    recv_buffer, send_buffer = _server_buffers(dispatcher_id)
    fused_comm_attn_backward(recv_buffer, send_buffer, packed_seq_params, fa_args, dtype)
    _server_done(dispatcher_id)
    if not qkv_grad_all2all:
        assert dispatcher_id is not None
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream())
        return event
    if stream is not None:
        stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        fast_a2a(*grad.fa2a_metadata, grad.my_rank_send_offset, grad.my_rank_recv_offset, grad.my_rank_send_sz,
                 instance_id=dispatcher_id)
    if dispatcher_id is None:
        DispatcherWrapper.switch_buffer()
    return None


def post_a2a_attn_out_with_lse(recv_buffer: Optional[Tensor], q: Tensor, num_heads_q: int, metadata, dtype: torch.dtype = None,
                               instance_id: int = None, switch_buffer: bool = False):
    """Linear side, forward of the reference's autograd function of the same name
    (fused_comm_attn.py:468-506): unpack the [out | lse | pad] tokens of the reply and split them.
    Returns (attn_out [T, 1, Hq*D] in q's dtype, softmax_lse_bytes [T, Hq*4] uint8).  `recv_buffer`
    None reads the receive buffer of dispatcher instance `instance_id`."""
    dtype = dtype or q.dtype
    recv_shape = tuple(metadata.tensor_shape[0].recv_shape)    # in elements of `dtype`, as the reference has it
    recv = torch.empty(recv_shape, dtype=dtype, device=q.device).view(torch.uint8)
    post_a2a_attn_out(recv, metadata.seq_lens[0].recv_seqlens, *metadata.recv_memcpy_metadata, switch_buffer=switch_buffer,
                      instance_id=instance_id, buffer=recv_buffer)
    itemsize = torch.empty((), dtype=dtype).element_size()
    hidden_bytes = math.prod(q.shape[1:]) * itemsize
    lse_bytes = num_heads_q * 4
    attn_out = recv[:, :hidden_bytes].contiguous().view(dtype).unsqueeze(1)
    softmax_lse_bytes = recv[:, hidden_bytes:hidden_bytes + lse_bytes]
    return attn_out, softmax_lse_bytes


def post_a2a_attn_out_with_lse_backward(send_buffer: Optional[Tensor], grad_attn_out: Tensor, attn_out: Tensor, softmax_lse_bytes: Tensor,
                                        q: Tensor, k: Tensor, v: Tensor, bwd_attn_out_qkv_metadata, instance_id: int = None):
    """Linear side, backward of the same function (fused_comm_attn.py:508-526): pack the request
    [dO | O | lse | q | pad] and the K/V shards for the attention server (`send_buffer` None: into the
    send buffer of dispatcher instance `instance_id`)."""
    flat = lambda t: t.reshape(t.shape[0], math.prod(t.shape[1:]))   # -1 is ambiguous for a rank that holds no tokens
    md = bwd_attn_out_qkv_metadata
    pre_a2a_attn_out_grad_resend_qkv(
        flat(grad_attn_out), flat(attn_out), softmax_lse_bytes, flat(q), flat(k), flat(v), md.kv_replica_mask,
        md.seq_lens[0].send_seqlens, md.seq_lens[1].send_seqlens, *md.send_memcpy_metadata,
        instance_id=instance_id, buffer=send_buffer)
