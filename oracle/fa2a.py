"""CPU oracle for the fa2a shard pack / unpack and duplicate-gradient kernels.
TEST INFRASTRUCTURE ONLY — nothing in the product path may import this module.

Restates, byte by byte in numpy / torch-CPU:
  * memcpy_nvshmem_non_cp   csrc/core/memcpy.cu:22-74   -> copy_non_cp
  * memcpy_nvshmem_cp       csrc/core/memcpy.cu:77-155  -> copy_cp
  * inplace_grad_sum_kernel csrc/core/memcpy.cu:158-236 -> grad_sum
following the kernels' token loops literally (one logical token at a time in the
`*_tokenwise` forms, used on small inputs) and as slice copies (the fast forms).

Pinned by (tests/test_oracle_fa2a.py): the reference's own pure-torch simulators
simulate_fa2a_copy_non_cp / simulate_fa2a_copy_cp (tests/test_fa2a_metadata.py:8-59),
re-expressed there as the expected results of hand-sized cases; the answer construction
of tests/all_to_all/test_grad_sum_kernel.py:84-98; pack-then-unpack identity; masked
shards leave the buffer untouched; cp unpack of a cp pack summed over replica planes equals
source x replica count (tests/test_shard_info_to_fa2a.py:212-227); and agreement of the
token-wise and slice forms.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch


def _bytes2d(t: np.ndarray) -> np.ndarray:
    assert t.flags["C_CONTIGUOUS"]
    return t.view(np.uint8).reshape(t.shape[0], int(np.prod(t.shape[1:])) * t.itemsize)


def copy_non_cp(tensor: np.ndarray, buffer: np.ndarray, seq_offset, seq_tokens, copy_seq_mask=None,
                to_buffer: bool = True) -> None:
    """tensor: [T, ...] any dtype (C-contiguous), buffer: 1-D uint8.  In place.

    memcpy.cu:39-72: token_idx walks 0..T-1; shard s covers tokens
    [start_s, start_s+len_s); masked shards are skipped when packing."""
    tb = _bytes2d(tensor)
    num_tokens, token_bytes = tb.shape
    start = 0
    for s, ln in enumerate(np.asarray(seq_tokens).tolist()):
        lo, hi = start, min(start + ln, num_tokens)  # the kernel never passes total_num_tokens
        start += ln
        if hi <= lo:
            continue
        if to_buffer and copy_seq_mask is not None and not copy_seq_mask[s]:
            continue
        off = int(seq_offset[s])
        nbytes = (hi - lo) * token_bytes
        if to_buffer:
            buffer[off:off + nbytes] = tb[lo:hi].reshape(-1)
        else:
            tb[lo:hi] = buffer[off:off + nbytes].reshape(hi - lo, token_bytes)


def copy_non_cp_tokenwise(tensor, buffer, seq_offset, seq_tokens, copy_seq_mask=None, to_buffer=True) -> None:
    """Literal restatement of the kernel's loop (memcpy.cu:33-73), one token at a time."""
    tb = _bytes2d(tensor)
    num_tokens, token_bytes = tb.shape
    seq_tokens = np.asarray(seq_tokens).tolist()
    cur_seq, cur_end, cur_start = 0, seq_tokens[0], 0
    for token_idx in range(num_tokens):
        while token_idx >= cur_end:
            cur_seq += 1
            cur_start = cur_end
            cur_end += seq_tokens[cur_seq]
        if to_buffer and copy_seq_mask is not None and not copy_seq_mask[cur_seq]:
            continue
        off = int(seq_offset[cur_seq]) + (token_idx - cur_start) * token_bytes
        if to_buffer:
            buffer[off:off + token_bytes] = tb[token_idx]
        else:
            tb[token_idx] = buffer[off:off + token_bytes]


def copy_cp(tensor: np.ndarray, buffer: np.ndarray, do_shard, seq_offset, seq_tokens, to_buffer: bool = True) -> None:
    """Packing: tensor [T, ...]; unpacking: tensor [max_cp, T, ...].  do_shard [S, max_cp],
    seq_offset [max_cp, S].  memcpy.cu:91-154: logical tokens run over (replica, shard,
    token); packing reads row (logical % T), unpacking writes row logical of the flattened
    [max_cp*T] tensor."""
    do_shard = np.asarray(do_shard)
    seq_offset = np.asarray(seq_offset)
    max_cp, num_seq = seq_offset.shape
    if to_buffer:
        tb = _bytes2d(tensor)
        num_tokens = tb.shape[0]
    else:
        tb = tensor.view(np.uint8).reshape(tensor.shape[0] * tensor.shape[1], int(np.prod(tensor.shape[2:])) * tensor.itemsize)
        num_tokens = tensor.shape[1]
    token_bytes = tb.shape[1]
    logical_total = num_tokens * max_cp
    logical = 0
    lens = np.asarray(seq_tokens).tolist()
    for cp in range(max_cp):
        for s, ln in enumerate(lens):
            lo, hi = logical, min(logical + ln, logical_total)
            logical += ln
            if hi <= lo or not do_shard[s, cp]:
                continue
            off = int(seq_offset[cp, s])
            for i, lg in enumerate(range(lo, hi)):  # row-wise: packing rows wrap modulo T
                b0 = off + i * token_bytes
                if to_buffer:
                    buffer[b0:b0 + token_bytes] = tb[lg % num_tokens]
                else:
                    tb[lg] = buffer[b0:b0 + token_bytes]


def grad_sum(data: torch.Tensor, num_copies, copy_start_id, seq_lens) -> None:
    """In place on a CPU torch tensor [T, hidden] of dtype fp32 / fp16 / bf16.

    memcpy.cu:176-233: for every shard with copies, main_row += copy_row for each copy in
    order, every addition rounded to the tensor dtype (torch CPU `+=` on half types adds in
    fp32 and rounds to nearest even, the same single rounding as the device `+=`)."""
    start = 0
    num_tokens = data.shape[0]
    for s, ln in enumerate([int(x) for x in seq_lens]):
        lo, hi = start, min(start + ln, num_tokens)
        start += ln
        n = int(num_copies[s])
        if n == 0 or hi <= lo:
            continue
        for c in range(n):
            c0 = int(copy_start_id[s][c])
            data[lo:hi] += data[c0:c0 + (hi - lo)]
