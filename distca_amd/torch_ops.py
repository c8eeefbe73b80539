"""The pack / unpack / duplicate-gradient ops as PyTorch custom ops, `torch.ops.distca_amd.*`.

The reference exposes its kernels as `torch.ops.dispatch_kernels.*`
(csrc/bindings/all_to_all.cpp:395-408, inside TORCH_LIBRARY(dispatch_kernels, m),
csrc/bindings/bindings.cpp:13-16); its Python wrappers (distca/runtime/attn_kernels/ops.py:153-215)
call the `_debug` forms when given an explicit buffer.  Importing this module registers ops of the
same names, schemas and argument order under the namespace `distca_amd`, bound to the HIP kernels,
so that code written against `torch.ops.dispatch_kernels.<op>` only changes the namespace.  They are
registered for device tensors only: a call with CPU tensors fails in the dispatcher, there is no
host path.  The handle-based forms (`fast_a2a_memcpy_non_cp(int fptr, ...)`) belong to the NVSHMEM
dispatcher and have no counterpart here.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import ops

NAMESPACE = "distca_amd"

SCHEMAS = {
    # csrc/bindings/all_to_all.cpp:102-113
    "fast_a2a_memcpy_non_cp_debug": "(Tensor(a!) tensor, Tensor seq_nvshmem_offset, Tensor seq_tokens, "
                                    "Tensor? copy_seq_mask, bool to_nvshmem, Tensor(b!) buffer) -> ()",
    # csrc/bindings/all_to_all.cpp:243-254
    "fast_a2a_memcpy_cp_debug": "(Tensor(a!) tensor, Tensor do_shard, Tensor seq_nvshmem_offset, Tensor seq_tokens, "
                                "bool to_nvshmem, Tensor(b!) buffer) -> ()",
    # csrc/bindings/all_to_all.cpp:182-240
    "fast_a2a_grad_acc": "(Tensor(a!) tensor, Tensor num_copies, Tensor copy_start_id, Tensor seq_lens) -> ()",
}


def _non_cp(tensor: torch.Tensor, seq_nvshmem_offset: torch.Tensor, seq_tokens: torch.Tensor,
            copy_seq_mask: Optional[torch.Tensor], to_nvshmem: bool, buffer: torch.Tensor) -> None:
    ops.a2a_memcpy_non_cp(tensor, seq_nvshmem_offset, seq_tokens, to_nvshmem, copy_seq_mask, buffer)


def _cp(tensor: torch.Tensor, do_shard: torch.Tensor, seq_nvshmem_offset: torch.Tensor, seq_tokens: torch.Tensor,
        to_nvshmem: bool, buffer: torch.Tensor) -> None:
    ops.a2a_memcpy_cp(tensor, do_shard, seq_nvshmem_offset, seq_tokens, to_nvshmem, buffer)


def _grad_acc(tensor: torch.Tensor, num_copies: torch.Tensor, copy_start_id: torch.Tensor, seq_lens: torch.Tensor) -> None:
    ops.pre_a2a_grad_acc(tensor, num_copies, copy_start_id, seq_lens)


_library = torch.library.Library(NAMESPACE, "DEF")
for _name, _schema in SCHEMAS.items():
    _library.define(_name + _schema)
_library.impl("fast_a2a_memcpy_non_cp_debug", _non_cp, "CUDA")   # the dispatch key of HIP devices in PyTorch-ROCm
_library.impl("fast_a2a_memcpy_cp_debug", _cp, "CUDA")
_library.impl("fast_a2a_grad_acc", _grad_acc, "CUDA")
