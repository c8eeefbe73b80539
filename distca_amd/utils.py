"""Small host helpers shared by the op wrappers (same names and meaning as
distca/runtime/utils.py:8-35 in the reference)."""
from __future__ import annotations

import torch

_INT4_BYTES = 16


def size_pad_by_int4(hidden_size: int, itemsize: int):
    """(padded element count, pad element count) so that a row is a multiple of 16 bytes."""
    hidden_bytes = hidden_size * itemsize
    if hidden_bytes % _INT4_BYTES != 0:
        hidden_bytes += _INT4_BYTES - (hidden_bytes % _INT4_BYTES)
    hidden_size_pad = hidden_bytes // itemsize
    return hidden_size_pad, hidden_size_pad - hidden_size


def prepend_zero_fn(tensor: torch.Tensor, dim: int = 0):
    zero = torch.zeros_like(tensor.select(dim, 0)).unsqueeze(dim)
    return torch.cat([zero, tensor], dim=dim)


def exclusive_cumsum(tensor: torch.Tensor, dim: int = 0) -> torch.Tensor:
    cumsum = tensor.cumsum(dim=dim)
    zero = torch.zeros_like(tensor.select(dim, 0))
    return torch.cat([zero.unsqueeze(dim), cumsum.narrow(dim, 0, cumsum.size(dim) - 1)], dim=dim)
