"""Host helpers shared by the op wrappers.  The three public names and their meaning are those of
distca/runtime/utils.py:8-35 in the reference, so that code written against it keeps working."""
from __future__ import annotations

import torch

TRANSPORT_ALIGN = 16  # bytes: one 128-bit vector, the unit the pack kernels move


def round_up(n: int, unit: int = TRANSPORT_ALIGN) -> int:
    return -(-int(n) // unit) * unit


def size_pad_by_int4(hidden_size: int, itemsize: int):
    """A token row of `hidden_size` elements of `itemsize` bytes, padded so that the row is a whole number of
    128-bit vectors: returns (padded element count, elements of padding)."""
    padded = round_up(hidden_size * itemsize) // itemsize
    return padded, padded - hidden_size


def prepend_zero_fn(tensor: torch.Tensor, dim: int = 0) -> torch.Tensor:
    """`tensor` with one zero slice put in front along `dim` (a cumulative sum turned into cu_seqlens)."""
    shape = list(tensor.shape)
    shape[dim] = 1
    return torch.cat((tensor.new_zeros(shape), tensor), dim=dim)


def exclusive_cumsum(tensor: torch.Tensor, dim: int = 0) -> torch.Tensor:
    """Sum of the elements before each position along `dim`: the inclusive sum less the element itself."""
    return tensor.cumsum(dim=dim) - tensor
