"""Host mirror of the tile scheduler the attention kernels build on device.

distca_ca_schedule_host runs the same cost functions and the same bin sort as the device
builder, on host arrays, so the balance invariants can be checked without a GPU.  The
reference has no GPU-side scheduler (flash-attn launches a static grid); the cost unit is
the causal-pair count its planner balances across ranks (distca/planner/planner.py:366-378).
"""
from __future__ import annotations

import ctypes
from typing import Sequence, Tuple

import numpy as np

from . import _lib

FWD, BWD = 0, 1


def _params(cu_q, cu_k, hq, hkv, d, causal, deterministic=False) -> _lib.CaParams:
    cu_q = np.asarray(cu_q, dtype=np.int64)
    cu_k = np.asarray(cu_k, dtype=np.int64)
    lq, lk = np.diff(cu_q), np.diff(cu_k)
    return _lib.CaParams(len(lq), int(cu_q[-1]), int(cu_k[-1]), hq, hkv, d,
                         int(lq.max()) if len(lq) else 0, int(lk.max()) if len(lk) else 0,
                         float(d) ** -0.5, 1 if causal else 0, 1 if deterministic else 0, 0)


def tile_shape(kind: int, hq: int, hkv: int, d: int = 128) -> Tuple[int, int]:
    """(flattened query rows per block, keys per block) of the kernels of `kind`."""
    p = _lib.CaParams(1, 1, 1, hq, hkv, d, 1, 1, 1.0, 1, 0, 0)
    out = (ctypes.c_int32 * 2)()
    _lib.check(_lib.load().distca_ca_tile_shape(kind, ctypes.byref(p), ctypes.byref(out)), "tile_shape")
    return int(out[0]), int(out[1])


DQ = 2  # a third list kind for capacity queries: the dQ kernel's blocks of query rows


def schedule_capacity(kind: int, cu_seqlens_q: Sequence[int], cu_seqlens_k: Sequence[int], num_heads_q: int,
                      num_heads_kv: int, head_dim: int = 128, causal: bool = True, deterministic: bool = False,
                      total_k: int | None = None) -> int:
    """Room, in items, of the work list an attention call reserves in its workspace for this batch (sized on
    the host from total_q, total_k, max_seqlen_* and the task count alone).  `total_k` overrides the sum of the
    key lengths: tasks that share stored K/V rows (kv_task_offsets) have fewer rows than their lengths add up to."""
    p = _params(cu_seqlens_q, cu_seqlens_k, num_heads_q, num_heads_kv, head_dim, causal, deterministic)
    if total_k is not None:
        p.total_k = int(total_k)
    n = _lib.load().distca_ca_schedule_capacity(kind, ctypes.byref(p))
    if n < 0:
        _lib.check(int(n), "schedule_capacity")
    return int(n)


def build_schedule(kind: int, cu_seqlens_q: Sequence[int], cu_seqlens_k: Sequence[int], num_heads_q: int,
                   num_heads_kv: int, head_dim: int = 128, causal: bool = True, deterministic: bool = False,
                   total_k: int | None = None) -> np.ndarray:
    """Work items as an int32 array [n, 4] of (task, block, cost, piece | pieces << 16), most expensive
    first; in a backward list bit 31 of the fourth word (WALK_UP) marks items walked upwards from the diagonal
    (`item_piece`, `item_pieces` take the word apart).  Backward items of a batch too small to occupy the device are cut into pieces of
    consecutive query blocks unless `deterministic`; everything else has pieces = 1, piece = 0."""
    cu_q = np.ascontiguousarray(cu_seqlens_q, dtype=np.int32)
    cu_k = np.ascontiguousarray(cu_seqlens_k, dtype=np.int32)
    p = _params(cu_q, cu_k, num_heads_q, num_heads_kv, head_dim, causal, deterministic)
    if total_k is not None:
        p.total_k = int(total_k)
    lib = _lib.load()
    n = lib.distca_ca_schedule_host(kind, cu_q.ctypes.data, cu_k.ctypes.data, ctypes.byref(p), None, 0)
    if n < 0:
        _lib.check(int(n), "build_schedule")
    items = np.zeros((int(n), 4), dtype=np.int32)
    if n:
        m = lib.distca_ca_schedule_host(kind, cu_q.ctypes.data, cu_k.ctypes.data, ctypes.byref(p), items.ctypes.data, int(n))
        assert m == n
    return items


WALK_UP = -(1 << 31)   # bit 31 of an item's fourth word, as int32


def item_piece(w):
    return w & 0xffff


def item_pieces(w):
    return (w >> 16) & 0x7fff


def whole_items(items: np.ndarray) -> np.ndarray:
    """[m, 3] (task, block, cost) with the pieces of every block put together again, most expensive first."""
    total = {}
    for t, b, c, _ in items.tolist():
        total[(t, b)] = total.get((t, b), 0) + c
    out = np.array([(t, b, c) for (t, b), c in total.items()], dtype=np.int32).reshape(-1, 3)
    return out[np.argsort(-out[:, 2], kind="stable")] if len(out) else out
