"""ctypes binding of libdistca_ca.so (the C ABI declared in include/distca_ca.h).

The library is the product: there is no Python or CPU fallback.  Importing this module
without a built library raises, and every wrapper turns a non-zero return code into a
RuntimeError carrying distca_last_error().
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdistca_ca.so")

ABI_VERSION = 4


class CaParams(Structure):
    """struct distca_ca_params (include/distca_ca.h)."""
    _fields_ = [
        ("num_tasks", c_int32), ("total_q", c_int32), ("total_k", c_int32),
        ("num_heads_q", c_int32), ("num_heads_kv", c_int32), ("head_dim", c_int32),
        ("max_seqlen_q", c_int32), ("max_seqlen_k", c_int32),
        ("softmax_scale", c_float), ("causal", c_int32), ("deterministic", c_int32),
        ("dtype", c_int32),
    ]


class PackJob(Structure):
    """struct distca_pack_job (include/distca_ca.h)."""
    _fields_ = [
        ("tensor", c_void_p), ("seq_offset", c_void_p), ("seq_tokens", c_void_p), ("copy_seq_mask", c_void_p),
        ("num_seq", c_int64), ("token_bytes", c_int64), ("num_tokens", c_int64),
    ]


class KvShards(Structure):
    """struct distca_kv_shards (include/distca_ca.h)."""
    _fields_ = [
        ("num_shards", c_int32), ("row_start", c_void_p), ("k_offset", c_void_p), ("v_offset", c_void_p),
        ("task_shard", c_void_p), ("dk_offset", c_void_p), ("dv_offset", c_void_p),
    ]


PACK_MAX_JOBS = 4

# name -> (restype, argtypes); every symbol include/distca_ca.h declares
SYMBOLS = {
    "distca_last_error": (c_char_p, []),
    "distca_abi_version": (c_int, []),
    "distca_memcpy_non_cp": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]),
    "distca_memcpy_non_cp_multi": (c_int, [POINTER(PackJob), c_int32, c_void_p, c_int, c_void_p]),
    "distca_memcpy_cp": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32, c_int64, c_int, c_void_p]),
    "distca_grad_sum": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "distca_ca_fwd_workspace_bytes": (c_int64, [POINTER(CaParams)]),
    "distca_ca_bwd_workspace_bytes": (c_int64, [POINTER(CaParams)]),
    "distca_ca_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                              POINTER(CaParams), c_void_p, c_int64, c_void_p]),
    "distca_ca_fwd_noalloc_max_bytes": (c_int64, []),
    "distca_ca_fwd_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      POINTER(CaParams), c_void_p]),
    "distca_ca_fwd_tokens": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                     c_void_p, c_void_p, c_void_p, POINTER(CaParams), c_void_p, c_int64, c_void_p]),
    "distca_ca_fwd_buffers": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, POINTER(KvShards), c_void_p, c_void_p, c_int64,
                                      c_void_p, c_void_p, c_void_p, c_void_p, POINTER(CaParams), c_void_p, c_int64, c_void_p]),
    "distca_ca_bwd_buffers": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, POINTER(KvShards), c_void_p, c_void_p, c_int64,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(CaParams), c_void_p, c_int64, c_void_p]),
    "distca_ca_bwd": (c_int, [c_void_p] * 9 + [c_void_p, c_void_p, c_void_p, POINTER(CaParams), c_void_p, c_int64, c_void_p]),
    "distca_ca_bwd_tokens": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                     c_void_p, c_void_p, c_void_p, POINTER(CaParams), c_void_p, c_int64, c_void_p]),
    "distca_ca_schedule_capacity": (c_int64, [c_int, POINTER(CaParams)]),
    "distca_ca_schedule_host": (c_int64, [c_int, c_void_p, c_void_p, POINTER(CaParams), c_void_p, c_int64]),
    "distca_timing_enable": (None, [c_int]),
    "distca_timing_read": (c_int, [c_int, POINTER(ctypes.c_double), POINTER(c_int64)]),
    "distca_ca_tile_shape": (c_int, [c_int, POINTER(CaParams), POINTER(c_int32 * 2)]),
    "distca_probe_mfma_rate": (c_int, [c_int, c_int, c_void_p, POINTER(ctypes.c_double), POINTER(ctypes.c_double),
                                       POINTER(ctypes.c_double), c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Loads the library once; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m distca_amd._build` (needs hipcc); "
            "distca_amd has no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SYMBOLS.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    if lib.distca_abi_version() != ABI_VERSION:
        raise RuntimeError(f"libdistca_ca.so ABI {lib.distca_abi_version()} != binding ABI {ABI_VERSION}: rebuild")
    _lib = lib
    return lib


TIMER_CA_FWD, TIMER_CA_BWD, TIMER_MEMCPY_NON_CP, TIMER_MEMCPY_CP, TIMER_GRAD_SUM, TIMER_CA_BWD_DQ = range(6)


def timing_enable(on: bool) -> None:
    load().distca_timing_enable(1 if on else 0)


def timing_read(which: int):
    """(total milliseconds, launches) of kernel `which` since the last read."""
    ms, n = ctypes.c_double(0), c_int64(0)
    check(load().distca_timing_read(which, ctypes.byref(ms), ctypes.byref(n)), "timing_read")
    return ms.value, n.value


PROBE_MFMA_ONLY, PROBE_LDS_READ, PROBE_FMA4, PROBE_EXP2, PROBE_MIX = range(5)


def probe_mfma_rate(kind: int, iters: int, scratch_ptr: int, stream_ptr: int = 0):
    """(TFLOP/s, cycles per MFMA, shader clock in GHz) of a loop of MFMAs on every SIMD of the device, with
    nothing (PROBE_MFMA_ONLY), an LDS read, four FMAs, two exponentials, or the attention backward's average side
    work (PROBE_MIX) behind every MFMA.  `scratch_ptr`: 32
    bytes of device memory.  Synchronises the stream."""
    tf, cyc, ghz = ctypes.c_double(0), ctypes.c_double(0), ctypes.c_double(0)
    check(load().distca_probe_mfma_rate(kind, iters, scratch_ptr, ctypes.byref(tf), ctypes.byref(cyc), ctypes.byref(ghz),
                                        stream_ptr), "probe_mfma_rate")
    return tf.value, cyc.value, ghz.value


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().distca_last_error()
        raise RuntimeError(f"{what} failed ({rc}): {msg.decode() if msg else ''}")
