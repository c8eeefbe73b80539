"""The C-ABI library loads without a GPU, exports every symbol include/distca_ca.h declares,
and rejects bad arguments on the host before anything is launched."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

from distca_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "distca_ca.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    return sorted(set(re.findall(r"\b(distca_[a-z0-9_]+)\s*\(", text)))


def test_header_compiles_as_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "distca_ca.h"\nint main(void) { distca_ca_params p; (void)p; return 0; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src),
                    "-o", str(tmp_path / "t.o")], check=True)


def test_every_declared_symbol_is_exported_and_bound():
    names = _declared_functions()
    assert len(names) >= 12
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} declared in distca_ca.h but not exported"
    assert set(names) == set(_lib.SYMBOLS), "ctypes table and header disagree"


def test_params_struct_layout_matches_header():
    text = open(HEADER).read()
    body = re.search(r"typedef struct distca_ca_params \{(.*?)\} distca_ca_params;", text, re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    body = re.sub(r"//[^\n]*", "", body)
    fields = re.findall(r"(int32_t|float)\s+([a-z_]+)\s*;", body)
    assert [f for _, f in fields] == [f for f, _ in _lib.CaParams._fields_]
    assert ctypes.sizeof(_lib.CaParams) == 4 * len(fields)


def test_abi_version_and_error_string():
    lib = _lib.load()
    assert lib.distca_abi_version() == _lib.ABI_VERSION
    assert isinstance(lib.distca_last_error(), bytes)


def _p(**kw):
    base = dict(num_tasks=1, total_q=16, total_k=16, num_heads_q=32, num_heads_kv=8, head_dim=128,
                max_seqlen_q=16, max_seqlen_k=16, softmax_scale=0.088, causal=1, deterministic=0, dtype=0)
    base.update(kw)
    return _lib.CaParams(*[base[f] for f, _ in _lib.CaParams._fields_])


@pytest.mark.parametrize("bad", [dict(head_dim=64), dict(num_heads_q=30), dict(num_heads_kv=0), dict(num_tasks=-1),
                                 dict(total_q=-5), dict(dtype=3), dict(dtype=-1)])
def test_unsupported_shapes_are_rejected_on_the_host(bad):
    lib = _lib.load()
    p = _p(**bad)
    assert lib.distca_ca_fwd_workspace_bytes(ctypes.byref(p)) < 0
    # validation precedes any device call: with null pointers the call must return an error code
    rc = lib.distca_ca_fwd(None, None, None, None, None, None, None, None, ctypes.byref(p), None, 0, None)
    assert rc in (-1, -2)
    assert lib.distca_last_error()


def test_workspace_sizes_are_positive_and_monotone():
    lib = _lib.load()
    # element type: 0 (callers from before the field existed) and DISTCA_DTYPE_BF16 = 2 mean bf16, 1 is fp16; same sizes
    sizes = {lib.distca_ca_bwd_workspace_bytes(ctypes.byref(_p(dtype=t))) for t in (0, 1, 2)}
    assert len(sizes) == 1 and min(sizes) > 0
    small = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(_p()))
    big = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(_p(total_q=131072, total_k=131072, num_tasks=27,
                                                              max_seqlen_q=65536, max_seqlen_k=65536)))
    assert 0 < small < big
    assert lib.distca_ca_fwd_workspace_bytes(ctypes.byref(_p())) > 0


def test_pack_argument_checks_need_no_gpu():
    lib = _lib.load()
    # token size not a multiple of 16 bytes: rejected as the reference rejects it (memcpy.cu:246)
    dummy = ctypes.create_string_buffer(64)        # host memory, never dereferenced: the size check comes first
    a = ctypes.addressof(dummy)
    assert lib.distca_memcpy_non_cp(a, a, a, a, None, 1, 24, 8, 1, None) < 0
    assert b"16" in lib.distca_last_error()
    assert lib.distca_memcpy_cp(a, a, a, a, a, 24, 8, 2, 1, 1, None) < 0
    assert b"16" in lib.distca_last_error()
    assert lib.distca_memcpy_non_cp(None, None, None, None, None, 1, 32, 8, 1, None) < 0
    assert b"null" in lib.distca_last_error()
    assert lib.distca_grad_sum(None, 99, None, None, None, 8, 128, 1, 1, None) < 0   # unknown dtype code
    # zero-sized problems are no-ops that never touch the device
    assert lib.distca_memcpy_non_cp(None, None, None, None, None, 0, 32, 0, 1, None) == 0


def test_timing_api_without_launches():
    lib = _lib.load()
    ms, n = ctypes.c_double(-1), ctypes.c_int64(-1)
    assert lib.distca_timing_read(99, ctypes.byref(ms), ctypes.byref(n)) < 0
    lib.distca_timing_enable(0)
    assert lib.distca_timing_read(0, ctypes.byref(ms), ctypes.byref(n)) == 0 and n.value == 0


def test_schedule_host_reports_needed_capacity():
    lib = _lib.load()
    cu = np.array([0, 1000], dtype=np.int32)
    p = _p(total_q=1000, total_k=1000, max_seqlen_q=1000, max_seqlen_k=1000)
    n = lib.distca_ca_schedule_host(0, cu.ctypes.data, cu.ctypes.data, ctypes.byref(p), None, 0)
    assert n > 0
    small = np.full((2, 4), -7, dtype=np.int32)
    # a short array receives the first max_items items; the full count is still returned
    assert lib.distca_ca_schedule_host(0, cu.ctypes.data, cu.ctypes.data, ctypes.byref(p), small.ctypes.data, 1) == n
    assert small[0, 0] == 0 and (small[1] == -7).all()


def test_attention_argument_errors_are_reported_before_any_launch():
    """Null, misaligned and undersized arguments come back as error codes with a message; the
    pointers are fake host addresses, so reaching a kernel launch would fail differently."""
    lib = _lib.load()
    buf = ctypes.create_string_buffer(4096)
    base = (ctypes.addressof(buf) + 255) // 256 * 256
    ptr = ctypes.c_void_p(base)
    odd = ctypes.c_void_p(base + 2)
    p = _p()
    need = lib.distca_ca_fwd_workspace_bytes(ctypes.byref(p))
    args = lambda **kw: [kw.get("q", ptr), ptr, ptr, ptr, ptr, ptr, ptr, None, ctypes.byref(p), kw.get("ws", ptr), kw.get("ws_bytes", need), None]
    assert lib.distca_ca_fwd(*args(ws_bytes=need - 1)) == -3
    assert b"workspace" in lib.distca_last_error()
    assert lib.distca_ca_fwd(*args(ws=None)) == -3
    assert lib.distca_ca_fwd(*args(q=odd)) == -1
    assert b"aligned" in lib.distca_last_error()
    assert lib.distca_ca_fwd(*args(q=None)) == -1
    # backward: deterministic together with shared KV rows is served (one work item owns a key block on behalf of every
    # task that reads it), so the call passes validation up to the workspace check, like the form without kv_task_offsets
    pd = _p(deterministic=1)
    needb = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(pd))
    bargs = [ptr] * 9 + [ptr, ptr, ptr, ctypes.byref(pd), ptr, 64, None]
    assert lib.distca_ca_bwd(*bargs) == -3
    assert b"workspace" in lib.distca_last_error()
    bargs[11] = None
    assert lib.distca_ca_bwd(*bargs) == -3
    bargs[14] = needb
    bargs[0] = odd
    assert lib.distca_ca_bwd(*bargs) == -1
    assert b"aligned" in lib.distca_last_error()
    # a batch without tasks or rows is a no-op that touches nothing
    assert lib.distca_ca_fwd(None, None, None, None, None, None, None, None, ctypes.byref(_p(num_tasks=0, total_q=0, total_k=0)), None, 0, None) == 0


def test_backward_workspace_is_sized_for_what_the_call_needs():
    """The work lists and the two row statistics, and nothing else, for a batch large enough to occupy the device or a
    deterministic one: 131072 tokens with 32 query heads need 34 MB.  Only a small batch whose caller allows float
    atomics (its key blocks are then cut into pieces) also brings the fp32 dK/dV accumulators."""
    lib = _lib.load()
    big = _p(num_tasks=27, total_q=131072, total_k=131072, num_heads_q=32, num_heads_kv=8, max_seqlen_q=65536, max_seqlen_k=65536)
    n = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(big))
    stats = 2 * 32 * 131072 * 4
    assert stats < n <= 40e6
    big.deterministic = 1
    assert lib.distca_ca_bwd_workspace_bytes(ctypes.byref(big)) == n
    cfg5 = _p(num_tasks=40, total_q=524288, total_k=524288, num_heads_q=64, num_heads_kv=8, max_seqlen_q=262144, max_seqlen_k=262144)
    assert lib.distca_ca_bwd_workspace_bytes(ctypes.byref(cfg5)) <= 2 * 64 * 524288 * 4 + 8e6
    small = _p(num_tasks=3, total_q=4096, total_k=4096, num_heads_q=32, num_heads_kv=8, max_seqlen_q=2560, max_seqlen_k=2560)
    pieces = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(small))
    small.deterministic = 1
    whole = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(small))
    assert pieces - whole >= 2 * 4096 * 8 * 128 * 4          # the two accumulators
    assert whole < 2 * 32 * 4096 * 4 + 1e6


def test_python_wrappers_reject_wrong_inputs():
    """The host layer raises RuntimeError for what the reference's C++ wrappers check
    (all_to_all.cpp:18-21, 47-99): device, rank, dtype of metadata."""
    import torch
    from distca_amd import ops
    from distca_amd.fused_comm_attn import ca_varlen_fwd
    t = torch.zeros((4, 8), dtype=torch.bfloat16)
    off = torch.zeros(1, dtype=torch.int64)
    with pytest.raises(AssertionError, match="DispatcherWrapper not initialized"):   # ops.py:112-115 of the reference
        ops.a2a_memcpy_non_cp(t, off, off, True)
    with pytest.raises(NotImplementedError):
        ops.DispatcherWrapper.init(0, 0, 2, 1024, device="cpu")
    ops.DispatcherWrapper.init(0, 0, 1, 1024, device="cpu")
    try:
        with pytest.raises(AssertionError, match="no all-to-all has filled"):
            ops.a2a_memcpy_non_cp(t, off, off, False, instance_id=0)
        ops.DispatcherWrapper.acquire(0)
        with pytest.raises(AssertionError, match="not released"):
            ops.a2a_memcpy_non_cp(t, off, off, True, instance_id=0)
        ops.DispatcherWrapper.release(0)
        ops.DispatcherWrapper.get_instance(0).send_buffer[:8] = torch.arange(8, dtype=torch.uint8)
        one = torch.ones((1, 1), dtype=torch.int64)
        ops.fast_a2a(one, one, one, one, 0, 16, 8, instance_id=0)
        assert ops.DispatcherWrapper.is_acquired[0]
        assert ops.DispatcherWrapper.get_instance(0).recv_buffer[16:24].tolist() == list(range(8))
        with pytest.raises(RuntimeError, match="do not fit"):
            ops.fast_a2a(one, one, one, one, 0, 1020, 8)
        assert ops.DispatcherWrapper.get_instance() is ops.DispatcherWrapper.instance[0]
        ops.DispatcherWrapper.switch_buffer()
        assert ops.DispatcherWrapper.get_instance() is ops.DispatcherWrapper.instance[1]
    finally:
        ops.DispatcherWrapper.instance = None
        ops.DispatcherWrapper.is_acquired = [False, False]
        ops.DispatcherWrapper.cur_instance = 0
    with pytest.raises(RuntimeError):
        ops.a2a_memcpy_non_cp(t, off.to(torch.int32), off, True, buffer=torch.zeros(64, dtype=torch.uint8))
    with pytest.raises(RuntimeError):
        ops.pre_a2a_grad_acc(t.to(torch.float64), off.to(torch.int32), off.reshape(1, 1), off)
    q = torch.zeros((4, 2, 128), dtype=torch.bfloat16)
    cu = torch.tensor([0, 4], dtype=torch.int32)
    with pytest.raises(RuntimeError, match="CUDA"):
        ca_varlen_fwd(q, q, q, cu, cu, 4, 4)


def test_token_layout_entry_points_check_their_layouts():
    """distca_ca_fwd_tokens / distca_ca_bwd_tokens refuse token sizes that cannot hold their parts, a
    missing lse destination, and (backward) head counts that put q off 16-byte alignment; all before
    any launch."""
    lib = _lib.load()
    ptr = ctypes.c_void_p(0x1000)
    p = _lib.CaParams(2, 64, 64, 8, 2, 128, 32, 32, 0.088, 1, 0, 0)
    need = lib.distca_ca_fwd_workspace_bytes(ctypes.byref(p))
    row = 8 * 128 * 2
    fwd = lambda **kw: lib.distca_ca_fwd_tokens(*[kw.get(n, d) for n, d in (
        ("q", ptr), ("q_off", ptr), ("q_tok", row), ("k", ptr), ("v", ptr), ("out", ptr), ("out_off", ptr), ("out_tok", row + 32),
        ("lse", None), ("cu_q", ptr), ("cu_k", ptr), ("kv_off", None), ("p", ctypes.byref(p)), ("ws", ptr), ("ws_bytes", 16), ("stream", None))])
    assert fwd() == -3 and b"workspace" in lib.distca_last_error()          # everything else is in order
    assert fwd(q_tok=row - 16) == -1 and b"query token" in lib.distca_last_error()
    assert fwd(out_tok=row) == -1 and b"output token" in lib.distca_last_error()   # no room for the lse
    assert fwd(out_tok=row + 8) == -1
    assert fwd(out_off=None, out_tok=0) == -1 and b"lse is null" in lib.distca_last_error()
    assert fwd(q=None) == -1
    assert need > 16
    needb = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(p))
    bwd = lambda **kw: lib.distca_ca_bwd_tokens(*[kw.get(n, d) for n, d in (
        ("req", ptr), ("req_off", ptr), ("req_tok", 3 * row + 32), ("k", ptr), ("v", ptr), ("dq", ptr), ("dq_off", ptr), ("dq_tok", row),
        ("dk", ptr), ("dv", ptr), ("cu_q", ptr), ("cu_k", ptr), ("kv_off", None), ("p", ctypes.byref(kw.get("params", p))), ("ws", ptr),
        ("ws_bytes", 64), ("stream", None))])
    assert bwd() == -3 and needb > 64
    assert bwd(req_tok=3 * row) == -1 and b"request token" in lib.distca_last_error()
    assert bwd(dq_tok=row - 16) == -1 and b"dq token" in lib.distca_last_error()
    assert bwd(req_off=None) == -1 and b"offset" in lib.distca_last_error()
    p6 = _lib.CaParams(2, 64, 64, 6, 2, 128, 32, 32, 0.088, 1, 0, 0)
    assert bwd(params=p6) == -2 and b"alignment" in lib.distca_last_error()
    # a server without a task this tick: empty (null) arrays everywhere, nothing to do, no error
    idle = _lib.CaParams(0, 0, 0, 8, 2, 128, 0, 0, 0.088, 1, 0, 0)
    nothing = dict(req=None, req_off=None, k=None, v=None, dq=None, dq_off=None, dk=None, dv=None, cu_q=None, cu_k=None, ws=None, ws_bytes=0)
    assert bwd(params=idle, **nothing) == 0
    p_save = p
    p = idle
    assert fwd(q=None, q_off=None, k=None, v=None, out=None, out_off=None, cu_q=None, cu_k=None, ws=None, ws_bytes=0) == 0
    p = p_save


def test_torch_ops_are_registered_for_device_tensors_only():
    """`torch.ops.distca_amd.*` carry the reference's op names and schemas
    (csrc/bindings/all_to_all.cpp:102-113,182-254) and have no host implementation."""
    import torch
    from distca_amd import torch_ops
    for name, schema in torch_ops.SCHEMAS.items():
        op = getattr(torch.ops.distca_amd, name)
        got = str(op.default._schema)
        assert got == f"distca_amd::{name}{schema}", got
    t = torch.zeros((4, 8), dtype=torch.bfloat16)
    i64 = torch.zeros(1, dtype=torch.int64)
    with pytest.raises(NotImplementedError):
        torch.ops.distca_amd.fast_a2a_memcpy_non_cp_debug(t, i64, i64, None, True, torch.zeros(64, dtype=torch.uint8))
    with pytest.raises(NotImplementedError):
        torch.ops.distca_amd.fast_a2a_grad_acc(t, torch.zeros(1, dtype=torch.int32), torch.zeros((1, 1), dtype=torch.int64), i64)
