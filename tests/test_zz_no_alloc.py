"""distca_ca_fwd_noalloc (the forward over the library's static device scratch array) against distca_ca_fwd with a
caller workspace, through the C ABI: same kernels, so out and lse must agree bit for bit.  Two calls in a row on the
same GPU, the second with a smaller batch, so that what the first call left in the array would show."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import cu, make_qkv

pytestmark = pytest.mark.gpu


def _both(lib, CaParams, cuda, q_lens, k_lens, hq, hkv, seed, kv_off=None, total_k=None):
    cu_q, cu_k = cu(q_lens), cu(k_lens)
    tq, tk = int(cu_q[-1]), int(total_k if total_k is not None else cu_k[-1])
    q, k, v, _ = (t.to(cuda) for t in make_qkv(tq, tk, hq, hkv, 128, seed))
    dq_, dk_ = torch.tensor(cu_q, device=cuda), torch.tensor(cu_k, device=cuda)
    off = torch.tensor(np.asarray(kv_off, dtype=np.int32), device=cuda) if kv_off is not None else None
    p = CaParams(len(q_lens), tq, tk, hq, hkv, 128, int(max(q_lens)), int(max(k_lens)), 128 ** -0.5, 1, 0, 0)
    need = lib.distca_ca_fwd_workspace_bytes(ctypes.byref(p))
    assert 0 < need <= lib.distca_ca_fwd_noalloc_max_bytes()
    res = []
    for noalloc in (False, True):
        out = torch.full_like(q, float("nan"))
        lse = torch.full((hq, tq), float("nan"), dtype=torch.float32, device=cuda)
        args = [q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), lse.data_ptr(), dq_.data_ptr(), dk_.data_ptr(),
                off.data_ptr() if off is not None else None, ctypes.byref(p)]
        stream = torch.cuda.current_stream().cuda_stream
        print(f"  forward noalloc={noalloc} q_lens={list(q_lens)} heads {hq}/{hkv}", flush=True)
        if noalloc:
            rc = lib.distca_ca_fwd_noalloc(*args, stream)
        else:
            ws = torch.empty(need, dtype=torch.uint8, device=cuda)
            rc = lib.distca_ca_fwd(*args, ws.data_ptr(), need, stream)
        assert rc == 0, lib.distca_last_error()
        torch.cuda.synchronize()
        res.append((out, lse))
    (o0, l0), (o1, l1) = res
    assert torch.isfinite(o1.float()).all()
    assert torch.equal(o0.view(torch.int16), o1.view(torch.int16)), "out differs from the workspace form"
    assert torch.equal(l0.view(torch.int32), l1.view(torch.int32)), "lse differs from the workspace form"


def test_noalloc_forward_equals_workspace_forward_twice(cuda):
    from distca_amd._lib import CaParams, load
    lib = load()
    # a larger batch first (prefix tasks, 32q/8kv heads), then a smaller one with another head layout: the second
    # call finds the first call's work list, zero row and ticket counters in the array
    _both(lib, CaParams, cuda, [700, 1, 257, 1200, 64], [700, 300, 257, 2000, 64], 32, 8, 5)
    _both(lib, CaParams, cuda, [130, 33], [130, 33], 8, 2, 6)
    # tasks over one stored K/V copy, and once more the first shape
    _both(lib, CaParams, cuda, [200, 150, 250], [200, 350, 600], 8, 2, 7, kv_off=[0, 0, 0], total_k=600)
    _both(lib, CaParams, cuda, [700, 1, 257, 1200, 64], [700, 300, 257, 2000, 64], 32, 8, 8)


def test_noalloc_forward_rejects_a_batch_beyond_the_array(cuda):
    from distca_amd._lib import CaParams, load
    lib = load()
    # 70 000 tasks alone need more than 1 MiB of list: rejected on the host, nothing launched
    n = 70000
    p = CaParams(n, n, n, 8, 2, 128, 1, 1, 128 ** -0.5, 1, 0, 0)
    assert lib.distca_ca_fwd_workspace_bytes(ctypes.byref(p)) > lib.distca_ca_fwd_noalloc_max_bytes()
    dummy = torch.zeros(64, dtype=torch.uint8, device=cuda)
    ptr = dummy.data_ptr()
    rc = lib.distca_ca_fwd_noalloc(ptr, ptr, ptr, ptr, ptr, ptr, ptr, None, ctypes.byref(p), None)
    assert rc == -3 and b"static array" in lib.distca_last_error()
