"""Full-size runs of the benchmark workloads, checked through properties that do not need the
full fp32 oracle (which would take hours on host cores at these sizes):

  * sampled query rows against the oracle (out, lse, dq for those rows over the whole prefix);
  * sampled key rows against the oracle (dk, dv of those keys from every query row that sees them, summed
    over the tasks that share the stored row);
  * <V, dV> = <O, dO>  (O is linear in V) and  <Q, dQ> = <K, dK>  (scores depend on Q K^T only,
    so scaling Q or K by 1+eps moves the loss equally), per kv head;
  * two runs give bit-identical results (no atomics anywhere in the unaliased path);
  * a document served as prefix tasks equals the same document served whole;
  * the schedule the device built is the one the host mirror predicts.
"""
import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, assert_identity, randn_bf16, task_sums
from oracle.attention import ca_reference_key_rows, ca_reference_rows

pytestmark = pytest.mark.gpu


def _dev_inputs(batch, hq, hkv, cuda, seed):
    """Seeded N(0,1) bf16 inputs generated on the device (host generation of 10^9 values is slow)."""
    d = 128
    tq, tk = batch.total_q, batch.kv_rows
    g = torch.Generator(device=cuda).manual_seed(seed)
    rnd = lambda *shape: torch.randn(shape, generator=g, device=cuda, dtype=torch.float32).to(torch.bfloat16)
    q, k, v, do = rnd(tq, hq, d), rnd(tk, hkv, d), rnd(tk, hkv, d), rnd(tq, hq, d)
    cu_q = torch.tensor(batch.cu_seqlens_q, dtype=torch.int32, device=cuda)
    cu_k = torch.tensor(batch.cu_seqlens_k, dtype=torch.int32, device=cuda)
    return q, k, v, do, cu_q, cu_k


def _fwd_bwd(batch, hq, hkv, cuda, seed=0):
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    q, k, v, do, cu_q, cu_k = _dev_inputs(batch, hq, hkv, cuda, seed)
    mq, mk = int(max(batch.q_lens)), int(max(batch.k_lens))
    out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mk)
    dq, dk, dv = ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mk)
    torch.cuda.synchronize()
    return q, k, v, do, out, lse, dq, dk, dv


def _rows_ref(batch, q, k, v, do, t, r0, r1, out=None, lse=None):
    """Oracle (out, lse, dq) of rows [r0, r1) of task t; only that task's slices leave the device."""
    q0, q1 = int(batch.cu_seqlens_q[t]), int(batch.cu_seqlens_q[t + 1])
    k0, k1 = int(batch.cu_seqlens_k[t]), int(batch.cu_seqlens_k[t + 1])
    k1 -= (q1 - q0) - r1            # keys beyond the last sampled row's horizon are masked anyway
    q1 = q0 + r1
    return ca_reference_rows(q[q0:q1].cpu(), k[k0:k1].cpu(), v[k0:k1].cpu(), None if do is None else do[q0:q1].cpu(),
                             [0, q1 - q0], [0, k1 - k0], 0, r0, r1,
                             out_rows=None if out is None else out[q0 + r0:q0 + r1].cpu(),
                             lse_rows=None if lse is None else lse[:, q0 + r0:q0 + r1].cpu())


def _check_sampled_rows(batch, q, k, v, do, out, lse, dq, rng, n_samples=6, rows=16):
    lens = np.asarray(batch.q_lens)
    tasks = list(np.argsort(lens)[-2:]) + list(rng.choice(len(lens), size=n_samples - 2))
    for t in tasks:
        lq = int(lens[t])
        if lq == 0:
            continue
        r0 = int(rng.integers(0, max(1, lq - rows + 1)))
        r1 = min(lq, r0 + rows)
        if t == tasks[0]:
            r0, r1 = lq - min(rows, lq), lq                   # the longest rows of the longest task
        # the gradient oracle consumes the (out, lse) the backward kernel was handed
        o_ref, l_ref, dq_ref = _rows_ref(batch, q, k, v, do, int(t), r0, r1, out, lse)
        g0 = int(batch.cu_seqlens_q[t]) + r0
        sl = slice(g0, g0 + (r1 - r0))
        print(f"  rows task={t} [{r0},{r1}) of {lq}", flush=True)
        assert_close_bf16(out[sl], o_ref, f"out task {t}")
        assert (lse[:, sl].cpu() - l_ref).abs().max().item() <= 2e-3
        assert_close_bf16(dq[sl], dq_ref, f"dq task {t}")


def _rows_ref_group(batch, q, k, v, do, out, lse, t, r0, r1, kvh, g):
    """Oracle (out, lse, dq) of rows [r0, r1) of task t for the g query heads of kv head kvh only: with 64 query
    heads and a prefix of 262144 keys the full-width evaluation would hold 17 GB of repeated K/V on the host."""
    q0 = int(batch.cu_seqlens_q[t])
    lq, lk = int(batch.q_lens[t]), int(batch.k_lens[t])
    k0 = int(batch.kv_task_offsets[t]) if batch.kv_task_offsets is not None else int(batch.cu_seqlens_k[t])
    kvis = r1 + (lk - lq)                  # keys beyond the last sampled row's horizon are masked anyway
    hs = slice(kvh * g, (kvh + 1) * g)
    return ca_reference_rows(q[q0:q0 + r1, hs].cpu(), k[k0:k0 + kvis, kvh:kvh + 1].cpu(), v[k0:k0 + kvis, kvh:kvh + 1].cpu(),
                             do[q0:q0 + r1, hs].cpu(), [0, r1], [0, kvis], 0, r0, r1,
                             out_rows=out[q0 + r0:q0 + r1, hs].cpu(), lse_rows=lse[hs, q0 + r0:q0 + r1].cpu())


def _check_rows_of_group(batch, q, k, v, do, out, lse, dq, t, r0, r1, kvh, g):
    o_ref, l_ref, dq_ref = _rows_ref_group(batch, q, k, v, do, out, lse, t, r0, r1, kvh, g)
    q0 = int(batch.cu_seqlens_q[t])
    sl, hs = slice(q0 + r0, q0 + r1), slice(kvh * g, (kvh + 1) * g)
    print(f"  rows task={t} [{r0},{r1}) of {int(batch.q_lens[t])}, prefix {int(batch.k_lens[t])}, kv head {kvh}", flush=True)
    assert_close_bf16(out[sl, hs], o_ref, f"out task {t}")
    assert (lse[hs, sl].cpu() - l_ref).abs().max().item() <= 2e-3
    assert_close_bf16(dq[sl, hs], dq_ref, f"dq task {t}")


def _check_key_rows(batch, q, k, v, do, out, lse, dk, dv, row0, n, kvh, g):
    """dk, dv of stored K/V rows [row0, row0 + n) of kv head kvh against the oracle: the sum, over every task whose
    prefix holds the rows, of the contributions of that task's query rows that see them."""
    d = q.shape[2]
    ref_k, ref_v = torch.zeros(n, d), torch.zeros(n, d)
    hs = slice(kvh * g, (kvh + 1) * g)
    used = []
    for t in range(len(batch.q_lens)):
        lq, lk = int(batch.q_lens[t]), int(batch.k_lens[t])
        k0 = int(batch.kv_task_offsets[t]) if batch.kv_task_offsets is not None else int(batch.cu_seqlens_k[t])
        lo, hi = max(row0, k0), min(row0 + n, k0 + lk)          # stored rows of the sample inside this task's prefix
        if lo >= hi or lq == 0:
            continue
        j0 = lo - k0
        first = max(0, j0 - (lk - lq))                           # rows before it see none of the keys
        if first >= lq:
            continue
        q0 = int(batch.cu_seqlens_q[t])
        rows = slice(q0 + first, q0 + lq)
        gk, gv = ca_reference_key_rows(q[rows, hs].cpu(), do[rows, hs].cpu(), out[rows, hs].cpu(), lse[hs, rows].cpu(),
                                       k[lo:hi, kvh].cpu(), v[lo:hi, kvh].cpu(), first, lq, lk, j0)
        ref_k[lo - row0:hi - row0] += gk
        ref_v[lo - row0:hi - row0] += gv
        used.append((t, lq - first))
    print(f"  keys stored rows [{row0},{row0 + n}) kv head {kvh}: (task, query rows) {used}", flush=True)
    assert_close_bf16(dk[row0:row0 + n, kvh], ref_k, f"dk rows {row0}")
    assert_close_bf16(dv[row0:row0 + n, kvh], ref_v, f"dv rows {row0}")


def test_config2_llama8b_128k_properties(cuda):
    """The benchmark workload at full size: 131072 packed tokens, 32q/8kv heads."""
    from distca_amd import workloads
    b = workloads.config2_llama8b_128k()
    print("cfg2 fwd+bwd", flush=True)
    q, k, v, do, out, lse, dq, dk, dv = _fwd_bwd(b, 32, 8, cuda)
    for name, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert torch.isfinite(t.float()).all(), name
    _check_sampled_rows(b, q, k, v, do, out, lse, dq, np.random.default_rng(0))
    # dk / dv of sampled keys: the first, a middle and the last keys of the longest document, all keys of a short one
    big = int(np.argmax(b.q_lens))
    k_big, n_big = int(b.cu_seqlens_k[big]), int(b.k_lens[big])
    small = int(np.argmin(b.q_lens))
    # (32 rows of 128 values per sample: the mean relative error of a thousand values scatters by a tenth of itself)
    for row0, n, kvh in ((k_big, 32, 0), (k_big + n_big // 2 + 77, 32, 5), (k_big + n_big - 32, 32, 7),
                         (int(b.cu_seqlens_k[small]), 32, 3), (int(b.cu_seqlens_k[small]) + int(b.k_lens[small]) - 32, 32, 2)):
        _check_key_rows(b, q, k, v, do, out, lse, dk, dv, row0, n, kvh, 4)
    # linearity identities per (task, kv head)
    cu = b.cu_seqlens_q
    assert_identity(task_sums(v, dv, cu, 8), task_sums(out, do, cu, 8), "<V,dV> = <O,dO>")
    assert_identity(task_sums(q, dq, cu, 8), task_sums(k, dk, cu, 8), "<Q,dQ> = <K,dK>")
    print("cfg2 second run (bit reproducibility)", flush=True)
    again = _fwd_bwd(b, 32, 8, cuda)
    for name, x, y in zip(("out", "lse", "dq", "dk", "dv"), (out, lse, dq, dk, dv), again[4:]):
        assert torch.equal(x, y), f"{name} differs between two identical runs"


def test_config5_llama70b_heads_fwd_bwd_full_size(cuda):
    """BASELINE config 5 as stated: 524288 packed tokens, one 262144-token document among lognormal ones, 64q/8kv heads,
    forward and backward.  The backward at this size has 65536 query blocks per key block (the cost bins use a shift)
    and a group of 8 heads per kv head.  Checked: sampled rows of out, lse, dq (the last rows of the long document
    among them) and sampled key rows of dk, dv (first, middle, last keys of the long document; a short document)
    against the oracle for one head group each, and the two linearity identities over every (task, kv head)."""
    from distca_amd import workloads
    b = workloads.config5_llama70b_skewed()
    print("cfg5 fwd+bwd", flush=True)
    q, k, v, do, out, lse, dq, dk, dv = _fwd_bwd(b, 64, 8, cuda, seed=40)
    for name, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert torch.isfinite(t.float()).all(), name
    big = int(np.argmax(b.q_lens))
    n_big = int(b.q_lens[big])
    short = 0 if big else 1
    g = 8
    for t, r0, kvh in ((big, n_big - 8, 6), (big, 100000, 1), (big, 0, 4), (short, max(0, int(b.q_lens[short]) - 8), 2)):
        _check_rows_of_group(b, q, k, v, do, out, lse, dq, t, r0, min(int(b.q_lens[t]), r0 + 8), kvh, g)
    k_big = int(b.cu_seqlens_k[big])
    for row0, kvh in ((k_big, 3), (k_big + 100000, 1), (k_big + n_big - 32, 6), (int(b.cu_seqlens_k[short]), 2)):
        _check_key_rows(b, q, k, v, do, out, lse, dk, dv, row0, 32, kvh, g)
    cu = b.cu_seqlens_q
    assert_identity(task_sums(v, dv, cu, 8), task_sums(out, do, cu, 8), "<V,dV> = <O,dO>")
    assert_identity(task_sums(q, dq, cu, 8), task_sums(k, dk, cu, 8), "<Q,dQ> = <K,dK>")


@pytest.mark.parametrize("variant", ["a", "b"])
def test_config3_ca_tasks_full_size(cuda, variant):
    """BASELINE config 3 at full size: 262144 query rows cut into CA tasks from 8 documents of up to 524288 tokens whose
    K/V is stored once per document and read through kv_task_offsets (variant a: 64 tasks of 4096 rows; variant b:
    chunks uniform in [4096, 32768]).  Sampled rows of out, lse, dq; sampled stored key rows of dk, dv, whose
    reference is the sum over the tasks that read them; the linearity identities over the batch per kv head."""
    from distca_amd import workloads
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    b = workloads.config3_ca_tasks(variant=variant)
    q, k, v, do, cu_q, cu_k = _dev_inputs(b, 32, 8, cuda, 60)
    kv_off = torch.tensor(b.kv_task_offsets, dtype=torch.int32, device=cuda)
    mq, mk = int(max(b.q_lens)), int(max(b.k_lens))
    print(f"cfg3{variant} full size: {len(b.q_lens)} tasks, {b.total_q} query rows, kv rows {b.kv_rows}, longest prefix {mk}", flush=True)
    out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mk, kv_task_offsets=kv_off)
    # deterministic, as the reference's server is unless told otherwise (fused_comm_attn.py:95-104 of the reference)
    dq, dk, dv = ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mk, deterministic=True, kv_task_offsets=kv_off)
    torch.cuda.synchronize()
    for name, t in (("out", out), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert torch.isfinite(t.float()).all(), name
    if variant == "b":
        print("second run (bit reproducibility)", flush=True)
        again = ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mk, deterministic=True, kv_task_offsets=kv_off)
        torch.cuda.synchronize()
        for name, x, y in zip(("dq", "dk", "dv"), (dq, dk, dv), again):
            assert torch.equal(x, y), f"{name} differs between two deterministic runs"
        del again
    rng = np.random.default_rng(2)
    longest = int(np.argmax(b.k_lens))
    tasks = [longest] + [int(t) for t in rng.choice(len(b.q_lens), size=3, replace=False)]
    for i, t in enumerate(tasks):
        lq = int(b.q_lens[t])
        r0 = lq - 8 if i == 0 else int(rng.integers(0, lq - 8))
        _check_rows_of_group(b, q, k, v, do, out, lse, dq, t, r0, r0 + 8, int(rng.integers(8)), 4)
    # stored key rows: inside the query chunk of the task with the longest prefix (its diagonal), at the start of
    # its document (read by every task of the document), and two more drawn from rows some task queries
    k0, lk, lq = int(b.kv_task_offsets[longest]), int(b.k_lens[longest]), int(b.q_lens[longest])
    # 64 stored rows per sample: these gradients are small everywhere (1e-5 .. 1e-2), so they are held to the mean
    # relative error alone, which over the 1024 values of an 8-row sample scatters around the tolerance
    ns = 64
    samples = [(k0 + lk - lq + lq // 2, 1), (k0, 4), (k0 + lk - ns, 7)]
    for t in tasks[1:3]:
        kk, ll, qq = int(b.kv_task_offsets[t]), int(b.k_lens[t]), int(b.q_lens[t])
        samples.append((kk + ll - qq + int(rng.integers(0, qq - ns)), int(rng.integers(8))))
    for row0, kvh in samples:
        _check_key_rows(b, q, k, v, do, out, lse, dk, dv, row0, ns, kvh, 4)
    whole_q, whole_k = [0, b.total_q], [0, b.kv_rows]
    assert_identity(task_sums(q, dq, whole_q, 8), task_sums(k, dk, whole_k, 8), "<Q,dQ> = <K,dK>")
    assert_identity(task_sums(v, dv, whole_k, 8), task_sums(out, do, whole_q, 8), "<V,dV> = <O,dO>")


def test_prefix_tasks_equal_whole_document(cuda):
    """One 24576-token document as 6 CA tasks over a shared KV copy == the document served whole,
    forward and backward (dK/dV of the shared rows are summed across tasks on device)."""
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    n, hq, hkv = 24576, 32, 8
    cuts = [0, 2048, 6144, 7000, 13000, 20480, n]
    q = randn_bf16((n, hq, 128), 1).to(cuda); k = randn_bf16((n, hkv, 128), 2).to(cuda)
    v = randn_bf16((n, hkv, 128), 3).to(cuda); do = randn_bf16((n, hq, 128), 4).to(cuda)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=cuda)
    whole = i32([0, n])
    print("whole document", flush=True)
    out_w, lse_w = ca_varlen_fwd(q, k, v, whole, whole, n, n)
    dq_w, dk_w, dv_w = ca_varlen_bwd(do, q, k, v, out_w, lse_w, whole, whole, n, n)
    cu_q = i32(cuts)
    cu_k = i32([0] + list(np.cumsum(cuts[1:])))           # task i sees keys [0, cuts[i+1])
    kv_off = i32([0] * (len(cuts) - 1))
    print("prefix tasks", flush=True)
    mq, mk = int(np.diff(cuts).max()), n
    out_s, lse_s = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mk, kv_task_offsets=kv_off)
    dq_s, dk_s, dv_s = ca_varlen_bwd(do, q, k, v, out_s, lse_s, cu_q, cu_k, mq, mk, kv_task_offsets=kv_off)
    torch.cuda.synchronize()
    assert_close_bf16(out_s, out_w.float(), "out")
    assert (lse_s - lse_w).abs().max().item() <= 2e-3
    assert_close_bf16(dq_s, dq_w.float(), "dq", max_abs=3e-2)
    assert_close_bf16(dk_s, dk_w.float(), "dk", max_abs=3e-2)
    assert_close_bf16(dv_s, dv_w.float(), "dv", max_abs=3e-2)
    # a batch of this size is not cut into pieces, so dK/dV of the shared rows are summed by the work item that owns the
    # key block, in registers: the deterministic switch changes nothing, and a second run gives the same bits
    print("prefix tasks, deterministic", flush=True)
    det = ca_varlen_bwd(do, q, k, v, out_s, lse_s, cu_q, cu_k, mq, mk, deterministic=True, kv_task_offsets=kv_off)
    torch.cuda.synchronize()
    for name, x, y in zip(("dq", "dk", "dv"), (dq_s, dk_s, dv_s), det):
        assert torch.equal(x, y), f"{name}: the deterministic switch changed the result of a batch that is never cut"


def test_device_walk_marks_equal_host_mirror_with_many_equal_documents(cuda):
    """A hundred documents of one length: every cost bin of the dK/dV list holds a hundred entries, more than the
    builder ranks against each other, so all entries of a bin take the mark of its first one; a second batch of
    distinct lengths, where every entry is ranked.  The device list carries the marks of the host mirror, entry by
    entry (as sets: entries of one bin may come in any order), and is the same in a second run."""
    from distca_amd import scheduler, workloads
    from distca_amd._lib import CaParams, load
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    import ctypes
    hq, hkv = 8, 8
    for lens in ([1536] * 100, list(range(300, 300 + 37 * 60, 37))):
        ql = np.asarray(lens, dtype=np.int64)
        b = workloads.TaskBatch("walk_marks", ql, ql, hq, hkv)
        q, k, v, do, cu_q, cu_k = _dev_inputs(b, hq, hkv, cuda, 5)
        mq = int(ql.max())
        p = CaParams(len(ql), b.total_q, b.kv_rows, hq, hkv, 128, mq, mq, 128 ** -0.5, 1, 1, 0)
        nbytes = load().distca_ca_bwd_workspace_bytes(ctypes.byref(p))
        host = scheduler.build_schedule(scheduler.BWD, b.cu_seqlens_q, b.cu_seqlens_k, hq, hkv, deterministic=True)
        assert (host[:, 3] < 0).any() and (host[:, 3] > 0).any()
        header = (4 + len(ql) + 1 + 3) // 4 * 4
        lists = []
        for run in range(2):
            ws = torch.zeros((nbytes,), dtype=torch.uint8, device=cuda)
            out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mq)
            ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mq, None, True, True, None, workspace=ws)
            torch.cuda.synchronize()
            w = ws.cpu().view(torch.int32).numpy()
            assert int(w[0]) == len(host) and int(w[2]) == 0
            lists.append(sorted(map(tuple, w[header:header + 4 * len(host)].reshape(-1, 4).tolist())))
        assert lists[0] == lists[1] == sorted(map(tuple, host.tolist()))


def test_device_schedule_over_shared_kv_groups(cuda):
    """The dK/dV list of tasks over shared stored rows: one item per (group of tasks that start at one stored row, key
    block of the group's longest prefix), its cost the number of query blocks of all the group's tasks that see the
    block, groups numbered by their first task with queries; tasks without queries belong to no group.  Checked
    against a restatement in numpy, as are the group tables behind the list; word 3 of the header counts groups that
    run into the next one (none here, one in a second batch made to overlap)."""
    from distca_amd import workloads
    from distca_amd._lib import CaParams, load
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    import ctypes
    hq, hkv, g = 8, 2, 4
    k_lens = np.array([255, 256, 257, 700, 700, 33, 512, 513, 300, 130], dtype=np.int64)
    q_lens = np.array([255, 1, 1, 443, 100, 33, 212, 1, 0, 64], dtype=np.int64)
    offs = np.array([40, 40, 40, 40, 40, 40, 1000, 1000, 1000, 800], dtype=np.int64)
    total_k = 1600
    for offs_case, want_violations in ((offs, 0), (np.where(offs == 800, 600, offs), 1)):
        b = workloads.TaskBatch("shared_groups", q_lens, k_lens, hq, hkv)
        tq = int(q_lens.sum())
        gen = torch.Generator(device=cuda).manual_seed(3)
        rnd = lambda *shape: torch.randn(shape, generator=gen, device=cuda, dtype=torch.float32).to(torch.bfloat16)
        q, k, v, do = rnd(tq, hq, 128), rnd(total_k, hkv, 128), rnd(total_k, hkv, 128), rnd(tq, hq, 128)
        cu_q = torch.tensor(b.cu_seqlens_q, dtype=torch.int32, device=cuda)
        cu_k = torch.tensor(b.cu_seqlens_k, dtype=torch.int32, device=cuda)
        kv_off = torch.tensor(offs_case, dtype=torch.int32, device=cuda)
        mq, mk = int(q_lens.max()), int(k_lens.max())
        p = CaParams(len(q_lens), tq, total_k, hq, hkv, 128, mq, mk, 128 ** -0.5, 1, 1, 0)
        nbytes = load().distca_ca_bwd_workspace_bytes(ctypes.byref(p))
        ws = torch.zeros((nbytes,), dtype=torch.uint8, device=cuda)
        out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mk, kv_task_offsets=kv_off)
        ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mk, deterministic=True, kv_task_offsets=kv_off, workspace=ws)
        torch.cuda.synchronize()
        w = ws.cpu().view(torch.int32).numpy()
        # numpy restatement
        live = [t for t in range(len(q_lens)) if q_lens[t] > 0]
        starts = []
        for t in live:
            if offs_case[t] not in starts:
                starts.append(int(offs_case[t]))
        members = [sorted([t for t in live if offs_case[t] == o], key=lambda t: (k_lens[t], t)) for o in starts]
        expect = []
        for u, ts in enumerate(members):
            for n in range(-(-int(max(k_lens[t] for t in ts)) // 256)):
                cost = 0
                for t in ts:
                    if n * 256 < k_lens[t]:
                        first_tok = max(0, n * 256 - int(k_lens[t] - q_lens[t]))
                        cost += max(0, -(-int(q_lens[t]) * g // 32) - first_tok * g // 32)
                expect.append((u, n, cost))
        assert int(w[0]) == len(expect) and int(w[2]) == 0 and int(w[3]) == want_violations
        header = (4 + len(q_lens) + 1 + 3) // 4 * 4
        dev = w[header:header + 4 * len(expect)].reshape(-1, 4)
        assert sorted(map(tuple, dev[:, :3].tolist())) == sorted(expect)
        assert (np.diff(dev[:, 2]) <= 0).all()
        if want_violations:
            continue
        # the group tables behind the ticket counters
        cap = int(load().distca_ca_schedule_capacity(1, ctypes.byref(p)))
        sched_bytes = (header + 4 * cap) * 4
        tables = ((sched_bytes + 255) // 256 * 256 + 256 + 1024) // 4
        nb = len(q_lens)
        first = w[tables:tables + nb + 1]
        tasks = w[tables + nb + 1:tables + 2 * nb + 1]
        off = w[tables + 2 * nb + 1:tables + 3 * nb + 1]
        lmax = w[tables + 3 * nb + 1:tables + 4 * nb + 1]
        gap_lo = w[tables + 4 * nb + 1:tables + 5 * nb + 2]
        gap_hi = w[tables + 5 * nb + 2:tables + 6 * nb + 3]
        assert first[:len(members) + 1].tolist() == np.concatenate([[0], np.cumsum([len(m) for m in members])]).tolist()
        assert tasks[:len(live)].tolist() == [t for m in members for t in m]
        assert off[:len(members)].tolist() == starts
        assert lmax[:len(members)].tolist() == [int(max(k_lens[t] for t in m)) for m in members]
        gaps = sorted((int(a), int(c)) for a, c in zip(gap_lo[:len(members) + 1], gap_hi[:len(members) + 1]) if c > a)
        assert gaps == [(0, 40), (740, 800), (930, 1000), (1513, 1600)]


@pytest.mark.parametrize("kind", ["fwd", "bwd"])
def test_device_schedule_equals_host_mirror(cuda, kind):
    """The workspace begins with the schedule the device built ([0] = item count, then the
    per-task block prefix, then (task, block, cost, piece | pieces << 16) items): same items, same order of cost
    bins as distca_ca_schedule_host."""
    from distca_amd import scheduler, workloads
    from distca_amd._lib import CaParams, load
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    import ctypes
    rng = np.random.default_rng(4)
    ql = rng.integers(1, 3000, size=14).astype(np.int64); ql[3] = 0
    b = workloads.TaskBatch("prefix_tasks", ql, ql + rng.integers(0, 4000, size=14) * (rng.random(14) < 0.6), 32, 8)
    hq, hkv = 32, 8
    q, k, v, do, cu_q, cu_k = _dev_inputs(b, hq, hkv, cuda, 9)
    mq, mk = int(max(b.q_lens)), int(max(b.k_lens))
    p = CaParams(len(b.q_lens), b.total_q, b.kv_rows, hq, hkv, 128, mq, mk, 128 ** -0.5, 1, 0, 0)
    lib = load()
    nbytes = lib.distca_ca_bwd_workspace_bytes(ctypes.byref(p))
    ws = torch.zeros((nbytes,), dtype=torch.uint8, device=cuda)
    out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mk, workspace=ws)
    if kind == "bwd":
        ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mk, workspace=ws)
    torch.cuda.synchronize()
    w = ws.cpu().view(torch.int32).numpy()
    host = scheduler.build_schedule(scheduler.BWD if kind == "bwd" else scheduler.FWD, b.cu_seqlens_q, b.cu_seqlens_k, hq, hkv)
    n = int(w[0])
    assert n == len(host)
    header = (4 + len(b.q_lens) + 1 + 3) // 4 * 4
    dev = w[header:header + 4 * n].reshape(n, 4)
    assert (np.diff(dev[:, 2]) <= 0).all()
    as_set = lambda a: sorted(map(tuple, a.tolist()))
    assert as_set(dev) == as_set(host)
    assert np.array_equal(dev[:, 2], host[:, 2])          # identical cost sequence; ties may permute


def test_pack_round_trip_full_size(cuda):
    """cfg4 at full size: pack then unpack returns the source bit for bit, q-sized and k-sized tokens."""
    from distca_amd import workloads
    from distca_amd.ops import a2a_memcpy_non_cp
    lay = workloads.config4_pack()
    for hidden in (4096, 1024):
        tb = hidden * 2
        lens = torch.tensor(lay.seq_tokens, dtype=torch.int64)
        sizes = lens * tb
        perm = torch.randperm(len(lens), generator=torch.Generator().manual_seed(3))
        off = torch.zeros(len(lens), dtype=torch.int64)
        off[perm] = torch.cumsum(sizes[perm], 0) - sizes[perm]
        src = torch.randint(-32768, 32767, (lay.num_tokens, hidden), dtype=torch.int16, device=cuda).view(torch.bfloat16)
        buf = torch.zeros(int(sizes.sum()), dtype=torch.uint8, device=cuda)
        a2a_memcpy_non_cp(src, off.to(cuda), lens.to(cuda), True, buffer=buf)
        back = torch.zeros_like(src)
        a2a_memcpy_non_cp(back, off.to(cuda), lens.to(cuda), False, buffer=buf)
        torch.cuda.synchronize()
        assert torch.equal(back.view(torch.int16), src.view(torch.int16))
        # a checksum of the buffer equals the checksum of the source: every byte landed exactly once
        assert int(buf.view(torch.int16).to(torch.int64).sum()) == int(src.view(torch.int16).to(torch.int64).sum())


def test_config3_shared_kv_tasks_sampled_rows(cuda):
    """CA tasks cut from long documents whose K/V is stored once and shared through kv_task_offsets
    (config 3, both variants, at a quarter of the full size): sampled rows of out, lse and dq
    against the oracle; dK/dV against the sum over tasks through <K,dK> = <Q,dQ> per document."""
    from distca_amd import workloads
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    for variant in ("a", "b"):
        b = workloads.config3_ca_tasks(variant=variant, total_q=65536, num_docs=4, max_doc=131072)
        q, k, v, do, cu_q, cu_k = _dev_inputs(b, 32, 8, cuda, 60)
        kv_off = torch.tensor(b.kv_task_offsets, dtype=torch.int32, device=cuda)
        mq, mk = int(max(b.q_lens)), int(max(b.k_lens))
        print(f"cfg3{variant}: {len(b.q_lens)} tasks, kv rows {b.kv_rows}", flush=True)
        out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mk, kv_task_offsets=kv_off)
        dq, dk, dv = ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mk, kv_task_offsets=kv_off)
        torch.cuda.synchronize()
        rng = np.random.default_rng(1)
        for t in rng.choice(len(b.q_lens), size=4, replace=False):
            lq, lk = int(b.q_lens[t]), int(b.k_lens[t])
            r0 = int(rng.integers(0, lq - 8)); r1 = r0 + 8
            q0 = int(b.cu_seqlens_q[t]); k0 = int(b.kv_task_offsets[t])
            kvis = r1 + (lk - lq)                         # keys beyond the last sampled row's horizon are masked anyway
            o_ref, l_ref, dq_ref = ca_reference_rows(q[q0:q0 + r1].cpu(), k[k0:k0 + kvis].cpu(), v[k0:k0 + kvis].cpu(), do[q0:q0 + r1].cpu(),
                                                     [0, r1], [0, kvis], 0, r0, r1, out_rows=out[q0 + r0:q0 + r1].cpu(),
                                                     lse_rows=lse[:, q0 + r0:q0 + r1].cpu())
            print(f"  task {t}: rows [{r0},{r1}) of {lq}, prefix {lk}", flush=True)
            assert_close_bf16(out[q0 + r0:q0 + r1], o_ref, f"out task {t}")
            assert (lse[:, q0 + r0:q0 + r1].cpu() - l_ref).abs().max().item() <= 2e-3
            assert_close_bf16(dq[q0 + r0:q0 + r1], dq_ref, f"dq task {t}")
        # scale invariance over the whole batch per kv head: sum <Q,dQ> = sum <K,dK>, sum <V,dV> = sum <O,dO>
        whole_q, whole_k = [0, b.total_q], [0, b.kv_rows]
        assert_identity(task_sums(q, dq, whole_q, 8), task_sums(k, dk, whole_k, 8), "<Q,dQ> = <K,dK>")
        assert_identity(task_sums(v, dv, whole_k, 8), task_sums(out, do, whole_q, 8), "<V,dV> = <O,dO>")


@pytest.mark.parametrize("deterministic", [True, False])
def test_ops_replay_from_a_captured_graph(cuda, deterministic):
    """Every entry point only enqueues work on the caller's stream (no allocation, no host
    synchronisation), so a tick can be captured once and replayed.  The replays run with other
    eager work in between and with changed inputs, and must match eager results each time: bit for
    bit, except dk and dv of the non-deterministic backward, which on a batch this small cuts key
    blocks into pieces and adds their sums with float atomics in whatever order they finish (the
    fp32 accumulators they go through are cleared by a kernel of the tick, so the replays test that
    too)."""
    from distca_amd import workloads
    from distca_amd._lib import CaParams, load
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    from distca_amd.ops import a2a_memcpy_non_cp
    import ctypes
    lens = [300, 45, 700]
    T, hq, hkv = sum(lens), 8, 2
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=cuda)
    g = torch.Generator(device=cuda).manual_seed(3)
    rnd = lambda *s: torch.randn(s, generator=g, device=cuda).to(torch.bfloat16)
    q, k, v, do = rnd(T, hq, 128), rnd(T, hkv, 128), rnd(T, hkv, 128), rnd(T, hq, 128)
    out, lse = torch.empty_like(q), torch.empty((hq, T), dtype=torch.float32, device=cuda)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    p = CaParams(3, T, T, hq, hkv, 128, 700, 700, 128 ** -0.5, 1, 0, 0)
    ws = torch.empty(load().distca_ca_bwd_workspace_bytes(ctypes.byref(p)), dtype=torch.uint8, device=cuda)
    shard = torch.tensor(lens, dtype=torch.int64, device=cuda)
    tb = hq * 256
    off = torch.tensor([T * tb + 4096, 0, 45 * tb + 1024], dtype=torch.int64, device=cuda)  # shards out of order, with gaps
    buf = torch.zeros(4 * T * hq * 256, dtype=torch.uint8, device=cuda)

    def tick():
        o, l = ca_varlen_fwd(q, k, v, cu, cu, 700, 700, workspace=ws)
        out.copy_(o); lse.copy_(l)
        ca_varlen_bwd(do, q, k, v, out, lse, cu, cu, 700, 700, deterministic=deterministic, dq=dq, dk=dk, dv=dv, workspace=ws)
        a2a_memcpy_non_cp(dq.reshape(T, -1), off, shard, True, buffer=buf)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        tick()                                      # warm-up outside capture (lazy module loading)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            tick()
    torch.cuda.synchronize()
    for rep in range(3):
        q.copy_(rnd(T, hq, 128)); do.copy_(rnd(T, hq, 128))          # eager work between replays, new inputs
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (out, lse, dq, dk, dv, buf)]
        tick()                                                        # the same tick, eagerly
        torch.cuda.synchronize()
        for name, a_, b_ in zip(("out", "lse", "dq", "dk", "dv", "buf"), got, (out, lse, dq, dk, dv, buf)):
            if name in ("dk", "dv") and not deterministic:
                # two orders of fp32 additions, each result rounded to bf16 once: a unit in the last place apart at most
                err = (a_.float() - b_.float()).abs() / b_.float().abs().clamp_min(2.0 ** -6)
                assert err.max().item() <= 2.0 ** -7, f"replay {rep}: {name} differs from the eager result by {err.max().item():.2e}"
            else:
                assert torch.equal(a_, b_), f"replay {rep}: {name} differs from the eager result"


def test_server_ticks_in_place_equal_step_by_step_at_full_size(cuda):
    """The 131072-token workload as one CA-server tick: the kernels that read request tokens from the
    receive buffer and write reply tokens into the send buffer leave exactly the bytes the unpack ->
    attention -> pack sequence leaves, forward and backward."""
    from distca_amd import metadata, workloads
    from distca_amd.fused_comm_attn import FlashAttnArgs, ca_server_backward, ca_server_forward
    batch = workloads.config2_llama8b_128k()
    plan = metadata.single_rank_plan([[int(n)] for n in batch.q_lens], 32, 8)
    attn, fwd, bwd, (f_recv, f_send, b_recv, b_send) = metadata.server_metas(plan, cuda)
    fa = FlashAttnArgs(32, 8, 128)
    g = torch.Generator(device=cuda).manual_seed(3)
    rnd_bytes = lambda n: torch.randn(n // 2, generator=g, device=cuda).to(torch.bfloat16).view(torch.uint8)
    recv = rnd_bytes(f_recv)
    sends = []
    for in_place in (True, False):
        send = torch.zeros(f_send, dtype=torch.uint8, device=cuda)
        print(f"forward tick in_place={in_place}", flush=True)
        ca_server_forward(recv, send, fwd, attn, fa, in_place=in_place)
        sends.append(send)
    torch.cuda.synchronize()
    assert torch.equal(sends[0], sends[1])
    # backward: any bytes will do as a request (the lse part is read as fp32: keep it finite and large
    # enough that P stays below 1, as a real lse would)
    breq = rnd_bytes(b_recv)
    row = 32 * 128 * 2
    tok = plan.merged_q_bytes
    q_off = plan.request_layout(True)[0]
    assert int(q_off[0]) == 0 and tok % 4 == 0
    tokens = breq[:plan.num_q_tokens * tok].view(plan.num_q_tokens, tok)
    tokens[:, 2 * row:2 * row + 32 * 4] = torch.full((plan.num_q_tokens, 32), 20.0, device=cuda).view(torch.uint8)
    sends = []
    for in_place in (True, False):
        send = torch.zeros(b_send, dtype=torch.uint8, device=cuda)
        print(f"backward tick in_place={in_place}", flush=True)
        ca_server_backward(breq, send, bwd, fa, attn.cu_seqlens_q, attn.cu_seqlens_kv, attn.max_seqlen_q, attn.max_seqlen_kv,
                           in_place=in_place)
        sends.append(send)
    torch.cuda.synchronize()
    # dq: the same bytes.  dk / dv: the in-place tick keeps one copy of every K/V shard and runs the dK/dV kernel over
    # (document, key block) items, the step-by-step tick over (task, key block) items; both are deterministic, but the
    # two lists rank their items differently, and the rank decides whether an item walks its query blocks up or
    # down, i.e. the order of its fp32 sums: equal to a unit in the last place of the bf16 result.
    nq = plan.num_q_tokens * plan.q_bytes
    assert int(plan.reply_layout(True)[0][0]) == 0
    assert torch.equal(sends[0][:nq], sends[1][:nq])
    a, b_ = (x[nq:].view(torch.bfloat16).float() for x in sends)
    err = ((a - b_).abs() / b_.abs().clamp_min(2.0 ** -6)).max().item()
    assert err <= 2.0 ** -7, f"dk / dv of the two ticks differ by {err:.2e}"


def test_mfma_rate_probe(cuda):
    """The diagnostic loop of MFMAs runs and reports finite, positive figures; an MFMA cannot take fewer than 32 cycles.
    What the figures are depends on the box's power state and is the benchmark's business, not a test's: they are
    printed."""
    from distca_amd import _lib
    scratch = torch.zeros(4, dtype=torch.int64, device=cuda)
    for kind in (_lib.PROBE_MFMA_ONLY, _lib.PROBE_LDS_READ, _lib.PROBE_FMA4, _lib.PROBE_EXP2, _lib.PROBE_MIX):
        _lib.probe_mfma_rate(kind, 2000, scratch.data_ptr())   # the first launch of a kernel also loads it
        tf, cyc, ghz = _lib.probe_mfma_rate(kind, 40000, scratch.data_ptr())
        print(f"probe kind {kind}: {tf:.0f} TFLOP/s, {cyc:.1f} cycles per MFMA, {ghz:.2f} GHz", flush=True)
        assert all(np.isfinite(x) and x > 0 for x in (tf, cyc, ghz))
        assert cyc >= 31.9
    with pytest.raises(RuntimeError):
        _lib.probe_mfma_rate(9, 10, scratch.data_ptr())
