"""GPU parity of the HIP attention kernels (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from helpers import assert_close_bf16, cu, make_qkv
from oracle.attention import ca_reference_bwd, ca_reference_fwd

pytestmark = pytest.mark.gpu


def _run(q_lens, k_lens, hq, hkv, seed, cuda, causal=True, kv_offsets=None, total_k=None, bwd=True, d=128, kv_grad_tol=None,
         dtype=torch.bfloat16, deterministic=False):
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    cu_q, cu_k = cu(q_lens), cu(k_lens)
    tq = int(cu_q[-1])
    tk = int(total_k if total_k is not None else cu_k[-1])
    q, k, v, do = (t.to(dtype) for t in make_qkv(tq, tk, hq, hkv, d, seed))   # bf16 values are exact in fp16 at this scale
    ref_out, ref_lse = ca_reference_fwd(q, k, v, cu_q, cu_k, causal=causal, kv_task_offsets=kv_offsets)
    dcu_q = torch.tensor(cu_q, device=cuda)
    dcu_k = torch.tensor(cu_k, device=cuda)
    dkv = torch.tensor(np.asarray(kv_offsets, dtype=np.int32), device=cuda) if kv_offsets is not None else None
    qd, kd, vd, dod = q.to(cuda), k.to(cuda), v.to(cuda), do.to(cuda)
    print(f"case q_lens={list(q_lens)[:6]} k_lens={list(k_lens)[:6]} hq={hq} hkv={hkv} causal={causal} alias={kv_offsets is not None}", flush=True)
    out, lse = ca_varlen_fwd(qd, kd, vd, dcu_q, dcu_k, int(max(q_lens)), int(max(k_lens)), None, causal, dkv)
    torch.cuda.synchronize()
    assert out.dtype == dtype and out.shape == qd.shape
    assert_close_bf16(out, ref_out, "out")
    finite = torch.isfinite(ref_lse)
    lse_c = lse.cpu()
    assert torch.equal(torch.isfinite(lse_c), finite)
    assert (lse_c[finite] - ref_lse[finite]).abs().max().item() <= 2e-3, "lse"
    if not bwd:
        return
    # the oracle consumes the same (out, lse) the kernel is handed, as the reference's backward does
    ref_dq, ref_dk, ref_dv = ca_reference_bwd(do, q, k, v, cu_q, cu_k, causal=causal, kv_task_offsets=kv_offsets,
                                              out=out.cpu(), softmax_lse=lse.cpu())
    dq, dk, dv = ca_varlen_bwd(dod, qd, kd, vd, out, lse, dcu_q, dcu_k, int(max(q_lens)), int(max(k_lens)), None, causal,
                               deterministic, dkv)
    torch.cuda.synchronize()
    assert dq.dtype == dk.dtype == dv.dtype == dtype and dq.shape == qd.shape and dk.shape == kd.shape
    if deterministic:
        again = ca_varlen_bwd(dod, qd, kd, vd, out, lse, dcu_q, dcu_k, int(max(q_lens)), int(max(k_lens)), None, causal, True, dkv)
        torch.cuda.synchronize()
        for name, x, y in zip(("dq", "dk", "dv"), (dq, dk, dv), again):
            assert torch.equal(x, y), f"{name} differs between two deterministic runs"
    assert_close_bf16(dq, ref_dq, "dq")
    tol = dict(max_abs=kv_grad_tol[0], mean_rel=kv_grad_tol[1]) if kv_grad_tol else {}
    assert_close_bf16(dk, ref_dk, "dk", **tol)
    assert_close_bf16(dv, ref_dv, "dv", **tol)


def test_config1_tiny_forward(cuda):
    """BASELINE config 1: docs [512, 1024, 2560], 32q/8kv, d128, causal, forward."""
    _run([512, 1024, 2560], [512, 1024, 2560], 32, 8, 1, cuda, bwd=False)


@pytest.mark.parametrize("lens", [[64], [1], [33, 1, 130], [257, 255, 256, 3]])
def test_whole_docs_fwd_bwd_small(cuda, lens):
    _run(lens, lens, 8, 2, 7, cuda)


def test_whole_docs_fwd_bwd_medium(cuda):
    _run([512, 1024, 700], [512, 1024, 700], 32, 8, 2, cuda)


@pytest.mark.parametrize("hq,hkv", [(4, 4), (8, 1), (6, 2), (16, 2), (64, 1), (24, 8), (32, 1), (16, 16), (3, 3), (80, 80)])
def test_head_groupings(cuda, hq, hkv):
    """MHA (also with 16, 3 and 80 kv heads: more lists of work items than XCDs, a count that does not divide
    their number, and more lists than a wave has lanes to look at them), MQA, a non-power-of-two group, the Llama-3-70B group of 8; groups of 64 (more heads per token than a
    backward row block holds), of 3 (a row block does not start at a token boundary) and of 32 (exactly one)."""
    # dK and dV of a kv head sum the bf16-rounded P and dS of all its query heads: with 32 or 64 of them the
    # rounding noise of the sum (growing as the square root of the count) is allowed twice the bar
    _run([300, 45], [300, 45], hq, hkv, 3, cuda, kv_grad_tol=(4e-2, 2e-3) if hq // hkv >= 32 else None)


def test_prefix_tasks_lk_gt_lq(cuda):
    """CA tasks: query shard shorter than its KV prefix (bottom-right causal)."""
    _run([128, 200, 64], [384, 200, 1000], 8, 2, 4, cuda)


@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 4), (16, 2)])
def test_prefix_lengths_around_tile_and_ring_boundaries(cuda, hq, hkv):
    """Tasks whose K/V prefixes end one key before, on and one key after multiples of 32 (a K/V tile of the dQ
    kernel), of 64 (a tile of the forward) and of 128 (one round of the dQ kernel's four ring stages), with query
    shards of 1 to 100 tokens: workgroups with one to a dozen tiles, with and without unmasked tiles, whose last
    waves own no row or only a few."""
    k_lens = [1, 31, 32, 33, 63, 64, 65, 95, 97, 127, 128, 129, 159, 161, 191, 193, 255, 256, 257, 289, 383, 385]
    q_lens = [1, 31, 17, 33, 5, 64, 65, 16, 97, 100, 3, 1, 64, 33, 100, 17, 8, 100, 65, 1, 100, 49]
    assert all(q <= k for q, k in zip(q_lens, k_lens))
    _run(q_lens, k_lens, hq, hkv, 21, cuda)


def test_shared_kv_prefix(cuda):
    """Three shards of one 600-token document reading one stored KV copy."""
    _run([200, 150, 250], [200, 350, 600], 8, 2, 5, cuda, kv_offsets=[0, 0, 0], total_k=600)


@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 4), (12, 4)])
@pytest.mark.parametrize("causal", [True, False])
def test_shared_kv_documents_deterministic(cuda, hq, hkv, causal):
    """Three stored documents read by tasks that are prefixes of them, with the deterministic switch the reference's
    server has by default: one work item per (document, key block) walks the query rows of every task that sees the
    block and writes dK/dV once.  The documents lie in the store out of order and with unread rows before, between
    and behind them (those come back as zeros); prefixes end around key-block (256) and tile (32, 64) edges, one task
    has no queries, one document is read by a single task, two tasks of a document have the same prefix length."""
    #          document at row 40 (700 rows)      at row 1000 (513 rows)   at row 800 (130 rows)
    k_lens = [255, 256, 257, 700, 700, 33,        512, 513, 300,            130]
    q_lens = [255, 1, 1, 443, 100, 33,            212, 1, 0,                64]
    offs = [40, 40, 40, 40, 40, 40,               1000, 1000, 1000,         800]
    _run(q_lens, k_lens, hq, hkv, 31, cuda, causal=causal, kv_offsets=offs, total_k=1600, deterministic=True)


def test_queries_that_see_no_key(cuda):
    """A task with more queries than keys under the bottom-right aligned mask: its first Lq - Lk rows see nothing.
    Their output and dq are zero and their lse is -inf, and they add nothing to dk / dv (the backward kernels meet
    exp2(+inf) for such rows and must mask it away)."""
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    _run([300, 64], [100, 64], 8, 2, 41, cuda)
    q, k, v, do = (t.to(cuda) for t in make_qkv(364, 164, 8, 2, 128, 41))
    cq, ck = torch.tensor(cu([300, 64]), device=cuda), torch.tensor(cu([100, 64]), device=cuda)
    out, lse = ca_varlen_fwd(q, k, v, cq, ck, 300, 100)
    dq, dk, dv = ca_varlen_bwd(do, q, k, v, out, lse, cq, ck, 300, 100)
    torch.cuda.synchronize()
    assert (out[:200] == 0).all() and (dq[:200] == 0).all() and torch.isinf(lse[:, :200]).all() and (lse[:, :200] < 0).all()
    assert torch.isfinite(dk.float()).all() and torch.isfinite(dv.float()).all() and torch.isfinite(dq.float()).all()


@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 4)])
def test_short_tasks_as_merged_work_items(cuda, hq, hkv):
    """A batch whose tasks average fewer than 2048 query tokens has the forward and dQ kernels work off several
    consecutive blocks of a task per work item (eight for the 1024-token document here, whose sixteen blocks at four
    heads per kv head make two items; the last item of a task is usually shorter), the next block's Q rows and first K
    tile requested while the present one is normalised and stored.  Whole documents and tasks with prefixes, lengths
    on and off the block edges."""
    _run([1024, 1000, 513, 1, 2047, 64], [1024, 1000, 513, 1, 2047, 64], hq, hkv, 51, cuda)
    _run([1024, 300, 700], [1024, 1324, 764], hq, hkv, 52, cuda)


def test_non_causal(cuda):
    _run([100, 260], [100, 260], 4, 2, 6, cuda, causal=False)


def test_long_document_in_pieces(cuda):
    """One document of 4096 tokens: too few key blocks to occupy the device, so the backward cuts every key
    block into pieces of consecutive query blocks (the first block into about thirty) and adds their dK/dV in
    fp32; also a deterministic run of the same, whole blocks, bit for bit equal to a second one."""
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    _run([4096], [4096], 8, 2, 11, cuda)
    q, k, v, do = (t.to(cuda) for t in make_qkv(4096, 4096, 8, 2, 128, 11))
    c = torch.tensor(cu([4096]), device=cuda)
    out, lse = ca_varlen_fwd(q, k, v, c, c, 4096, 4096, None, True, None)
    a = ca_varlen_bwd(do, q, k, v, out, lse, c, c, 4096, 4096, None, True, True, None)
    b = ca_varlen_bwd(do, q, k, v, out, lse, c, c, 4096, 4096, None, True, True, None)
    torch.cuda.synchronize()
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    n = ca_varlen_bwd(do, q, k, v, out, lse, c, c, 4096, 4096, None, True, False, None)
    torch.cuda.synchronize()
    for x, y, name in zip(n, a, ("dq", "dk", "dv")):
        # same products, summed per piece and then across pieces in fp32: a bf16 unit in the last place apart at most
        err = ((x.float() - y.float()).abs() / y.float().abs().clamp_min(2.0 ** -6)).max().item()
        assert err <= 2.0 ** -7, f"{name}: pieces against whole blocks {err:.2e}"


@pytest.mark.parametrize("hq,hkv,n", [(128, 8, 989), (64, 8, 1345), (64, 8, 1364), (32, 8, 2999), (4, 1, 3000), (8, 2, 1500),
                                      (16, 16, 7600), (16, 16, 7700)])
def test_single_documents_around_the_piece_cutting_threshold(cuda, hq, hkv, n):
    """One document per call, backward with key blocks cut into pieces: lengths at which the piece count comes
    closest to the room the work list has (989 tokens at 128/8 heads and 1345 at 64/8 made one piece too many when
    the piece size was rounded down), and a pair of lengths either side of the size from which blocks stay whole
    (7680 tokens at 16 kv heads).  Gradients against the oracle, and the builder's count of entries it had no
    room for must be zero."""
    from distca_amd._lib import CaParams, load
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    import ctypes
    q, k, v, do = make_qkv(n, n, hq, hkv, 128, 31)
    c = cu([n])
    dc = torch.tensor(c, device=cuda)
    qd, kd, vd, dod = q.to(cuda), k.to(cuda), v.to(cuda), do.to(cuda)
    p = CaParams(1, n, n, hq, hkv, 128, n, n, 128 ** -0.5, 1, 0, 0)
    ws = torch.zeros(load().distca_ca_bwd_workspace_bytes(ctypes.byref(p)), dtype=torch.uint8, device=cuda)
    print(f"case single document n={n} hq={hq} hkv={hkv}", flush=True)
    out, lse = ca_varlen_fwd(qd, kd, vd, dc, dc, n, n)
    dq, dk, dv = ca_varlen_bwd(dod, qd, kd, vd, out, lse, dc, dc, n, n, None, True, False, None, workspace=ws)
    torch.cuda.synchronize()
    head = ws[:16].view(torch.int32).cpu()
    assert int(head[2]) == 0, f"the key-block list dropped {int(head[2])} entries"
    from distca_amd import scheduler
    assert int(head[0]) == len(scheduler.build_schedule(scheduler.BWD, c, c, hq, hkv))
    ref_dq, ref_dk, ref_dv = ca_reference_bwd(do, q, k, v, c, c, out=out.cpu(), softmax_lse=lse.cpu())
    tol = dict(max_abs=4e-2, mean_rel=2e-3) if hq // hkv >= 16 else {}
    assert_close_bf16(dq, ref_dq, "dq")
    assert_close_bf16(dk, ref_dk, "dk", **tol)
    assert_close_bf16(dv, ref_dv, "dv", **tol)


def test_key_blocks_walked_in_both_directions(cuda):
    """The dK/dV list marks alternate rounds of items (as many as compute units serve a kv head: 16 here) to be
    walked upwards from the diagonal instead of downwards from the end.  Whole key blocks (deterministic), prefix
    tasks among them: both directions occur, the gradients match the oracle and a second run bit for bit."""
    from distca_amd import scheduler
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    q_lens, k_lens, hq, hkv = [2600, 900, 1800, 37], [2600, 2100, 1800, 300], 16, 16
    items = scheduler.build_schedule(scheduler.BWD, cu(q_lens), cu(k_lens), hq, hkv, deterministic=True)
    up = items[:, 3] < 0
    assert up.any() and (~up).any() and (scheduler.item_pieces(items[:, 3]) == 1).all()
    cu_q, cu_k = cu(q_lens), cu(k_lens)
    q, k, v, do = make_qkv(int(cu_q[-1]), int(cu_k[-1]), hq, hkv, 128, 77)
    dq_, dk_ = torch.tensor(cu_q, device=cuda), torch.tensor(cu_k, device=cuda)
    qd, kd, vd, dod = q.to(cuda), k.to(cuda), v.to(cuda), do.to(cuda)
    out, lse = ca_varlen_fwd(qd, kd, vd, dq_, dk_, max(q_lens), max(k_lens))
    a = ca_varlen_bwd(dod, qd, kd, vd, out, lse, dq_, dk_, max(q_lens), max(k_lens), None, True, True, None)
    b = ca_varlen_bwd(dod, qd, kd, vd, out, lse, dq_, dk_, max(q_lens), max(k_lens), None, True, True, None)
    torch.cuda.synchronize()
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    ref = ca_reference_bwd(do, q, k, v, cu_q, cu_k, out=out.cpu(), softmax_lse=lse.cpu())
    for x, r, name in zip(a, ref, ("dq", "dk", "dv")):
        assert_close_bf16(x, r, name)


def test_empty_task(cuda):
    _run([128, 0, 70], [128, 0, 70], 4, 2, 8, cuda)


@pytest.mark.parametrize("span", [6.0, 40.0, 400.0, -400.0])
def test_scores_that_drift_along_the_keys(cuda, span):
    """The forward keeps a running reference per row that trails the row maximum by up to 2^8 and
    is only corrected when a tile overshoots it.  Scores here carry a trend of `span` (natural-log
    units) from the first key to the last: a reference that is seldom, sometimes, or in every tile
    overtaken, and one that is never overtaken after the first tile."""
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    n, hq, hkv, d = 2048, 4, 2, 128
    q, k, v, do = make_qkv(n, n, hq, hkv, d, 21)
    q, k = q.float(), k.float()
    q[:, :, 0] = 16.0
    k[:, :, 0] = (span * (d ** 0.5) / 16.0) * torch.arange(n, dtype=torch.float32)[:, None] / n
    q, k = q.to(torch.bfloat16), k.to(torch.bfloat16)
    cu_q = cu([n])
    ref_out, ref_lse = ca_reference_fwd(q, k, v, cu_q, cu_q)
    dcu = torch.tensor(cu_q, device=cuda)
    qd, kd, vd, dod = q.to(cuda), k.to(cuda), v.to(cuda), do.to(cuda)
    print(f"case drift span={span}", flush=True)
    out, lse = ca_varlen_fwd(qd, kd, vd, dcu, dcu, n, n, None, True, None)
    torch.cuda.synchronize()
    assert_close_bf16(out, ref_out, "out")
    assert (lse.cpu() - ref_lse).abs().max().item() <= 2e-3 * max(1.0, abs(span) / 40), "lse"
    if abs(span) > 10:
        return  # the backward keeps no running reference, and K entries of tens amplify the bf16 rounding of dS beyond the bar
    ref_dq, ref_dk, ref_dv = ca_reference_bwd(do, q, k, v, cu_q, cu_q, out=out.cpu(), softmax_lse=lse.cpu())
    dq, dk, dv = ca_varlen_bwd(dod, qd, kd, vd, out, lse, dcu, dcu, n, n, None, True, False, None)
    torch.cuda.synchronize()
    assert_close_bf16(dq, ref_dq, "dq")
    assert_close_bf16(dk, ref_dk, "dk")
    assert_close_bf16(dv, ref_dv, "dv")


@pytest.mark.parametrize("seed", range(12))
def test_random_task_batches(cuda, seed):
    """Seeded random batches of CA tasks: lengths around the tile edges (32, 64, 128, 256 +- 1), prefixes
    longer than the query shard, every head grouping the kernels accept, causal or not, with and
    without tasks that share one stored K/V copy."""
    rng = np.random.default_rng(1000 + seed)
    edges = [1, 2, 31, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 383, 511, 513]
    n = int(rng.integers(1, 7))
    q_lens = [int(rng.choice(edges)) if rng.random() < 0.7 else int(rng.integers(1, 700)) for _ in range(n)]
    if rng.random() < 0.25:
        q_lens[int(rng.integers(n))] = 0
    hq, hkv = [(4, 4), (8, 2), (8, 1), (12, 4), (16, 2), (2, 1)][int(rng.integers(6))]
    causal = bool(rng.random() < 0.8)
    if rng.random() < 0.3 and all(q_lens):
        # shards of one document over one stored copy of its K/V
        ends = np.cumsum(q_lens)
        _run(q_lens, [int(e) for e in ends], hq, hkv, seed, cuda, causal=causal, kv_offsets=[0] * n, total_k=int(ends[-1]))
        return
    k_lens = [q + (int(rng.choice(edges)) if (q and rng.random() < 0.5) else 0) for q in q_lens]
    _run(q_lens, k_lens, hq, hkv, seed, cuda, causal=causal)


@pytest.mark.parametrize("case", ["whole", "prefix", "shared", "groups", "pieces"])
def test_fp16_inputs(cuda, case):
    """The same kernels compiled for IEEE half precision (the reference's own tests run fp16,
    tests/test_megatron_layer.py of the reference): whole documents, prefix tasks, tasks that share one stored K/V
    copy (float atomics in dK/dV), a group of 8 query heads, and a batch small enough for key blocks to be cut into
    pieces.  Same bar as bf16, with the rounding floor taken in fp16 (its rounding error is an eighth of bf16's, so the
    bar is the looser of the two here)."""
    f16 = torch.float16
    if case == "whole":
        _run([257, 255, 256, 3, 700], [257, 255, 256, 3, 700], 8, 2, 61, cuda, dtype=f16)
    elif case == "prefix":
        _run([128, 200, 64], [384, 200, 1000], 8, 2, 62, cuda, dtype=f16)
    elif case == "shared":
        _run([200, 150, 250], [200, 350, 600], 8, 2, 63, cuda, kv_offsets=[0, 0, 0], total_k=600, dtype=f16)
    elif case == "groups":
        _run([300, 45], [300, 45], 16, 2, 64, cuda, dtype=f16)
    else:
        _run([4096], [4096], 8, 2, 65, cuda, dtype=f16)


def test_fp16_and_bf16_agree_on_the_same_values(cuda):
    """Inputs that are exact in both types give outputs that differ by the types' rounding only: the fp16 build is
    the bf16 build with another element type, not another algorithm."""
    from distca_amd.fused_comm_attn import ca_varlen_fwd
    lens = [513, 64, 300]
    q, k, v, _ = make_qkv(sum(lens), sum(lens), 8, 2, 128, 66)
    c = torch.tensor(cu(lens), device=cuda)
    outs, lses = [], []
    for dt in (torch.bfloat16, torch.float16):
        o, l = ca_varlen_fwd(q.to(cuda).to(dt), k.to(cuda).to(dt), v.to(cuda).to(dt), c, c, max(lens), max(lens))
        outs.append(o.float().cpu()); lses.append(l.cpu())
    assert (lses[0] - lses[1]).abs().max().item() <= 2e-3
    assert (outs[0] - outs[1]).abs().max().item() <= 2e-2


@pytest.mark.parametrize("d,dtype", [(64, torch.bfloat16), (96, torch.float16), (40, torch.bfloat16), (8, torch.bfloat16)])
def test_head_dims_below_128(cuda, d, dtype):
    """Head dimensions that are multiples of 8 below 128 (the reference pads to a multiple of 8 and lets flash-attn
    handle the rest, fused_comm_attn.py:125-129): zero-padded to 128 on the way in, outputs and gradients cut back.
    The softmax scale is that of the true head dimension."""
    _run([130, 257, 64], [130, 300, 64], 4, 2, 67 + d, cuda, d=d, dtype=dtype)


def test_head_dims_that_are_refused(cuda):
    from distca_amd.fused_comm_attn import ca_varlen_fwd
    c = torch.tensor([0, 16], dtype=torch.int32, device=cuda)
    for d in (136, 256, 100):
        x = torch.zeros((16, 2, d), dtype=torch.bfloat16, device=cuda)
        with pytest.raises(RuntimeError, match="head_dim"):
            ca_varlen_fwd(x, x, x, c, c, 16, 16)
    q = torch.zeros((16, 2, 128), dtype=torch.float16, device=cuda)
    with pytest.raises(RuntimeError, match="same for q, k and v"):
        ca_varlen_fwd(q, q.to(torch.bfloat16), q, c, c, 16, 16)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        ca_varlen_fwd(q.float(), q.float(), q.float(), c, c, 16, 16)
