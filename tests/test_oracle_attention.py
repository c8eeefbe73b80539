"""Pins the attention oracle by mathematics (the reference holds no golden vectors for
attention): library routines on the special cases that reduce to them, autograd and finite
differences for gradients, a brute-force scalar loop, and the sharded-vs-whole identity the
reference asserts on its own layer tests (tests/test_megatron_layer.py:169,244-251)."""
import math

import numpy as np
import torch
import torch.nn.functional as F

import pytest

from helpers import cu, make_qkv
from oracle.attention import (ca_reference_key_rows, attention_flops, ca_reference_bwd, ca_reference_fwd, ca_reference_rows, causal_pairs)


def _rand(shape, seed, dtype=torch.float64):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=dtype)


def test_whole_doc_equals_sdpa():
    """Lq == Lk, Hq == Hkv: per-document torch SDPA with is_causal=True."""
    lens = [5, 17, 64]
    h, d = 3, 16
    q, k, v = (_rand((sum(lens), h, d), s, torch.float32) for s in (1, 2, 3))
    out, lse = ca_reference_fwd(q, k, v, cu(lens), cu(lens), row_block=7)
    start = 0
    for n in lens:
        sl = slice(start, start + n)
        ref = F.scaled_dot_product_attention(q[sl].permute(1, 0, 2)[None], k[sl].permute(1, 0, 2)[None],
                                             v[sl].permute(1, 0, 2)[None], is_causal=True)[0].permute(1, 0, 2)
        assert torch.allclose(out[sl], ref, atol=2e-6, rtol=1e-5)
        start += n


def test_gqa_equals_repeated_kv_sdpa_and_non_causal():
    n, hq, hkv, d = 40, 6, 2, 8
    q = _rand((n, hq, d), 4, torch.float32)
    k, v = _rand((n, hkv, d), 5, torch.float32), _rand((n, hkv, d), 6, torch.float32)
    kr, vr = k.repeat_interleave(3, dim=1), v.repeat_interleave(3, dim=1)
    for causal in (True, False):
        out, _ = ca_reference_fwd(q, k, v, [0, n], [0, n], causal=causal)
        ref = F.scaled_dot_product_attention(q.permute(1, 0, 2)[None], kr.permute(1, 0, 2)[None], vr.permute(1, 0, 2)[None],
                                             is_causal=causal)[0].permute(1, 0, 2)
        assert torch.allclose(out, ref, atol=2e-6, rtol=1e-5)


def _brute(q, k, v, lq, lk, scale, causal):
    """Scalar loops straight from the definition, one head."""
    out = torch.zeros(lq, q.shape[1], dtype=torch.float64)
    lse = torch.zeros(lq, dtype=torch.float64)
    for i in range(lq):
        js = [j for j in range(lk) if (not causal) or j <= i + (lk - lq)]
        s = [scale * float(sum(q[i, t] * k[j, t] for t in range(q.shape[1]))) for j in js]
        m = max(s)
        z = sum(math.exp(x - m) for x in s)
        lse[i] = m + math.log(z)
        for x, j in zip(s, js):
            out[i] += math.exp(x - lse[i]) * v[j]
    return out, lse


def test_bottom_right_mask_and_lse_brute_force():
    """Lk > Lq: row i sees columns j <= i + (Lk - Lq); LSE is the natural log with the scale inside."""
    lq, lk, d = 3, 7, 4
    q, k, v = _rand((lq, 1, d), 7), _rand((lk, 1, d), 8), _rand((lk, 1, d), 9)
    out, lse = ca_reference_fwd(q, k, v, [0, lq], [0, lk], softmax_scale=0.37, dtype=torch.float64)
    bo, bl = _brute(q[:, 0], k[:, 0], v[:, 0], lq, lk, 0.37, True)
    assert torch.allclose(out[:, 0], bo, atol=1e-12)
    assert torch.allclose(lse[0], bl, atol=1e-12)
    # default scale is D**-0.5
    out2, _ = ca_reference_fwd(q, k, v, [0, lq], [0, lk], dtype=torch.float64)
    bo2, _ = _brute(q[:, 0], k[:, 0], v[:, 0], lq, lk, d ** -0.5, True)
    assert torch.allclose(out2[:, 0], bo2, atol=1e-12)


def test_softmax_rows_sum_to_one_via_lse():
    lq, lk, hq, hkv, d = 9, 20, 4, 2, 8
    q, k, v = _rand((lq, hq, d), 10), _rand((lk, hkv, d), 11), _rand((lk, hkv, d), 12)
    _, lse = ca_reference_fwd(q, k, v, [0, lq], [0, lk], dtype=torch.float64)
    kr = k.repeat_interleave(2, dim=1)
    s = torch.einsum("qhd,khd->hqk", q, kr) * d ** -0.5
    i = torch.arange(lq)[:, None]; j = torch.arange(lk)[None]
    p = torch.exp(s - lse[:, :, None]).masked_fill((j > i + lk - lq)[None], 0)
    assert torch.allclose(p.sum(-1), torch.ones(hq, lq, dtype=torch.float64), atol=1e-12)


def _autograd(q, k, v, do, cu_q, cu_k, causal=True, offs=None):
    q, k, v = (t.clone().requires_grad_(True) for t in (q, k, v))
    hq, hkv = q.shape[1], k.shape[1]
    outs = []
    for b in range(len(cu_q) - 1):
        lq = cu_q[b + 1] - cu_q[b]; lk = cu_k[b + 1] - cu_k[b]
        k0 = offs[b] if offs is not None else cu_k[b]
        qb = q[cu_q[b]:cu_q[b + 1]].permute(1, 0, 2)
        kb = k[k0:k0 + lk].permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        vb = v[k0:k0 + lk].permute(1, 0, 2).repeat_interleave(hq // hkv, 0)
        s = qb @ kb.transpose(1, 2) * q.shape[-1] ** -0.5
        if causal:
            i = torch.arange(lq)[:, None]; j = torch.arange(lk)[None]
            s = s.masked_fill((j > i + lk - lq)[None], float("-inf"))
        outs.append((torch.softmax(s, -1) @ vb).permute(1, 0, 2))
    out = torch.cat(outs)
    out.backward(do)
    return out.detach(), q.grad, k.grad, v.grad


def test_backward_equals_autograd_gqa_prefix_and_alias():
    hq, hkv, d = 4, 2, 8
    q_lens, k_lens = [5, 9, 4], [12, 9, 30]
    cq, ck = cu(q_lens), cu(k_lens)
    q, k, v, do = _rand((18, hq, d), 13), _rand((51, hkv, d), 14), _rand((51, hkv, d), 15), _rand((18, hq, d), 16)
    for causal in (True, False):
        dq, dk, dv = ca_reference_bwd(do, q, k, v, cq, ck, causal=causal, dtype=torch.float64, row_block=4)
        _, aq, ak, av = _autograd(q, k, v, do, cq, ck, causal)
        for a, b in ((dq, aq), (dk, ak), (dv, av)):
            assert torch.allclose(a, b, atol=1e-11)
    # aliased prefixes: three shards of one 18-token document share 18 stored KV rows
    q_lens, k_lens, offs = [5, 9, 4], [5, 14, 18], [0, 0, 0]
    k2, v2 = k[:18], v[:18]
    dq, dk, dv = ca_reference_bwd(do, q, k2, v2, cu(q_lens), cu(k_lens), kv_task_offsets=offs, dtype=torch.float64)
    _, aq, ak, av = _autograd(q, k2, v2, do, cu(q_lens), cu(k_lens), True, offs)
    for a, b in ((dq, aq), (dk, ak), (dv, av)):
        assert torch.allclose(a, b, atol=1e-11)


def test_backward_with_given_out_and_lse_equals_recomputed():
    hq, hkv, d = 4, 2, 8
    q_lens, k_lens = [5, 9], [12, 9]
    q, k, v, do = _rand((14, hq, d), 40), _rand((21, hkv, d), 41), _rand((21, hkv, d), 42), _rand((14, hq, d), 43)
    out, lse = ca_reference_fwd(q, k, v, cu(q_lens), cu(k_lens), dtype=torch.float64)
    a = ca_reference_bwd(do, q, k, v, cu(q_lens), cu(k_lens), dtype=torch.float64)
    b = ca_reference_bwd(do, q, k, v, cu(q_lens), cu(k_lens), dtype=torch.float64, out=out, softmax_lse=lse)
    for x, y in zip(a, b):
        assert torch.allclose(x, y, atol=1e-12)


def test_backward_finite_differences():
    hq, hkv, d = 2, 1, 4
    q, k, v, do = _rand((3, hq, d), 17), _rand((6, hkv, d), 18), _rand((6, hkv, d), 19), _rand((3, hq, d), 20)
    cq, ck = [0, 3], [0, 6]
    dq, dk, dv = ca_reference_bwd(do, q, k, v, cq, ck, dtype=torch.float64)

    def loss(q_, k_, v_):
        o, _ = ca_reference_fwd(q_, k_, v_, cq, ck, dtype=torch.float64)
        return (o * do).sum().item()

    eps = 1e-6
    for t, g, idx in ((q, dq, (1, 1, 2)), (k, dk, (4, 0, 1)), (v, dv, (0, 0, 3)), (k, dk, (5, 0, 0))):
        tp, tm = t.clone(), t.clone()
        tp[idx] += eps; tm[idx] -= eps
        args_p = [tp if x is t else x for x in (q, k, v)]
        args_m = [tm if x is t else x for x in (q, k, v)]
        fd = (loss(*args_p) - loss(*args_m)) / (2 * eps)
        assert abs(fd - g[idx].item()) < 1e-7


def test_sharded_equals_whole_document():
    """Cutting a document into CA tasks (shard + KV prefix) and concatenating the outputs gives
    whole-document causal attention; summing dK/dV over the aliased prefixes gives whole-doc dK/dV."""
    n, hq, hkv, d = 50, 4, 2, 8
    q, k, v, do = _rand((n, hq, d), 21), _rand((n, hkv, d), 22), _rand((n, hkv, d), 23), _rand((n, hq, d), 24)
    whole, wl = ca_reference_fwd(q, k, v, [0, n], [0, n], dtype=torch.float64)
    cuts = [13, 20, 17]
    ends = np.cumsum(cuts)
    sh, sl = ca_reference_fwd(q, k, v, cu(cuts), cu(ends), kv_task_offsets=[0, 0, 0], dtype=torch.float64)
    assert torch.allclose(sh, whole, atol=1e-12) and torch.allclose(sl, wl, atol=1e-12)
    g1 = ca_reference_bwd(do, q, k, v, [0, n], [0, n], dtype=torch.float64)
    g2 = ca_reference_bwd(do, q, k, v, cu(cuts), cu(ends), kv_task_offsets=[0, 0, 0], dtype=torch.float64)
    for a, b in zip(g1, g2):
        assert torch.allclose(a, b, atol=1e-11)
    # duplicated prefixes (the reference's layout) + summing the copies = the aliased result
    kd = torch.cat([k[:e] for e in ends]); vd = torch.cat([v[:e] for e in ends])
    g3 = ca_reference_bwd(do, q, kd, vd, cu(cuts), cu(ends), dtype=torch.float64)
    dk_sum = torch.zeros_like(k); dv_sum = torch.zeros_like(v)
    pos = 0
    for e in ends:
        dk_sum[:e] += g3[1][pos:pos + e]; dv_sum[:e] += g3[2][pos:pos + e]; pos += e
    assert torch.allclose(dk_sum, g1[1], atol=1e-11) and torch.allclose(dv_sum, g1[2], atol=1e-11)


def test_row_sampler_matches_full():
    hq, hkv, d = 4, 2, 8
    q_lens, k_lens = [11, 6], [20, 6]
    q, k, v, do = _rand((17, hq, d), 25), _rand((26, hkv, d), 26), _rand((26, hkv, d), 27), _rand((17, hq, d), 28)
    out, lse = ca_reference_fwd(q, k, v, cu(q_lens), cu(k_lens), dtype=torch.float64)
    dq, _, _ = ca_reference_bwd(do, q, k, v, cu(q_lens), cu(k_lens), dtype=torch.float64)
    o, l, g = ca_reference_rows(q, k, v, do, cu(q_lens), cu(k_lens), 0, 3, 9, dtype=torch.float64)
    assert torch.allclose(o, out[3:9]) and torch.allclose(l, lse[:, 3:9]) and torch.allclose(g, dq[3:9])


def test_row_sampler_with_saved_forward_results_matches_full():
    """The out_rows= / lse_rows= branch (what every full-size dq check on the GPU goes through) against
    ca_reference_bwd(out=, softmax_lse=), itself pinned by autograd above when out and lse are exact.
    The saved results are perturbed (bf16-rounded out, lse off by up to 1e-2) so that the branch is observably
    different from recomputing them: the same rows without the saved results must NOT match."""
    hq, hkv, d = 4, 2, 8
    q_lens, k_lens = [11, 6], [20, 6]
    q, k, v, do = _rand((17, hq, d), 25), _rand((26, hkv, d), 26), _rand((26, hkv, d), 27), _rand((17, hq, d), 28)
    out, lse = ca_reference_fwd(q, k, v, cu(q_lens), cu(k_lens), dtype=torch.float64)
    out_s = out.to(torch.bfloat16).double()
    lse_s = lse + 1e-2 * torch.sin(torch.arange(lse.numel(), dtype=torch.float64)).reshape(lse.shape)
    dq, _, _ = ca_reference_bwd(do, q, k, v, cu(q_lens), cu(k_lens), dtype=torch.float64, out=out_s, softmax_lse=lse_s)
    for task, r0, r1, g0 in ((0, 3, 9, 3), (0, 0, 11, 0), (1, 2, 6, 13)):
        _, _, g = ca_reference_rows(q, k, v, do, cu(q_lens), cu(k_lens), task, r0, r1, dtype=torch.float64,
                                    out_rows=out_s[g0:g0 + r1 - r0], lse_rows=lse_s[:, g0:g0 + r1 - r0])
        assert torch.allclose(g, dq[g0:g0 + r1 - r0], atol=1e-12)
        _, _, g_plain = ca_reference_rows(q, k, v, do, cu(q_lens), cu(k_lens), task, r0, r1, dtype=torch.float64)
        assert not torch.allclose(g_plain, dq[g0:g0 + r1 - r0], atol=1e-6)


@pytest.mark.parametrize("causal", [True, False])
def test_key_row_sampler_matches_full(causal):
    """ca_reference_key_rows (dK/dV of a few keys of one task and kv head, from the query rows that see them)
    against the same rows of ca_reference_bwd(out=, softmax_lse=), for a prefix task (lk > lq), for a whole
    document, with perturbed saved results, with only the rows past the keys' horizon handed in, and in
    several row blocks."""
    hq, hkv, d = 6, 2, 8
    g = hq // hkv
    q_lens, k_lens = [11, 9], [20, 9]
    cq, ck = cu(q_lens), cu(k_lens)
    q, k, v, do = _rand((20, hq, d), 41), _rand((29, hkv, d), 42), _rand((29, hkv, d), 43), _rand((20, hq, d), 44)
    out, lse = ca_reference_fwd(q, k, v, cq, ck, dtype=torch.float64, causal=causal)
    out_s = out.to(torch.bfloat16).double()
    lse_s = lse + 1e-2 * torch.cos(torch.arange(lse.numel(), dtype=torch.float64)).reshape(lse.shape)
    _, dk, dv = ca_reference_bwd(do, q, k, v, cq, ck, dtype=torch.float64, out=out_s, softmax_lse=lse_s, causal=causal)
    for task, key0, key1 in ((0, 0, 4), (0, 12, 17), (0, 17, 20), (1, 3, 9)):
        lq, lk = q_lens[task], k_lens[task]
        q0, k0 = int(cq[task]), int(ck[task])
        first = max(0, key0 - (lk - lq)) if causal else 0          # rows before it see none of the keys
        for kvh in range(hkv):
            hs = slice(kvh * g, (kvh + 1) * g)
            rows = slice(q0 + first, q0 + lq)
            gk, gv = ca_reference_key_rows(q[rows, hs], do[rows, hs], out_s[rows, hs], lse_s[hs, rows],
                                           k[k0 + key0:k0 + key1, kvh], v[k0 + key0:k0 + key1, kvh], first, lq, lk, key0,
                                           causal=causal, row_block=4, dtype=torch.float64)
            assert torch.allclose(gk, dk[k0 + key0:k0 + key1, kvh], atol=1e-12)
            assert torch.allclose(gv, dv[k0 + key0:k0 + key1, kvh], atol=1e-12)


def test_empty_rows_when_lk_lt_lq():
    """Rows that see no key give out = 0 and lse = -inf."""
    q, k, v = _rand((4, 1, 4), 29), _rand((2, 1, 4), 30), _rand((2, 1, 4), 31)
    out, lse = ca_reference_fwd(q, k, v, [0, 4], [0, 2], dtype=torch.float64)
    assert torch.all(out[:2] == 0) and torch.all(torch.isinf(lse[0, :2])) and torch.all(torch.isfinite(lse[0, 2:]))


def test_pair_count_and_flops():
    """cfg-1 figure quoted for the metric: 131 328 + 524 800 + 3 278 080 pairs -> 6.446e10 fwd FLOP."""
    assert [causal_pairs(n, n) for n in (512, 1024, 2560)] == [131328, 524800, 3278080]
    assert causal_pairs(3, 7) == 3 * 7 - 3  # rows see 5, 6, 7 keys
    fwd, bwd = attention_flops(cu([512, 1024, 2560]), cu([512, 1024, 2560]), 32, 128)
    assert fwd == 4 * 32 * 128 * 3934208 and bwd == 10 * 32 * 128 * 3934208


def test_linearity_identities_hold_and_catch_a_dropped_tile():
    """<V,dV> = <O,dO> and <Q,dQ> = <K,dK> per (task, kv head) for bf16-rounded oracle results;
    removing one 64-key tile's contribution to dV of a 300-token task breaks the first."""
    from helpers import assert_identity, task_sums
    q_lens = [300, 70]
    q, k, v, do = make_qkv(370, 370, 4, 2, 128, 3)
    out, lse = ca_reference_fwd(q, k, v, cu(q_lens), cu(q_lens))
    dq, dk, dv = ca_reference_bwd(do, q, k, v, cu(q_lens), cu(q_lens))
    r = lambda x: x.to(torch.bfloat16)
    c = cu(q_lens)
    assert_identity(task_sums(v, r(dv), c, 2), task_sums(r(out), do, c, 2), "vdv")
    assert_identity(task_sums(q, r(dq), c, 2), task_sums(k, r(dk), c, 2), "qdq")
    # dV without the contribution of query rows 128..255 to keys 64..127 (one tile of one head group)
    _, _, dv_part = ca_reference_bwd(do[128:256], q[128:256], k[:256], v[:256], [0, 128], [0, 256])
    broken = dv.clone()
    broken[64:128] -= dv_part[64:128]
    with pytest.raises(AssertionError):
        assert_identity(task_sums(v, r(broken), c, 2), task_sums(r(out), do, c, 2), "vdv")
