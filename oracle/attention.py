"""CPU oracle for core attention over a batch of CA tasks.  TEST INFRASTRUCTURE ONLY.

Nothing in the product path may import this module; it exists so that tests, the
smoke check and the bench's CPU-baseline leg have an independent statement of the
arithmetic to compare the HIP kernels with.

What it restates.  The reference never computes attention itself: it hands packed
q/k/v and cu_seqlens to flash-attn 2.7.4 (third-party, pinned in
README.Installation.md:136-140, source absent from the reference tree) at
distca/runtime/megatron/ops/fused_comm_attn.py:151-197 (forward) and :259-272
(backward).  This file therefore restates flash-attn's *published* semantics for
that call: per task b and q-head h (kv-head h // (Hq/Hkv)),

    s_ij  = scale * <q_i, k_j>              scale = D**-0.5 (fused_comm_attn.py:121-123)
    seen  = j <= i + (Lk - Lq)              bottom-right causal (per_doc_cp_attn.py:326,406-411)
    LSE_i = log sum_j exp(s_ij)             natural log, scale included
    O_i   = sum_j exp(s_ij - LSE_i) v_j
    D_i   = <dO_i, O_i>
    dS_ij = P_ij (<dO_i, v_j> - D_i)
    dQ_i  = scale sum_j dS_ij k_j ;  dK_j = scale sum_h sum_i dS_ij q_i ;  dV_j = sum_h sum_i P_ij dO_i

with task b's rows q[cu_q[b]:cu_q[b+1]] and keys k[ks:ks+Lk], Lk = cu_k[b+1]-cu_k[b],
ks = kv_offsets[b] if given else cu_k[b]  (task = shard + KV prefix,
distca/runtime/compute_metadata.py:404-448; cu_seqlens construction :326-365).

Parity status: the reference holds no golden vectors for attention, so these
functions are pinned by mathematics only (tests/test_oracle_attention.py):
torch SDPA for whole documents, torch.autograd and finite differences for the
gradients, a brute-force scalar loop on tiny shapes, the sharded-vs-whole-document
identity the reference asserts at tests/test_megatron_layer.py:169,244-251, and
sum_j exp(s_ij - LSE_i) = 1.  Against flash-attn itself: parity unpinned.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import torch


def _task_ranges(cu_q, cu_k, kv_offsets, b):
    q0, q1 = int(cu_q[b]), int(cu_q[b + 1])
    lk = int(cu_k[b + 1]) - int(cu_k[b])
    k0 = int(kv_offsets[b]) if kv_offsets is not None else int(cu_k[b])
    return q0, q1, k0, k0 + lk


def _scores(qb, kb, scale, causal, row0, lq, lk):
    """qb [H, R, D] (rows row0..row0+R of the task), kb [H, Lk, D] -> masked scores [H, R, Lk]."""
    s = torch.matmul(qb, kb.transpose(1, 2)) * scale
    if causal:
        i = torch.arange(row0, row0 + qb.shape[1]).unsqueeze(1)
        j = torch.arange(lk).unsqueeze(0)
        s = s.masked_fill((j > i + (lk - lq)).unsqueeze(0), float("-inf"))
    return s


def ca_reference_fwd(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
    cu_seqlens_q: Sequence[int], cu_seqlens_k: Sequence[int],
    softmax_scale: Optional[float] = None, causal: bool = True,
    kv_task_offsets: Optional[Sequence[int]] = None,
    row_block: int = 1024, dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """q [Tq,Hq,D], k,v [Tk,Hkv,D] (any float dtype) -> out [Tq,Hq,D], lse [Hq,Tq], both in `dtype`.

    Follows the call at fused_comm_attn.py:151-197 (argument meaning) and the output
    contract used at :339-383 (LSE as [Hq, Tq] / [Tq, Hq])."""
    tq, hq, d = q.shape
    hkv = k.shape[1]
    g = hq // hkv
    scale = softmax_scale if softmax_scale is not None else d ** -0.5
    out = torch.zeros(tq, hq, d, dtype=dtype)
    lse = torch.full((hq, tq), float("-inf"), dtype=dtype)
    nb = len(cu_seqlens_q) - 1
    for b in range(nb):
        q0, q1, k0, k1 = _task_ranges(cu_seqlens_q, cu_seqlens_k, kv_task_offsets, b)
        lq, lk = q1 - q0, k1 - k0
        if lq == 0:
            continue
        kb = k[k0:k1].to(dtype).permute(1, 0, 2).repeat_interleave(g, dim=0)  # [Hq, Lk, D]
        vb = v[k0:k1].to(dtype).permute(1, 0, 2).repeat_interleave(g, dim=0)
        for r0 in range(0, lq, row_block):
            r1 = min(lq, r0 + row_block)
            qb = q[q0 + r0:q0 + r1].to(dtype).permute(1, 0, 2)  # [Hq, R, D]
            s = _scores(qb, kb, scale, causal, r0, lq, lk)
            l = torch.logsumexp(s, dim=-1)  # [Hq, R]
            p = torch.exp(s - l.unsqueeze(-1))
            p = torch.nan_to_num(p, nan=0.0)  # rows that see no key (Lk < Lq): out 0, lse -inf
            out[q0 + r0:q0 + r1] = torch.matmul(p, vb).permute(1, 0, 2)
            lse[:, q0 + r0:q0 + r1] = l
    return out, lse


def ca_reference_bwd(
    dout: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
    cu_seqlens_q: Sequence[int], cu_seqlens_k: Sequence[int],
    softmax_scale: Optional[float] = None, causal: bool = True,
    kv_task_offsets: Optional[Sequence[int]] = None,
    row_block: int = 1024, dtype: torch.dtype = torch.float32,
    out: Optional[torch.Tensor] = None, softmax_lse: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Closed-form gradients (dq [Tq,Hq,D], dk, dv [Tk,Hkv,D]) in `dtype`.

    With `out` [Tq,Hq,D] and `softmax_lse` [Hq,Tq] given, they are used the way the
    flash-attn backward uses the tensors the reference hands it (fused_comm_attn.py:259-261:
    dout, q, k, v, out, softmax_lse): D_i = <dO_i, out_i> and P_ij = exp(s_ij - lse_i),
    instead of being recomputed from q, k, v.  With exact fp32 out/lse both forms agree.

    Restates what the flash-attn varlen backward invoked at fused_comm_attn.py:259-272
    returns; GQA heads are summed into their kv head, and with aliased KV prefixes
    (kv_task_offsets) every task adds into the rows it read — the quantity the
    reference forms with duplicated copies plus inplace_grad_sum_kernel
    (csrc/core/memcpy.cu:158-236)."""
    tq, hq, d = q.shape
    tk, hkv, _ = k.shape
    g = hq // hkv
    scale = softmax_scale if softmax_scale is not None else d ** -0.5
    dq = torch.zeros(tq, hq, d, dtype=dtype)
    dk = torch.zeros(tk, hkv, d, dtype=dtype)
    dv = torch.zeros(tk, hkv, d, dtype=dtype)
    nb = len(cu_seqlens_q) - 1
    for b in range(nb):
        q0, q1, k0, k1 = _task_ranges(cu_seqlens_q, cu_seqlens_k, kv_task_offsets, b)
        lq, lk = q1 - q0, k1 - k0
        if lq == 0:
            continue
        kb = k[k0:k1].to(dtype).permute(1, 0, 2).repeat_interleave(g, dim=0)
        vb = v[k0:k1].to(dtype).permute(1, 0, 2).repeat_interleave(g, dim=0)
        dkb = torch.zeros_like(kb)
        dvb = torch.zeros_like(vb)
        for r0 in range(0, lq, row_block):
            r1 = min(lq, r0 + row_block)
            qb = q[q0 + r0:q0 + r1].to(dtype).permute(1, 0, 2)
            dob = dout[q0 + r0:q0 + r1].to(dtype).permute(1, 0, 2)
            s = _scores(qb, kb, scale, causal, r0, lq, lk)
            if softmax_lse is not None:
                l = softmax_lse[:, q0 + r0:q0 + r1].to(dtype).unsqueeze(-1)
            else:
                l = torch.logsumexp(s, dim=-1, keepdim=True)
            p = torch.nan_to_num(torch.exp(s - l), nan=0.0)
            if out is not None:
                ob = out[q0 + r0:q0 + r1].to(dtype).permute(1, 0, 2)
            else:
                ob = torch.matmul(p, vb)
            delta = (dob * ob).sum(-1, keepdim=True)
            dp = torch.matmul(dob, vb.transpose(1, 2))
            ds = p * (dp - delta)
            dq[q0 + r0:q0 + r1] = (torch.matmul(ds, kb) * scale).permute(1, 0, 2)
            dkb += torch.matmul(ds.transpose(1, 2), qb) * scale
            dvb += torch.matmul(p.transpose(1, 2), dob)
        dk[k0:k1] += dkb.reshape(hkv, g, lk, d).sum(1).permute(1, 0, 2)
        dv[k0:k1] += dvb.reshape(hkv, g, lk, d).sum(1).permute(1, 0, 2)
    return dq, dk, dv


def ca_reference_rows(
    q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, dout: Optional[torch.Tensor],
    cu_seqlens_q: Sequence[int], cu_seqlens_k: Sequence[int], task: int, row0: int, row1: int,
    softmax_scale: Optional[float] = None, causal: bool = True,
    kv_task_offsets: Optional[Sequence[int]] = None, dtype: torch.dtype = torch.float32,
    out_rows: Optional[torch.Tensor] = None, lse_rows: Optional[torch.Tensor] = None,
):
    """Rows [row0,row1) of one task against its full KV prefix: (out, lse, dq) for those
    rows (dq None without dout).  Used to spot-check long tasks whose full fp32
    evaluation would take hours on host cores; same formulas as above.  With `out_rows`
    [rows, Hq, D] and `lse_rows` [Hq, rows] the gradient is formed from those saved forward
    results, as ca_reference_bwd does with out= / softmax_lse=."""
    hq, d = q.shape[1], q.shape[2]
    g = hq // k.shape[1]
    scale = softmax_scale if softmax_scale is not None else d ** -0.5
    q0, q1, k0, k1 = _task_ranges(cu_seqlens_q, cu_seqlens_k, kv_task_offsets, task)
    lq, lk = q1 - q0, k1 - k0
    kb = k[k0:k1].to(dtype).permute(1, 0, 2).repeat_interleave(g, dim=0)
    vb = v[k0:k1].to(dtype).permute(1, 0, 2).repeat_interleave(g, dim=0)
    qb = q[q0 + row0:q0 + row1].to(dtype).permute(1, 0, 2)
    s = _scores(qb, kb, scale, causal, row0, lq, lk)
    l = torch.logsumexp(s, dim=-1, keepdim=True)
    p = torch.nan_to_num(torch.exp(s - l), nan=0.0)
    ob = torch.matmul(p, vb)
    dqb = None
    if dout is not None:
        dob = dout[q0 + row0:q0 + row1].to(dtype).permute(1, 0, 2)
        o_used = ob if out_rows is None else out_rows.to(dtype).permute(1, 0, 2)
        p_used = p if lse_rows is None else torch.nan_to_num(torch.exp(s - lse_rows.to(dtype).unsqueeze(-1)), nan=0.0)
        delta = (dob * o_used).sum(-1, keepdim=True)
        ds = p_used * (torch.matmul(dob, vb.transpose(1, 2)) - delta)
        dqb = (torch.matmul(ds, kb) * scale).permute(1, 0, 2)
    return ob.permute(1, 0, 2), l.squeeze(-1), dqb


def ca_reference_key_rows(
    q_rows: torch.Tensor, dout_rows: torch.Tensor, out_rows: torch.Tensor, lse_rows: torch.Tensor,
    k_rows: torch.Tensor, v_rows: torch.Tensor, row0: int, lq: int, lk: int, key0: int,
    softmax_scale: Optional[float] = None, causal: bool = True, row_block: int = 16384,
    dtype: torch.dtype = torch.float32,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """dK, dV of a few keys of one task, for one kv head: the column view of ca_reference_bwd.

    k_rows, v_rows [n, D]: keys key0 .. key0+n of the task (positions inside its prefix of lk keys).
    q_rows, dout_rows, out_rows [R, G, D] and lse_rows [G, R]: query rows row0 .. row0+R of the task
    (of its lq rows) for the G query heads of that kv head; the caller passes every row that sees one
    of the keys (with the causal mask: rows >= key0 - (lk - lq)) -- rows it leaves out contribute
    nothing to the result.  Gradients are formed from the saved forward results (out, lse) the way the
    flash-attn backward invoked at fused_comm_attn.py:259-272 forms them:
        P_ij = exp(s_ij - lse_i), D_i = <dO_i, out_i>, dS_ij = P_ij (<dO_i, v_j> - D_i),
        dV_j = sum_{h, i} P_ij dO_i,  dK_j = scale sum_{h, i} dS_ij q_i.
    Exists so that sampled dK/dV rows of tasks too long for the full fp32 evaluation can be checked."""
    r, g, d = q_rows.shape
    n = k_rows.shape[0]
    scale = softmax_scale if softmax_scale is not None else d ** -0.5
    kb = k_rows.to(dtype)
    vb = v_rows.to(dtype)
    dk = torch.zeros(n, d, dtype=dtype)
    dv = torch.zeros(n, d, dtype=dtype)
    j = torch.arange(key0, key0 + n).unsqueeze(0)
    for a in range(0, r, row_block):
        b = min(r, a + row_block)
        qb = q_rows[a:b].to(dtype).permute(1, 0, 2)        # [G, R', D]
        dob = dout_rows[a:b].to(dtype).permute(1, 0, 2)
        ob = out_rows[a:b].to(dtype).permute(1, 0, 2)
        l = lse_rows[:, a:b].to(dtype).unsqueeze(-1)       # [G, R', 1]
        s = torch.matmul(qb, kb.t()) * scale               # [G, R', n]
        if causal:
            i = torch.arange(row0 + a, row0 + b).unsqueeze(1)
            s = s.masked_fill((j > i + (lk - lq)).unsqueeze(0), float("-inf"))
        p = torch.nan_to_num(torch.exp(s - l), nan=0.0)
        delta = (dob * ob).sum(-1, keepdim=True)
        ds = p * (torch.matmul(dob, vb.t()) - delta)
        dv += torch.matmul(p.transpose(1, 2), dob).sum(0)
        dk += torch.matmul(ds.transpose(1, 2), qb).sum(0) * scale
    return dk, dv


def causal_pairs(lq: int, lk: int, causal: bool = True) -> int:
    """Visible (query,key) pairs of one task: Lq*Lk - Lq(Lq-1)/2 under the bottom-right
    causal mask with Lk >= Lq — the work unit of Item.get_flops,
    distca/planner/planner.py:366-378."""
    if not causal:
        return lq * lk
    if lk >= lq:
        return lq * lk - lq * (lq - 1) // 2
    return lk * (lk + 1) // 2  # only the last Lk rows see anything


def attention_flops(cu_q, cu_k, hq: int, d: int, causal: bool = True):
    """(fwd, bwd) algorithmic FLOPs: 4*Hq*D*pairs and 10*Hq*D*pairs."""
    pairs = sum(
        causal_pairs(int(cu_q[b + 1]) - int(cu_q[b]), int(cu_k[b + 1]) - int(cu_k[b]), causal)
        for b in range(len(cu_q) - 1)
    )
    return 4 * hq * d * pairs, 10 * hq * d * pairs
