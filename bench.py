#!/usr/bin/env python3
"""Benchmark of the CA-server hot path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input: varlen causal
attention forward + backward over the CA-task batch of the benchmark configuration
"Llama-3-8B heads, 131 072 packed tokens" (32 q heads / 8 kv heads, head_dim 128, bf16,
document lengths lognormal(8, 1.5) clipped to [128, 65 536]).  Inputs are resident in HBM
before the timed region.  One JSON line is printed on stdout; a human-readable table goes
to stderr.

Algorithmic work: causal pairs P = sum_tasks [Lq*Lk - Lq(Lq-1)/2]; forward 4*Hq*D*P FLOP,
backward 10*Hq*D*P FLOP.  `roofline` describes the dominant kernels, the two that make up the
attention backward (ca_bwd_dkdv64_kernel over key blocks, ca_bwd_dq64_kernel over query blocks):
algorithmic backward FLOPs over the sum of their launch durations, measured live by HIP events
the library records on the launch stream.  Both recompute S and dP, so together they execute
14*Hq*D*P FLOP for 10*Hq*D*P of algorithmic work; `executed_tflops` reports that rate per kernel.
`traffic` is the HBM bytes per backward (both kernels) measured once with rocprofv3 --pmc on
the default workload and scaled by a copy kernel of known size; null for other sizes.  `cpu_baseline` times the CPU oracle (per-document fp32 PyTorch attention,
forward + backward) on this box's host cores over a bounded sample of the same documents.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E
# HBM bytes per launch on the default 131072-token workload: rocprofv3 --pmc FETCH_SIZE (x2.000) and
# WRITE_SIZE (x1.000), factors from the pack kernels' known copy sizes in the same run
MEASURED_TRAFFIC_BYTES = {"ca_fwd_kernel": 10.95e9, "ca_bwd_dkdv64_kernel": 22.69e9, "ca_bwd_dq64_kernel": 13.24e9}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def cpu_baseline(batch, budget_s: float, seed: int):
    """Oracle forward+backward on host cores over the shortest documents of the batch until
    about `budget_s` seconds have been spent; TFLOP/s over the FLOPs actually executed."""
    import torch
    from oracle.attention import ca_reference_bwd, ca_reference_fwd, causal_pairs
    hq, hkv, d = batch.num_heads_q, batch.num_heads_kv, batch.head_dim
    order = np.argsort(batch.q_lens, kind="stable")
    g = torch.Generator().manual_seed(seed)
    spent, flops, docs, tokens = 0.0, 0, 0, 0
    for b in order:
        n = int(batch.q_lens[b])
        if n > 8192:
            break
        q = torch.randn((n, hq, d), generator=g).to(torch.bfloat16)
        k = torch.randn((n, hkv, d), generator=g).to(torch.bfloat16)
        v = torch.randn((n, hkv, d), generator=g).to(torch.bfloat16)
        do = torch.randn((n, hq, d), generator=g).to(torch.bfloat16)
        t0 = time.perf_counter()
        ca_reference_fwd(q, k, v, [0, n], [0, n])
        ca_reference_bwd(do, q, k, v, [0, n], [0, n])
        spent += time.perf_counter() - t0
        flops += 14 * hq * d * causal_pairs(n, n)
        docs += 1
        tokens += n
        if spent >= budget_s:
            break
    return {
        "value": round(flops / max(spent, 1e-9) / 1e12, 5), "unit": "TFLOP/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"oracle fwd+bwd (fp32 PyTorch, per document) on the {docs} shortest documents of the workload "
                  f"({tokens} tokens, {flops:.3e} FLOP) in {spent:.1f} s",
    }


def _timed(torch, _lib, timer, fn, iters):
    for _ in range(2):
        fn()
    torch.cuda.synchronize()
    _lib.timing_read(timer)
    _lib.timing_enable(True)
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    _lib.timing_enable(False)
    ms, launches = _lib.timing_read(timer)
    return ms / iters, launches // iters


def _rate(bytes_moved, ms):
    gbps = bytes_moved / (ms * 1e-3) / 1e9
    return {"GB/s": round(gbps, 1), "frac_hbm_peak": round(gbps / PEAK_HBM_GBPS, 4), "ms_per_pass": round(ms, 4)}


def pack_unpack_bench(torch, dev, iters: int = 10):
    """The HBM-bound kernels of the path on 262 144 tokens, GB/s over algorithmic bytes (kernel durations by HIP events
    on the launch stream):
      pack / unpack   q (8 192 B per token) + k, v (2 048 B each) against one buffer, bytes = 2 x payload; one launch for
                      the three tensors (what the server tick issues), and as three launches (the reference's call shape);
      memcpy_cp       replicating pack of k to up to 2 destinations per shard (every shard to the first, every other
                      shard to the second too) and the unpack into replica planes, bytes = 2 x bytes of live replicas;
      grad_sum        a third of the rows are main shards with 2 duplicate copies each, bytes = (2 + copies) x rows x
                      token bytes per main shard."""
    from distca_amd import _lib
    from distca_amd.ops import a2a_memcpy_cp, a2a_memcpy_non_cp, a2a_memcpy_non_cp_multi, pre_a2a_grad_acc
    from distca_amd.workloads import config4_pack
    lay = config4_pack()
    T = lay.num_tokens
    names = list(lay.token_bytes)
    tens = {n: torch.randint(-32768, 32767, (T, tb // 2), dtype=torch.int16, device=dev).view(torch.bfloat16)
            for n, tb in lay.token_bytes.items()}
    buf = torch.empty(lay.buffer_bytes, dtype=torch.uint8, device=dev)
    lens = torch.from_numpy(lay.seq_tokens).to(dev)
    offs = {n: torch.from_numpy(o).to(dev) for n, o in lay.offsets.items()}
    payload = sum(T * tb for tb in lay.token_bytes.values())
    res = {}
    for direction, to_buf in (("pack", True), ("unpack", False)):
        ms, n1 = _timed(torch, _lib, _lib.TIMER_MEMCPY_NON_CP, lambda: a2a_memcpy_non_cp_multi(
            [tens[n] for n in names], [offs[n] for n in names], [lens] * len(names), to_buf, buffer=buf), iters)
        res[direction] = dict(_rate(2 * payload, ms), launches_per_pass=n1)
        ms3, n3 = _timed(torch, _lib, _lib.TIMER_MEMCPY_NON_CP, lambda: [
            a2a_memcpy_non_cp(tens[n], offs[n], lens, to_buf, buffer=buf) for n in names], iters)
        res[direction]["as_separate_launches"] = dict(_rate(2 * payload, ms3), launches_per_pass=n3)
    res["workload"] = f"{lay.name}: {len(lay.seq_tokens)} shards, payload {payload} B per direction"

    # replicating pack / replica-plane unpack of k
    S, tb = len(lay.seq_tokens), lay.token_bytes["k"]
    do_shard = np.ones((S, 2), dtype=np.int8)
    do_shard[1::2, 1] = 0
    cp_off = np.zeros((2, S), dtype=np.int64)
    cur = 0
    for c in range(2):
        for sidx in range(S):
            cp_off[c, sidx] = cur
            if do_shard[sidx, c]:
                cur += int(lay.seq_tokens[sidx]) * tb
    live_bytes = cur
    cp_buf = torch.empty(live_bytes, dtype=torch.uint8, device=dev)
    d_do, d_off = torch.from_numpy(do_shard).to(dev), torch.from_numpy(cp_off).to(dev)
    planes = torch.zeros((2, T, tb // 2), dtype=torch.bfloat16, device=dev)
    ms, _ = _timed(torch, _lib, _lib.TIMER_MEMCPY_CP, lambda: a2a_memcpy_cp(tens["k"], d_do, d_off, lens, True, buffer=cp_buf), iters)
    res["memcpy_cp_pack"] = dict(_rate(2 * live_bytes, ms), workload=f"k of {T} tokens x {tb} B, {S} shards, {live_bytes / (T * tb):.2f} replicas per shard")
    ms, _ = _timed(torch, _lib, _lib.TIMER_MEMCPY_CP, lambda: a2a_memcpy_cp(planes, d_do, d_off, lens, False, buffer=cp_buf), iters)
    res["memcpy_cp_unpack"] = _rate(2 * live_bytes, ms)
    del planes, cp_buf

    # duplicate-gradient sum: main shards in the first third of the rows, their two copies in the other two thirds
    main, total = [], 0
    for n in lay.seq_tokens.tolist():
        if total + n > T // 3:
            break
        main.append(n)
        total += n
    m = len(main)
    seq_lens = torch.tensor(main * 3, dtype=torch.int64, device=dev)
    num_copies = torch.tensor([2] * m + [0] * (2 * m), dtype=torch.int32, device=dev)
    starts = np.concatenate([[0], np.cumsum(main)[:-1]]).astype(np.int64)
    copy_start = np.zeros((3 * m, 2), dtype=np.int64)
    copy_start[:m, 0] = total + starts
    copy_start[:m, 1] = 2 * total + starts
    dk = (torch.randn((3 * total, tb // 2), device=dev) * 0.1).to(torch.bfloat16)
    d_cs = torch.from_numpy(copy_start).to(dev)
    ms, _ = _timed(torch, _lib, _lib.TIMER_GRAD_SUM, lambda: pre_a2a_grad_acc(dk, num_copies, d_cs, seq_lens), iters)
    res["grad_sum"] = dict(_rate(4 * total * tb, ms), workload=f"bf16 [{3 * total}, {tb // 2}]: {m} main shards ({total} rows) with 2 copies each")
    return res


def server_tick_bench(torch, dev, batch, q, k, v, do, iters: int = 4, shard_cap: int = 4096, in_place_only: bool = False):
    """The CA server's ticks on the bench workload: every document cut into shards of at most `shard_cap`
    tokens, one CA task per shard reading its document's prefix.  Forward tick = unpack K/V (each stored shard
    once) + attention reading q from the receive buffer and writing [out | lse] tokens into the send buffer;
    backward tick = unpack K/V + attention backward reading [dO | O | lse | q] tokens from the receive buffer,
    writing dq into the send buffer + pack of dk / dv.  Same causal pairs as the attention step above, so the
    tick times compare directly with the kernel times."""
    from distca_amd import metadata
    from distca_amd.dispatch import TokenLayout
    from distca_amd.fused_comm_attn import FlashAttnArgs, ca_server_backward, ca_server_forward
    from distca_amd.ops import a2a_memcpy_non_cp_multi
    hq, hkv, d = batch.num_heads_q, batch.num_heads_kv, batch.head_dim
    docs = [[min(shard_cap, n - a) for a in range(0, n, shard_cap)] for n in (int(x) for x in batch.q_lens)]
    plan = metadata.single_rank_plan(docs, hq, hkv, d)
    fa_params, fmeta, bmeta, (f_recv, f_send, b_recv, b_send) = metadata.server_metas(plan, dev)
    T = plan.num_q_tokens
    flat = lambda x: x.reshape(T, -1)
    i64 = lambda t: t.to(device=dev, dtype=torch.int64)
    stored = i64(plan.stored_shard_tokens)
    first_entry = {}
    for e, s in enumerate(plan.kv_entry_shard.tolist()):
        first_entry.setdefault(s, e)
    first = torch.tensor([first_entry[s] for s in range(len(first_entry))], dtype=torch.int64)

    def fill(recv, q_rows, backward):
        q_off, k_off, v_off, _ = plan.request_layout(backward)
        a2a_memcpy_non_cp_multi([q_rows, flat(k), flat(v)], [i64(q_off), i64(k_off[first]), i64(v_off[first])],
                                [i64(plan.q_seqlens), stored, stored], True, buffer=recv)

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters

    recv = torch.zeros(f_recv, dtype=torch.uint8, device=dev)
    send = torch.zeros(f_send, dtype=torch.uint8, device=dev)
    fill(recv, flat(q), False)
    res = {"tasks": int(plan.q_seqlens.numel()), "documents": len(docs), "shard_cap": shard_cap,
           "stored_kv_rows": T, "kv_rows_one_copy_per_task": plan.num_kv_tokens}
    from distca_amd import _lib
    fa_det = FlashAttnArgs(hq, hkv, d, deterministic=True)      # the reference's server default (fused_comm_attn.py:95-104)

    def timed_with_kernels(fn, timers):
        """(tick time, time of the attention kernels inside it), both per tick, over the same `iters` ticks."""
        fn()
        torch.cuda.synchronize()
        _lib.timing_enable(True)
        for t in timers:
            _lib.timing_read(t)
        total = timed(fn)
        kern = sum(_lib.timing_read(t)[0] for t in timers) / (iters + 1)     # timed() warms up once more
        _lib.timing_enable(False)
        return round(total, 3), round(kern, 3)

    fwd_timers, bwd_timers = (_lib.TIMER_CA_FWD,), (_lib.TIMER_CA_BWD_DQ, _lib.TIMER_CA_BWD)
    res["forward_ms"], res["forward_attention_kernel_ms"] = timed_with_kernels(
        lambda: ca_server_forward(recv, send, fmeta, fa_params, fa_det), fwd_timers)
    if not in_place_only:
        res["forward_kv_unpacked_ms"], res["forward_kv_unpacked_attention_kernel_ms"] = timed_with_kernels(
            lambda: ca_server_forward(recv, send, fmeta, fa_params, fa_det, kv_shards_in_place=False), fwd_timers)
    out, lse = ca_server_forward(recv, send, fmeta, fa_params, fa_det, in_place=False)
    del recv, send
    request = TokenLayout.of([flat(do), out, lse.T.contiguous(), flat(q)]).merge([flat(do), out, lse.T.contiguous(), flat(q)])
    del out, lse
    recv = torch.zeros(b_recv, dtype=torch.uint8, device=dev)
    fill(recv, request, True)
    del request
    send = torch.zeros(b_send, dtype=torch.uint8, device=dev)
    bwd = lambda **kw: ca_server_backward(recv, send, bmeta, fa_det, fa_params.cu_seqlens_q, fa_params.cu_seqlens_kv,
                                          fa_params.max_seqlen_q, fa_params.max_seqlen_kv, **kw)
    res["backward_ms"], res["backward_attention_kernels_ms"] = timed_with_kernels(lambda: bwd(), bwd_timers)
    if not in_place_only:
        res["backward_kv_unpacked_ms"], res["backward_kv_unpacked_attention_kernels_ms"] = timed_with_kernels(
            lambda: bwd(kv_shards_in_place=False), bwd_timers)
    res["ticks_timed_per_form"] = iters + 2
    res["note"] = ("deterministic ticks (the reference's default).  forward_ms / backward_ms: everything in place: query and "
                   "request tokens and K/V shards read where they lie in the receive buffer, [out | lse], dq and the shards' "
                   "dk / dv written where they belong in the send buffer, no pack kernel; *_kv_unpacked_ms: every stored K/V "
                   "shard unpacked once into a tensor first, dk / dv packed afterwards; *_attention_kernel(s)_ms: the attention "
                   "kernels' own share of the tick above it, by events around them")
    return res


def mfma_probe(torch, _lib, dev, executed_tflops: float, rounds: int = 5, warm_seconds: float = 0.6):
    """What this device delivers for the MFMA instruction itself, measured right after the attention steps: a loop of
    MFMAs on every SIMD, alone and with other work in every MFMA's shadow.  The shader clock under such a load takes a
    few hundred milliseconds to settle at what the power limit allows, so the MFMA-only loop first runs for
    `warm_seconds`; the four variants are then run interleaved, round after round, and the median and the spread over
    the rounds are reported per variant (so that a clock still drifting cannot favour whichever variant runs last)."""
    scratch = torch.zeros(4, dtype=torch.int64, device=dev)
    stream_ptr = torch.cuda.current_stream().cuda_stream
    kinds = (("mfma_only", _lib.PROBE_MFMA_ONLY), ("with_1kb_lds_read_per_mfma", _lib.PROBE_LDS_READ),
             ("with_4_fma_per_mfma", _lib.PROBE_FMA4), ("with_2_exp_per_mfma", _lib.PROBE_EXP2),
             ("with_attention_side_work", _lib.PROBE_MIX))
    iters = 20000
    for _, kind in kinds:    # the first launch of a kernel also loads it
        _lib.probe_mfma_rate(kind, 200, scratch.data_ptr(), stream_ptr)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < warm_seconds:
        _lib.probe_mfma_rate(_lib.PROBE_MFMA_ONLY, iters, scratch.data_ptr(), stream_ptr)
    runs = {name: [] for name, _ in kinds}
    for _ in range(rounds):
        for name, kind in kinds:
            runs[name].append(_lib.probe_mfma_rate(kind, iters, scratch.data_ptr(), stream_ptr))
    probe = {"rounds": rounds}
    for name, _ in kinds:
        tf = sorted(r[0] for r in runs[name])
        probe[name] = {"TFLOP/s": round(float(np.median(tf)), 1), "TFLOP/s_min": round(tf[0], 1), "TFLOP/s_max": round(tf[-1], 1),
                       "cycles_per_mfma": round(float(np.median([r[1] for r in runs[name]])), 2),
                       "clock_GHz": round(float(np.median([r[2] for r in runs[name]])), 3)}
    probe["executed_TFLOP/s_of_the_three_attention_kernels"] = round(executed_tflops, 1)
    probe["executed_over_mfma_only"] = round(executed_tflops / probe["mfma_only"]["TFLOP/s"], 4)
    # with_attention_side_work: beside every MFMA half of a 1 KB LDS read, two multiply-adds, half an exponential and half
    # a conversion, the per-MFMA average of the backward kernels' tile loops (no tile requests, barriers or prologues)
    probe["executed_over_mfma_with_attention_side_work"] = round(executed_tflops / probe["with_attention_side_work"]["TFLOP/s"], 4)
    probe["note"] = (f"v_mfma_f32_32x32x16_bf16 on pseudo-random operands, one wave per SIMD on every SIMD, {8 * iters} per wave and run; "
                     f"{warm_seconds} s of the MFMA-only loop first, then the four variants interleaved for {rounds} rounds: median (min..max) "
                     "rate by HIP events, clock by the device's cycle and real-time counters: what the power limit leaves "
                     "of the published 2.5 PFLOP/s (every pipe busy at 2.4 GHz) on this device for this instruction")
    return probe


def other_workloads_bench(torch, dev, steps: int = 2):
    """The other attention configurations and two batches of short CA tasks through the same entry points: kernel times by
    the library's events (no gaps between launches), algorithmic TFLOP/s.  Parity of these configurations is the
    test suite's business (tests/test_gpu_scale.py); this leg times them where the headline is timed."""
    from distca_amd import _lib
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    from distca_amd import workloads
    short = np.full(128, 1024, dtype=np.int64)
    cases = [
        ("cfg3b_ca_tasks", workloads.config3_ca_tasks(variant="b"), "15 CA tasks over shared K/V prefixes of up to 524288 rows, 262144 query rows, 32q/8kv, deterministic"),
        ("cfg5_llama70b_skewed", workloads.config5_llama70b_skewed(), "524288 tokens with one 262144-token document, 64q/8kv"),
        ("short_documents", workloads.TaskBatch("128x1024", short, short.copy(), 32, 8), "128 whole documents of 1024 tokens, 32q/8kv"),
        ("shards_4096_long_prefixes", workloads.config3_ca_tasks(variant="a", total_q=131072, num_docs=4, max_doc=131072, seed=5013),
         "32 CA tasks of 4096 query rows over shared K/V prefixes of up to 131072 rows, 32q/8kv, deterministic"),
    ]
    res = {}
    for name, b, what in cases:
        hq, hkv, d = b.num_heads_q, b.num_heads_kv, b.head_dim
        gen = torch.Generator(device=dev).manual_seed(7)
        rnd = lambda *shape: torch.randn(shape, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
        q, k, v, do = rnd(b.total_q, hq, d), rnd(b.kv_rows, hkv, d), rnd(b.kv_rows, hkv, d), rnd(b.total_q, hq, d)
        cu_q, cu_k = torch.from_numpy(b.cu_seqlens_q).to(dev), torch.from_numpy(b.cu_seqlens_k).to(dev)
        off = torch.tensor(b.kv_task_offsets, dtype=torch.int32, device=dev) if b.kv_task_offsets is not None else None
        mq, mk = int(b.q_lens.max()), int(b.k_lens.max())
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

        def step():
            out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, mq, mk, None, True, off)
            ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, mq, mk, None, True, off is not None, off, dq, dk, dv)

        step()
        torch.cuda.synchronize()
        timers = (_lib.TIMER_CA_FWD, _lib.TIMER_CA_BWD_DQ, _lib.TIMER_CA_BWD)
        for t in timers:
            _lib.timing_read(t)
        _lib.timing_enable(True)
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        _lib.timing_enable(False)
        fwd, dqk, dkdv = (_lib.timing_read(t)[0] / steps for t in timers)
        f_fwd, f_bwd = b.flops()
        tf = lambda flop, ms: round(flop / (ms * 1e-3) / 1e12, 1)
        res[name] = {"workload": what, "causal_pairs": b.causal_pairs, "steps": steps,
                     "ca_fwd_kernel_ms": round(fwd, 3), "ca_bwd_dq64_kernel_ms": round(dqk, 3), "ca_bwd_dkdv64_kernel_ms": round(dkdv, 3),
                     "fwd_TFLOP/s": tf(f_fwd, fwd), "bwd_TFLOP/s": tf(f_bwd, dqk + dkdv), "fwd_bwd_TFLOP/s": tf(f_fwd + f_bwd, fwd + dqk + dkdv),
                     "pct_of_bf16_mfma_peak": round(100 * (f_fwd + f_bwd) / ((fwd + dqk + dkdv) * 1e-3) / 1e12 / PEAK_BF16_TFLOPS, 2)}
        log(f"  {name:26s} fwd {fwd:9.3f} ms ({res[name]['fwd_TFLOP/s']} TFLOP/s)  bwd {dqk:.3f} + {dkdv:.3f} ms ({res[name]['bwd_TFLOP/s']})  "
            f"fwd+bwd {res[name]['fwd_bwd_TFLOP/s']} TFLOP/s = {res[name]['pct_of_bf16_mfma_peak']} %")
        del q, k, v, do, dq, dk, dv
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--cpu-seconds", type=float, default=15.0, help="budget of the CPU-baseline leg (0 disables)")
    ap.add_argument("--tokens", type=int, default=131072)
    ap.add_argument("--no-pack", action="store_true")
    ap.add_argument("--no-tick", action="store_true")
    ap.add_argument("--no-probe", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the other attention configurations (cfg3b, cfg5, short tasks)")
    ap.add_argument("--tick-in-place-only", action="store_true",
                    help="server-tick leg: only the all-in-place ticks (for a kernel trace that shows them without pack kernels)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the CA-server path; --gpus must be 1 "
                 "(this build has no multi-GPU transport)")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    from distca_amd import _lib
    from distca_amd.fused_comm_attn import ca_varlen_bwd, ca_varlen_fwd
    from distca_amd.workloads import config2_llama8b_128k
    _lib.load()
    dev = torch.device("cuda:0")
    batch = config2_llama8b_128k(total=args.tokens)
    default_workload = args.tokens == 131072
    hq, hkv, d = batch.num_heads_q, batch.num_heads_kv, batch.head_dim
    tq = batch.total_q
    flop_fwd, flop_bwd = batch.flops()
    log(f"workload {batch.name}: {len(batch.q_lens)} docs, max {int(batch.q_lens.max())}, causal pairs {batch.causal_pairs:.4e}, "
        f"fwd {flop_fwd:.4e} FLOP, bwd {flop_bwd:.4e} FLOP")

    gen = torch.Generator(device=dev).manual_seed(1002)
    q = torch.randn((tq, hq, d), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    k = torch.randn((tq, hkv, d), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    v = torch.randn((tq, hkv, d), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    do = torch.randn((tq, hq, d), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
    cu_q = torch.from_numpy(batch.cu_seqlens_q).to(dev)
    cu_k = torch.from_numpy(batch.cu_seqlens_k).to(dev)
    max_q, max_k = int(batch.q_lens.max()), int(batch.k_lens.max())
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)

    def step():
        out, lse = ca_varlen_fwd(q, k, v, cu_q, cu_k, max_q, max_k, None, True)
        ca_varlen_bwd(do, q, k, v, out, lse, cu_q, cu_k, max_q, max_k, None, True, False, None, dq, dk, dv)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    for t in (_lib.TIMER_CA_FWD, _lib.TIMER_CA_BWD, _lib.TIMER_CA_BWD_DQ):
        _lib.timing_read(t)
    _lib.timing_enable(True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    _lib.timing_enable(False)
    fwd_ms, fwd_n = _lib.timing_read(_lib.TIMER_CA_FWD)
    bwd_ms, bwd_n = _lib.timing_read(_lib.TIMER_CA_BWD)
    dq_ms, dq_n = _lib.timing_read(_lib.TIMER_CA_BWD_DQ)
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    tflops = (flop_fwd + flop_bwd) / (ms_per_step * 1e-3) / 1e12
    fwd_k = fwd_ms / max(fwd_n, 1)
    dkdv_k = bwd_ms / max(bwd_n, 1)
    dq_k = dq_ms / max(dq_n, 1)
    bwd_k = dkdv_k + dq_k  # the backward is the pair of kernels; its 10*Hq*D*P FLOP are counted once
    fwd_tf = flop_fwd / (fwd_k * 1e-3) / 1e12
    bwd_tf = flop_bwd / (bwd_k * 1e-3) / 1e12
    log(f"step {ms_per_step:.3f} ms  -> {tflops:.1f} TFLOP/s fwd+bwd ({100 * tflops / PEAK_BF16_TFLOPS:.1f}% of bf16 MFMA peak)")
    log(f"  ca_fwd_kernel {fwd_k:.3f} ms -> {fwd_tf:.1f} TFLOP/s ({100 * fwd_tf / PEAK_BF16_TFLOPS:.1f}%)")
    log(f"  ca_bwd kernels {bwd_k:.3f} ms (dkdv {dkdv_k:.3f} + dq {dq_k:.3f}) -> {bwd_tf:.1f} TFLOP/s ({100 * bwd_tf / PEAK_BF16_TFLOPS:.1f}%)")

    # what this device delivers for the MFMA instruction itself, right after the attention steps (the part is warm):
    # a loop of MFMAs on every SIMD, alone and with other work in every MFMA's shadow
    probe = None
    if not args.no_probe:
        executed = 1e-12 * (flop_fwd + 1.4 * flop_bwd) / ((fwd_k + bwd_k) * 1e-3)  # S and dP are computed in both backward kernels
        probe = mfma_probe(torch, _lib, dev, executed)
        log(f"  MFMA-only loop {probe['mfma_only']['TFLOP/s']} TFLOP/s (median of {probe['rounds']} rounds, {probe['mfma_only']['TFLOP/s_min']}"
            f"..{probe['mfma_only']['TFLOP/s_max']}) at {probe['mfma_only']['clock_GHz']} GHz; the attention kernels execute "
            f"{probe['executed_TFLOP/s_of_the_three_attention_kernels']} TFLOP/s = {100 * probe['executed_over_mfma_only']:.1f} % of it, "
            f"{100 * probe['executed_over_mfma_with_attention_side_work']:.1f} % of the loop with the backward's per-MFMA side work "
            f"({probe['with_attention_side_work']['TFLOP/s']} TFLOP/s at {probe['with_attention_side_work']['clock_GHz']} GHz, "
            f"{probe['with_attention_side_work']['cycles_per_mfma']} cycles per MFMA)")

    pack = None
    if not args.no_pack:
        del dq, dk, dv
        pack = pack_unpack_bench(torch, dev)
        for key in ("pack", "unpack", "memcpy_cp_pack", "memcpy_cp_unpack", "grad_sum"):
            log(f"  {key:17s} {pack[key]['GB/s']} GB/s ({100 * pack[key]['frac_hbm_peak']:.1f}% of HBM peak)")
        for key in ("pack", "unpack"):
            sep = pack[key]["as_separate_launches"]
            log(f"  {key:17s} as three launches {sep['GB/s']} GB/s ({100 * sep['frac_hbm_peak']:.1f}%)")

    tick = None
    if not args.no_tick:
        tick = server_tick_bench(torch, dev, batch, q, k, v, do, in_place_only=args.tick_in_place_only)
        log(f"  server tick over {tick['tasks']} tasks: forward {tick['forward_ms']} ms (kernel {tick['forward_attention_kernel_ms']}; "
            f"K/V unpacked first: {tick.get('forward_kv_unpacked_ms')}, kernel {tick.get('forward_kv_unpacked_attention_kernel_ms')}), "
            f"backward {tick['backward_ms']} ms (kernels {tick['backward_attention_kernels_ms']}; K/V unpacked first: "
            f"{tick.get('backward_kv_unpacked_ms')}, kernels {tick.get('backward_kv_unpacked_attention_kernels_ms')})")

    extra = None
    if not args.no_extra:
        del q, k, v, do
        torch.cuda.empty_cache()
        extra = other_workloads_bench(torch, dev)

    cpu = None
    if args.cpu_seconds > 0:
        cpu = cpu_baseline(batch, args.cpu_seconds, 77)
        log(f"  cpu baseline {cpu['value']} TFLOP/s on {cpu['cores']} threads: {cpu['sample']}")

    line = {
        "metric": "causal-attn TFLOP/s fwd+bwd, Llama-3-8B heads, 128K varlen; % MFMA peak",
        "value": round(tflops, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"{batch.name}: {len(batch.q_lens)} whole documents, lognormal(8,1.5) lengths in [128,65536], "
                               f"{tq} packed tokens, 32q/8kv heads, d=128, causal, fwd+bwd",
                   "causal_pairs": batch.causal_pairs, "flop_fwd": flop_fwd, "flop_bwd": flop_bwd,
                   "pct_of_bf16_mfma_peak": round(100 * tflops / PEAK_BF16_TFLOPS, 2)},
        "roofline": {"bound": "mfma", "kernel": "ca_bwd_dkdv64_kernel + ca_bwd_dq64_kernel", "achieved": round(bwd_tf, 2), "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(bwd_tf / PEAK_BF16_TFLOPS, 4),
                     "traffic": (MEASURED_TRAFFIC_BYTES["ca_bwd_dkdv64_kernel"] + MEASURED_TRAFFIC_BYTES["ca_bwd_dq64_kernel"]) if default_workload else None,
                     "traffic_unit": "bytes per launch (both kernels)",
                     "avg_launch_ms": round(bwd_k, 4), "avg_launch_ms_parts": {"ca_bwd_dkdv64_kernel": round(dkdv_k, 4), "ca_bwd_dq64_kernel": round(dq_k, 4)},
                     "executed_tflops": {"ca_bwd_dkdv64_kernel": round(0.8 * flop_bwd / dkdv_k / 1e9, 1), "ca_bwd_dq64_kernel": round(0.6 * flop_bwd / dq_k / 1e9, 1)},
                     "launches": bwd_n,
                     "mfma_probe": probe,
                     "also": {"ca_fwd_kernel": {"achieved": round(fwd_tf, 2), "frac": round(fwd_tf / PEAK_BF16_TFLOPS, 4),
                                                "avg_launch_ms": round(fwd_k, 4), "launches": fwd_n}}},
        "cpu_baseline": cpu,
        "pack_unpack": pack,
        "server_tick": tick,
        "extra": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
