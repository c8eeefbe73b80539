"""Writes the committed fixtures of this folder from the CPU oracle (run from the repo root:
`python tests/golden/make_fixtures.py`).  The reference ships no golden vectors for this
path (its tests compare kernels with torch simulators on fresh random tensors), so these
freeze the oracle's own answers, evaluated in float64, on inputs stored bit for bit: a later
change to the oracle or to a kernel that moves a result shows up against the same numbers.

  attention_small.npz   3 tasks (whole document, KV-prefix task, 1-token task), 4q/2kv heads,
                        d=128: bf16 inputs as uint16 bit patterns; out, lse, dq, dk, dv as float32
  fa2a_small.npz        pack / replicating pack / duplicate-gradient sum on a 7-shard layout
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

from oracle import fa2a  # noqa: E402
from oracle.attention import ca_reference_bwd, ca_reference_fwd  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bits(x: torch.Tensor) -> np.ndarray:
    return x.view(torch.int16).numpy().view(np.uint16)


def attention_small():
    q_lens, k_lens = [40, 23, 1], [40, 87, 1]
    g = torch.Generator().manual_seed(20240517)
    rnd = lambda *s: torch.randn(s, generator=g).to(torch.bfloat16)
    q, k, v, do = rnd(64, 4, 128), rnd(128, 2, 128), rnd(128, 2, 128), rnd(64, 4, 128)
    cu_q = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    cu_k = np.concatenate([[0], np.cumsum(k_lens)]).astype(np.int32)
    out, lse = ca_reference_fwd(q, k, v, cu_q, cu_k, dtype=torch.float64)
    dq, dk, dv = ca_reference_bwd(do, q, k, v, cu_q, cu_k, dtype=torch.float64)
    f32 = lambda x: x.to(torch.float32).numpy()
    np.savez_compressed(os.path.join(HERE, "attention_small.npz"), q=bits(q), k=bits(k), v=bits(v), dout=bits(do),
                        cu_seqlens_q=cu_q, cu_seqlens_k=cu_k, out=f32(out), lse=f32(lse), dq=f32(dq), dk=f32(dk), dv=f32(dv))


def fa2a_small():
    rng = np.random.default_rng(77)
    lens = np.array([3, 0, 5, 1, 4, 2, 6], np.int64)
    tb = 32
    t = rng.integers(0, 256, size=(int(lens.sum()), tb), dtype=np.uint8)
    perm = rng.permutation(len(lens))
    off = np.zeros(len(lens), np.int64); cur = 0
    for s in perm:
        off[s] = cur; cur += int(lens[s]) * tb + 16
    mask = np.array([1, 1, 0, 1, 0, 1, 1], np.int8)
    packed = np.full(cur, 0xEE, np.uint8); fa2a.copy_non_cp(t, packed, off, lens, None, True)
    packed_masked = np.full(cur, 0xEE, np.uint8); fa2a.copy_non_cp(t, packed_masked, off, lens, mask, True)
    max_cp = 3
    do_shard = (rng.random((len(lens), max_cp)) < 0.6).astype(np.int8)
    off_cp = np.zeros((max_cp, len(lens)), np.int64); cur_cp = 0
    for c in range(max_cp):
        for s in rng.permutation(len(lens)):
            off_cp[c, s] = cur_cp; cur_cp += int(lens[s]) * tb
    packed_cp = np.full(cur_cp, 0xEE, np.uint8); fa2a.copy_cp(t, packed_cp, do_shard, off_cp, lens, True)
    planes = np.zeros((max_cp, t.shape[0], tb), np.uint8); fa2a.copy_cp(planes, packed_cp, do_shard, off_cp, lens, False)
    # duplicate-gradient sum: shards 0 and 4 own copies elsewhere (equal lengths by construction)
    glens = np.array([3, 5, 3, 3, 5], np.int64)
    gt = torch.Generator().manual_seed(5)
    grad = (torch.randn((int(glens.sum()), 16), generator=gt) * 50).to(torch.bfloat16)
    num_copies = np.array([2, 1, 0, 0, 0], np.int32)
    copy_start = np.array([[8, 11], [14, 0], [0, 0], [0, 0], [0, 0]], np.int64)
    summed = grad.clone(); fa2a.grad_sum(summed, num_copies, copy_start, glens)
    np.savez_compressed(os.path.join(HERE, "fa2a_small.npz"), tensor=t, seq_tokens=lens, offsets=off, mask=mask,
                        packed=packed, packed_masked=packed_masked, do_shard=do_shard, offsets_cp=off_cp,
                        packed_cp=packed_cp, planes=planes, grad=bits(grad), grad_lens=glens, num_copies=num_copies,
                        copy_start=copy_start, grad_summed=bits(summed))


if __name__ == "__main__":
    attention_small()
    fa2a_small()
    for f in sorted(os.listdir(HERE)):
        print(f, os.path.getsize(os.path.join(HERE, f)))
