"""Synthetic CA-task batches and shard layouts of the benchmark configurations.

Only lengths and offsets are produced here (numpy, seeded); tensors are drawn by the
caller on the device it runs on.  A task batch follows the reference's attention layout:
task = one query shard plus the KV prefix of its document up to the shard's end
(distca/runtime/compute_metadata.py:404-448), cu_seqlens as in get_attn_metadata (:326-365).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np


@dataclass
class TaskBatch:
    name: str
    q_lens: np.ndarray                 # [B] query rows per task
    k_lens: np.ndarray                 # [B] KV-prefix rows per task
    num_heads_q: int
    num_heads_kv: int
    head_dim: int = 128
    kv_task_offsets: Optional[np.ndarray] = None  # [B] first KV row of each task when prefixes are shared
    total_k: Optional[int] = None      # rows of the K/V tensors (defaults to sum(k_lens))
    notes: str = ""

    @property
    def cu_seqlens_q(self) -> np.ndarray:
        return np.concatenate([[0], np.cumsum(self.q_lens)]).astype(np.int32)

    @property
    def cu_seqlens_k(self) -> np.ndarray:
        return np.concatenate([[0], np.cumsum(self.k_lens)]).astype(np.int32)

    @property
    def total_q(self) -> int:
        return int(self.q_lens.sum())

    @property
    def kv_rows(self) -> int:
        return int(self.total_k if self.total_k is not None else self.k_lens.sum())

    @property
    def causal_pairs(self) -> int:
        lq = self.q_lens.astype(np.int64)
        lk = self.k_lens.astype(np.int64)
        return int((lq * lk - lq * (lq - 1) // 2).sum())

    def flops(self):
        """(fwd, bwd) algorithmic FLOPs: 4 and 10 x Hq x D x causal pairs."""
        base = self.num_heads_q * self.head_dim * self.causal_pairs
        return 4 * base, 10 * base


def _lognormal_docs(rng: np.random.Generator, total: int, lo: int, hi: int, mu: float = 8.0, sigma: float = 1.5) -> List[int]:
    lens: List[int] = []
    s = 0
    while s < total:
        n = int(np.clip(round(float(np.exp(rng.normal(mu, sigma)))), lo, hi))
        n = min(n, total - s)
        lens.append(n)
        s += n
    # a trailing remainder shorter than the minimum joins the previous document
    if len(lens) > 1 and lens[-1] < lo:
        last = lens.pop()
        lens[-1] += last
    return lens


def config1_tiny() -> TaskBatch:
    """3 packed docs [512, 1024, 2560], Llama-3-8B heads, forward only."""
    l = np.array([512, 1024, 2560], dtype=np.int64)
    return TaskBatch("cfg1_tiny_3docs_4096", l, l.copy(), 32, 8)


def config2_llama8b_128k(seed: int = 5002, total: int = 131072) -> TaskBatch:
    """Whole documents, lengths lognormal(8, 1.5) clipped to [128, 65536], summing to `total`."""
    rng = np.random.default_rng(seed)
    l = np.array(_lognormal_docs(rng, total, 128, 65536), dtype=np.int64)
    return TaskBatch(f"cfg2_llama8b_{total}", l, l.copy(), 32, 8)


def config3_ca_tasks(seed: int = 5003, variant: str = "b", total_q: int = 262144, num_docs: int = 8,
                     max_doc: int = 524288, chunk_lo: int = 4096, chunk_hi: int = 32768) -> TaskBatch:
    """Disaggregated shards: query chunks cut from `num_docs` documents, each attending to its
    document's KV prefix (kv_len = chunk end).  KV is stored once per document and shared by
    the tasks through kv_task_offsets.
      variant "a": total_q/4096 tasks of 4096 rows, chunk starts on multiples of 4096;
      variant "b": chunk lengths uniform in [chunk_lo, chunk_hi] until total_q rows."""
    rng = np.random.default_rng(seed)
    doc_lens = (rng.integers(max_doc // 8 // 4096, max_doc // 4096 + 1, size=num_docs) * 4096).astype(np.int64)
    doc_lens[0] = max_doc
    doc_starts = np.concatenate([[0], np.cumsum(doc_lens)[:-1]])
    q_lens, k_lens, offs = [], [], []
    if variant == "a":
        n = total_q // 4096
        for i in range(n):
            d = i % num_docs
            start = int(rng.integers(0, doc_lens[d] // 4096)) * 4096
            q_lens.append(4096); k_lens.append(start + 4096); offs.append(int(doc_starts[d]))
    else:
        s, i = 0, 0
        while s < total_q:
            ln = int(rng.integers(chunk_lo, chunk_hi + 1))
            ln = min(ln, total_q - s)
            d = i % num_docs
            start = int(rng.integers(0, (doc_lens[d] - ln) // 128 + 1)) * 128
            q_lens.append(ln); k_lens.append(start + ln); offs.append(int(doc_starts[d]))
            s += ln; i += 1
    return TaskBatch(f"cfg3{variant}_ca_tasks_{total_q}", np.array(q_lens, np.int64), np.array(k_lens, np.int64), 32, 8,
                     kv_task_offsets=np.array(offs, np.int32), total_k=int(doc_lens.sum()),
                     notes=f"{len(q_lens)} tasks over {num_docs} docs, doc_lens={doc_lens.tolist()}")


def config5_llama70b_skewed(seed: int = 5005, total: int = 524288, big: int = 262144) -> TaskBatch:
    """One `big`-token document plus lognormal documents in [256, 32768], Llama-3-70B heads."""
    rng = np.random.default_rng(seed)
    l = np.array([big] + _lognormal_docs(rng, total - big, 256, 32768), dtype=np.int64)
    return TaskBatch(f"cfg5_llama70b_{total}", l, l.copy(), 64, 8)


@dataclass
class ShardLayout:
    """fa2a pack/unpack case: shards of a [T, hidden] tensor and their byte offsets in a buffer."""
    name: str
    seq_tokens: np.ndarray   # int64 [S]
    offsets: dict = field(default_factory=dict)  # tensor name -> int64 [S] byte offsets
    token_bytes: dict = field(default_factory=dict)
    buffer_bytes: int = 0

    @property
    def num_tokens(self) -> int:
        return int(self.seq_tokens.sum())


def config4_pack(seed: int = 5004, total: int = 262144, lo: int = 128, hi: int = 16384,
                 token_bytes=None) -> ShardLayout:
    """Shard lengths uniform in [lo, hi] until `total` tokens; a seeded permutation of the shards
    defines their order in the buffer, q region first, then k, then v."""
    token_bytes = token_bytes or {"q": 32 * 128 * 2, "k": 8 * 128 * 2, "v": 8 * 128 * 2}
    rng = np.random.default_rng(seed)
    lens: List[int] = []
    s = 0
    while s < total:
        n = min(int(rng.integers(lo, hi + 1)), total - s)
        lens.append(n); s += n
    lens_a = np.array(lens, dtype=np.int64)
    perm = rng.permutation(len(lens))
    lay = ShardLayout(f"cfg4_pack_{total}", lens_a, token_bytes=dict(token_bytes))
    base = 0
    for name, tb in token_bytes.items():
        off = np.zeros(len(lens), dtype=np.int64)
        cur = base
        for s_id in perm:
            off[s_id] = cur
            cur += int(lens_a[s_id]) * tb
        lay.offsets[name] = off
        base = cur
    lay.buffer_bytes = base
    return lay
