// K/V rows read where they lie in a transport buffer.
//
// The CA server receives every stored K/V shard once, somewhere in its receive buffer (the reference unpacks the
// shards into contiguous tensors first, distca/runtime/attn_kernels/dispatch.py:60-94, and packs dK/dV back,
// :39-56).  Here the attention kernels address a stored row through a table of shards instead: stored rows
// [row_start[s], row_start[s + 1]) are the rows of shard s, which lie token after token (Hkv * D elements each) from
// byte k_off[s] of the K base pointer (v_off[s] of the V base).  A tile request whose rows lie in one shard is made
// from a scalar base as before; one that straddles shards, or the end of a task's prefix, computes per-lane addresses.
#pragma once
#include <stdint.h>

#include "common.h"

namespace distca {

struct KvShards {
  const int32_t *row_start;     // [num_shards + 1], ascending; row_start[num_shards] = stored rows in all
  const int64_t *k_off, *v_off;  // [num_shards] byte offsets of the shards' K and V rows
  const int64_t *dk_off, *dv_off;  // backward: where the shards' dK and dV rows go
  const int32_t *task_shard;    // [num_tasks] the shard that holds the first row of each task's prefix
  int32_t num_shards;           // 0: the rows are one dense tensor (none of the above is read)
};

// Largest s in [0, n) with row_start[s] <= r.
__device__ __forceinline__ int find_shard(const int32_t *row_start, int n, int r) {
  int lo = 0, hi = n;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (row_start[mid] <= r) lo = mid; else hi = mid;
  }
  return lo;
}

// The shard that holds the rows a wave is about to request, carried along a walk over ascending rows (all of it
// wave-uniform: scalar registers and scalar loads).
// The values are forced into scalar registers as they are loaded (the loads are vector loads from a uniform address): the
// comparisons and address arithmetic of every later request then run on the scalar unit and occupy no vector register.
__device__ __forceinline__ int uniform_i32(int x) { return (int)uniform32((uint32_t)x); }
__device__ __forceinline__ int64_t uniform_i64(int64_t x) {
  // (the builtin behind uniform32 returns a signed int: each half is taken as unsigned before it is widened, or a low
  // half with its top bit set would fill the high half with ones)
  const uint64_t u = (uint64_t)x;
  const uint64_t hi = uniform32((uint32_t)(u >> 32)), lo = uniform32((uint32_t)u);
  return (int64_t)((hi << 32) | lo);
}
struct ShardCursor {
  int idx, lo, hi;
  int64_t k, v;  // byte offsets of the shard's first row
  __device__ __forceinline__ void open(const KvShards &s, int shard) {
    idx = uniform_i32(shard);
    lo = uniform_i32(s.row_start[idx]);
    hi = uniform_i32(s.row_start[idx + 1]);
    k = uniform_i64(s.k_off[idx]);
    v = uniform_i64(s.v_off[idx]);
  }
  // moves on to the shard that holds row r (r not below the present shard's first row)
  __device__ __forceinline__ void seek(const KvShards &s, int r) {
    while (r >= hi && idx + 1 < s.num_shards) {
      ++idx;
      lo = hi;
      hi = uniform_i32(s.row_start[idx + 1]);
      k = uniform_i64(s.k_off[idx]);
      v = uniform_i64(s.v_off[idx]);
    }
  }
  __device__ __forceinline__ bool holds(int r0, int n) const { return r0 >= lo && r0 + n <= hi; }
};

// Byte offset of stored row r (per lane) given that the cursor's shard starts at or before it: rows of later shards
// are found by walking on from the cursor.  `which`: 0 = K, 1 = V.
__device__ __forceinline__ int64_t shard_row_offset(const KvShards &s, const ShardCursor &c, int r, int which, int64_t row_bytes) {
  if (r < c.hi) return (which ? c.v : c.k) + (int64_t)(r - c.lo) * row_bytes;
  int i = c.idx + 1;
  while (i + 1 < s.num_shards && r >= s.row_start[i + 1]) ++i;
  return (which ? s.v_off[i] : s.k_off[i]) + (int64_t)(r - s.row_start[i]) * row_bytes;
}

}  // namespace distca
