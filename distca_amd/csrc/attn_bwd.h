// Arguments shared by the kernels of the attention backward (attn_bwd.hip, attn_bwd_dkdv64.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/distca_ca.h"
#include "common.h"
#include "kv_shards.h"

namespace distca {

struct BwdArgs {
  const elem_t *q, *k, *v, *dout;
  const float *lse2, *dscaled;  // [Hq][Tq]: lse*log2e and -delta, written by the dQ kernel, read by the dK/dV kernel
  // what the dQ kernel makes them from: O laid out like q and dout, and the forward's lse either as [Hq][Tq] or as Hq
  // floats per token in the query-side region (first byte of that part in token 0), one of the two null
  const elem_t *out;
  const float *lse;
  const uint8_t *lse_tok;
  float *lse2_w, *dscaled_w;
  elem_t *dq, *dk, *dv;
  float *dk_acc, *dv_acc;  // used instead of dk/dv when tasks may alias KV rows
  const int32_t *cu_q, *cu_k, *kv_off;
  // the dK/dV list over groups of tasks that share stored K/V rows (sched.h, SharedGroups); null otherwise
  const int32_t *grp_first, *grp_tasks, *grp_off, *grp_lmax;
  KvShards shards;  // kernels that read K/V in place: k, v, dk, dv are then the bases the shards' offsets count from
  const int32_t *sched;
  int32_t *tickets;  // one counter per kv head (sched.h)
  const void *zero_row;  // 256 zero bytes: source of tile rows past the end of a task
  int32_t sched_items_off;
  int32_t merge_tiles;  // dQ kernel: merge_tiles of its list (sched.h, fwd_merge), 0 = one block per item
  int32_t hq, hkv, group, total_q;
  uint32_t group_magic;  // ceil(2^32 / group), 0 when group == 1: n / group == umulhi(n, magic) for n * group < 2^32
  int32_t causal;
  float scale;
  // Where the query-side tokens live: q and dout point at the first byte of their part of token 0 of a
  // region in which token t of task b starts at off[b] + t * tok_bytes (off == nullptr: the packed
  // tensors, off[b] = cu_q[b] * tok_bytes); head h at + h * 256 bytes.  dq likewise.
  const int64_t *qs_task_off, *dq_task_off;
  int64_t qs_tok_bytes, dq_tok_bytes;
};


// The query side of a backward call: where dO, O, lse, q are read and dq is written.
struct BwdQuerySide {
  const void *dout, *q, *out;      // first byte of each part in token 0 of its region
  const float *lse;                // [Hq][Tq], or nullptr with lse_tok
  const void *lse_tok;             // first byte of the lse part in token 0, or nullptr
  const int64_t *task_off;         // shared by dout, q, out, lse_tok; nullptr = packed tensors
  int64_t tok_bytes;
  void *dq;
  const int64_t *dq_task_off;
  int64_t dq_tok_bytes;
};
// The backward behind distca_ca_bwd and distca_ca_bwd_tokens, per element type (attn_bwd.hip compiled for each).
// kv_shards: null, or the table through which K/V rows are read and dK/dV rows written in place (kv_shards.h)
int run_bwd(const BwdQuerySide &qs, const void *k, const void *v, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k,
            const int32_t *kv_off, const distca_kv_shards *kv_shards, const distca_ca_params *p, void *workspace,
            int64_t workspace_bytes, void *stream);
int run_bwd_f16(const BwdQuerySide &qs, const void *k, const void *v, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k,
                const int32_t *kv_off, const distca_kv_shards *kv_shards, const distca_ca_params *p, void *workspace,
                int64_t workspace_bytes, void *stream);
// The forward behind distca_ca_fwd_tokens, per element type (attn_fwd.hip compiled for each).
int run_fwd_tokens(const void *q_base, const int64_t *q_task_off, int64_t q_tok_bytes, const void *k, const void *v,
                   const distca_kv_shards *kv_shards, void *out_base, const int64_t *out_task_off, int64_t out_tok_bytes, float *lse,
                   const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off, const distca_ca_params *p, void *workspace,
                   int64_t workspace_bytes, void *stream);
int run_fwd_tokens_f16(const void *q_base, const int64_t *q_task_off, int64_t q_tok_bytes, const void *k, const void *v,
                       const distca_kv_shards *kv_shards, void *out_base, const int64_t *out_task_off, int64_t out_tok_bytes, float *lse,
                       const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off, const distca_ca_params *p, void *workspace,
                       int64_t workspace_bytes, void *stream);
// Checks a table of shards (host-visible fields only) and turns it into the kernels' form.
int make_kv_shards(const distca_kv_shards *in, const int32_t *kv_off, bool backward, KvShards *out);

// The dK/dV kernel with 64 keys per wave (attn_bwd_dkdv64.hip): LDS bytes it needs, and its launch.
int dkdv64_lds_bytes();
// atomic_sums: items add to the fp32 accumulators (pieces of key blocks); shared: items are (group of tasks, key block)
int launch_dkdv64(const BwdArgs &a, int64_t grid, bool atomic_sums, bool shared, hipStream_t stream);       // bf16 elements
int launch_dkdv64_f16(const BwdArgs &a, int64_t grid, bool atomic_sums, bool shared, hipStream_t stream);   // fp16 elements
// The dQ kernel with 64 query rows per wave (attn_bwd_dq64.hip).
int launch_dq64(const BwdArgs &a, int64_t grid, hipStream_t stream);
int launch_dq64_f16(const BwdArgs &a, int64_t grid, hipStream_t stream);

}  // namespace distca
