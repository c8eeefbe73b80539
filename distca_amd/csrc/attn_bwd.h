// Arguments shared by the kernels of the attention backward (attn_bwd.hip, attn_bwd_dkdv64.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace distca {

struct BwdArgs {
  const __bf16 *q, *k, *v, *dout;
  const float *lse2, *dscaled;  // [Hq][Tq]: lse*log2e and -delta
  __bf16 *dq, *dk, *dv;
  float *dk_acc, *dv_acc;  // used instead of dk/dv when tasks may alias KV rows
  const int32_t *cu_q, *cu_k, *kv_off;
  const int32_t *sched;
  int32_t *tickets;  // one counter per kv head (sched.h)
  const void *zero_row;  // 256 zero bytes: source of tile rows past the end of a task
  int32_t sched_items_off;
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


// The dK/dV kernel with 64 keys per wave (attn_bwd_dkdv64.hip): LDS bytes it needs, and its launch.
int dkdv64_lds_bytes();
int launch_dkdv64(const BwdArgs &a, int64_t grid, bool alias, hipStream_t stream);

}  // namespace distca
