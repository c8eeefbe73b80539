// Varlen causal flash-attention backward (dQ, dK, dV) for gfx950.
//
// Stands where the reference calls flash-attn's varlen backward
// (distca/runtime/megatron/ops/fused_comm_attn.py:259-272).
//
// The backward runs as two kernels that both recompute P from (Q, K, LSE), so that neither
// needs floating-point atomics and the result is bit-reproducible (the `deterministic` switch
// of the reference's FlashAttnArgs holds by construction).  A single-kernel form that added
// dQ partial sums with fp32 atomics was measured first: the atomics alone (a 16 KB patch per
// 32 rows x 256 keys, 62 GB at 131 072 tokens, at the 1.3 TB/s the device adds floats at) took
// longer than the two kernels together.
//
//   1. ca_bwd_dq64_kernel (attn_bwd_dq64.hip): dQ, one workgroup of 4 waves per (task, block of 256 flattened
//      query rows, kv head), in the order of the forward tile schedule.  Its prologue, which reads a row's dO
//      anyway, also makes the row statistics both kernels need (delta = <dO, O>, lse * log2(e)) and leaves them in
//      the workspace.
//   2. ca_bwd_dkdv64_kernel (attn_bwd_dkdv64.hip): dK and dV, one workgroup of 4 waves per (task, block of
//      256 keys, kv head), in the order of the backward tile schedule.
#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

#include "api_util.h"
#include "attn_bwd.h"
#include "attn_cfg.h"
#include "common.h"

#include <type_traits>

namespace distca {
namespace {

// Zeroes the dk / dv rows that no workgroup of the dK/dV kernel writes when every task owns its K/V rows: the
// rows of tasks without queries (they get no work item) and the rows past the last task.  Workgroup (b, y):
// part y of task b's rows, b == num_tasks standing for the tail.
__global__ __launch_bounds__(256) void fill_unowned_rows_kernel(u32x4 *__restrict__ dk, u32x4 *__restrict__ dv,
                                                               const int32_t *__restrict__ cu_q, const int32_t *__restrict__ cu_k,
                                                               int32_t num_tasks, int32_t total_k, int64_t row_vecs) {
  const int b = blockIdx.x;
  int64_t r0, r1;
  if (b < num_tasks) {
    if (cu_q[b + 1] > cu_q[b]) return;
    r0 = cu_k[b];
    r1 = cu_k[b + 1];
  } else {
    r0 = cu_k[num_tasks];
    r1 = total_k;
  }
  if (r0 < 0) r0 = 0;
  if (r1 > total_k) r1 = total_k;
  const int64_t v0 = r0 * row_vecs, v1 = r1 * row_vecs;
  for (int64_t i = v0 + (int64_t)blockIdx.y * 256 + threadIdx.x; i < v1; i += (int64_t)gridDim.y * 256) {
    dk[i] = u32x4{0, 0, 0, 0};
    dv[i] = u32x4{0, 0, 0, 0};
  }
}

// The same for tasks over shared stored rows: zeroes the stored rows no group of tasks covers (sched.h, SharedGroups:
// gap u, u <= num_tasks; those past the number of groups are empty).  Workgroup (u, y): part y of gap u.
__global__ __launch_bounds__(256) void fill_gap_rows_kernel(u32x4 *__restrict__ dk, u32x4 *__restrict__ dv,
                                                           const int32_t *__restrict__ gap_lo, const int32_t *__restrict__ gap_hi,
                                                           int32_t total_k, int64_t row_vecs) {
  int64_t r0 = gap_lo[blockIdx.x], r1 = gap_hi[blockIdx.x];
  if (r0 < 0) r0 = 0;
  if (r1 > total_k) r1 = total_k;
  const int64_t v0 = r0 * row_vecs, v1 = r1 * row_vecs;
  for (int64_t i = v0 + (int64_t)blockIdx.y * 256 + threadIdx.x; i < v1; i += (int64_t)gridDim.y * 256) {
    dk[i] = u32x4{0, 0, 0, 0};
    dv[i] = u32x4{0, 0, 0, 0};
  }
}

// The same with the dK/dV rows addressed through a table of shards (kv_shards.h): one row per 128-thread slice.
__global__ __launch_bounds__(256) void fill_gap_rows_shards_kernel(uint8_t *__restrict__ dk, uint8_t *__restrict__ dv,
                                                                  const int32_t *__restrict__ gap_lo, const int32_t *__restrict__ gap_hi,
                                                                  int32_t total_k, int64_t row_bytes, KvShards sh) {
  int64_t r0 = gap_lo[blockIdx.x], r1 = gap_hi[blockIdx.x];
  if (r0 < 0) r0 = 0;
  if (r1 > total_k) r1 = total_k;
  for (int64_t r = r0 + blockIdx.y; r < r1; r += gridDim.y) {
    const int s = find_shard(sh.row_start, sh.num_shards, (int)r);
    const int64_t in_shard = (r - sh.row_start[s]) * row_bytes;
    u32x4 *pk = reinterpret_cast<u32x4 *>(dk + sh.dk_off[s] + in_shard), *pv = reinterpret_cast<u32x4 *>(dv + sh.dv_off[s] + in_shard);
    for (int64_t i = threadIdx.x; i < row_bytes / 16; i += 256) {
      pk[i] = u32x4{0, 0, 0, 0};
      pv[i] = u32x4{0, 0, 0, 0};
    }
  }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(u32x4 *__restrict__ p, int64_t nvec) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < nvec; i += stride) p[i] = u32x4{0, 0, 0, 0};
}

// fp32 accumulator -> bf16, 8 elements per thread
__global__ __launch_bounds__(256) void cvt_elem_kernel(const float *__restrict__ src, elem_t *__restrict__ dst, int64_t n8) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n8; i += stride) {
    const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + 2 * i);
    const f32x4 y = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + 2 * i + 1);
    reinterpret_cast<elemx8 *>(dst)[i] = cvt8(x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]);
  }
}

struct BwdWorkspace {
  int64_t sched_kv, sched_q, delta, lse2, dk_acc, dv_acc, total;
};
// acc: with the fp32 dK/dV accumulators (needed only when key blocks are cut into pieces); max_items_kv: room of the dK/dV list
BwdWorkspace bwd_layout(const distca_ca_params *p, bool alias, int64_t max_items_kv) {
  BwdWorkspace w;
  int64_t o = 0;
  w.sched_kv = o; o += sched_shared_region_bytes(p->num_tasks, max_items_kv);
  w.sched_q = o; o += sched_region_bytes(p->num_tasks, dq_max_items(p));
  w.delta = o; o += align_up((int64_t)p->num_heads_q * p->total_q * 4, 256);
  w.lse2 = o; o += align_up((int64_t)p->num_heads_q * p->total_q * 4, 256);
  w.dk_acc = o; if (alias) o += align_up((int64_t)p->total_k * p->num_heads_kv * kHeadDim * 4, 256);
  w.dv_acc = o; if (alias) o += align_up((int64_t)p->total_k * p->num_heads_kv * kHeadDim * 4, 256);
  w.total = o;
  return w;
}

int grid_for(int64_t work_items) {
  int64_t g = (work_items + 255) / 256;
  const int64_t cap = (int64_t)num_compute_units() * 16;
  if (g > cap) g = cap;
  return g < 1 ? 1 : (int)g;
}

}  // namespace
}  // namespace distca

using namespace distca;

#ifndef DISTCA_F16
extern "C" int64_t distca_ca_bwd_workspace_bytes(const distca_ca_params *p) {
  if (!p) return fail(DISTCA_E_INVALID, "bwd_workspace_bytes: null params");
  int rc = validate_params(p);
  if (rc) return rc;
  // the work lists and row statistics, and, only when key blocks are cut into pieces (small batches whose caller
  // allows float atomics), the fp32 dK/dV accumulators
  return bwd_layout(p, bwd_split_target(p) > 0, bwd_max_items(p)).total;
}

extern "C" int distca_ca_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out, const float *lse,
                             void *dq, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off,
                             const distca_ca_params *p, void *workspace, int64_t workspace_bytes, void *stream) {
  if (!p) return fail(DISTCA_E_INVALID, "ca_bwd: null params");
  const int64_t row_bytes = (int64_t)p->num_heads_q * kHeadDim * 2;
  const BwdQuerySide qs{dout, q, out, lse, nullptr, nullptr, row_bytes, dq, nullptr, row_bytes};
  return (p->dtype == DISTCA_DTYPE_F16 ? run_bwd_f16 : run_bwd)(qs, k, v, dk, dv, cu_q, cu_k, kv_off, nullptr, p, workspace, workspace_bytes, stream);
}

extern "C" int distca_ca_bwd_tokens(const void *req_base, const int64_t *req_task_off, int64_t req_tok_bytes, const void *k,
                                    const void *v, void *dq_base, const int64_t *dq_task_off, int64_t dq_tok_bytes, void *dk,
                                    void *dv, const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off,
                                    const distca_ca_params *p, void *workspace, int64_t workspace_bytes, void *stream) {
  return distca_ca_bwd_buffers(req_base, req_task_off, req_tok_bytes, k, v, nullptr, dq_base, dq_task_off, dq_tok_bytes, dk, dv, cu_q,
                               cu_k, kv_off, p, workspace, workspace_bytes, stream);
}

// kv_shards may be null here (distca_ca_bwd_tokens comes through this function); the public contract of the name
// requires it, which the header says.
extern "C" int distca_ca_bwd_buffers(const void *req_base, const int64_t *req_task_off, int64_t req_tok_bytes, const void *k,
                                     const void *v, const distca_kv_shards *kv_shards, void *dq_base, const int64_t *dq_task_off,
                                     int64_t dq_tok_bytes, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k,
                                     const int32_t *kv_off, const distca_ca_params *p, void *workspace, int64_t workspace_bytes,
                                     void *stream) {
  if (!p) return fail(DISTCA_E_INVALID, "ca_bwd: null params");
  int rc = validate_params(p);
  if (rc) return rc;
  const int64_t row_bytes = (int64_t)p->num_heads_q * kHeadDim * 2, lse_bytes = (int64_t)p->num_heads_q * 4;
  if (lse_bytes & 15)
    return fail(DISTCA_E_UNSUPPORTED, "ca_bwd_tokens: %d query heads put the q part of a request token off 16-byte alignment", p->num_heads_q);
  // a server with no task this tick has empty offset arrays, which may come as null pointers; nothing reads them then
  if ((!req_task_off || !dq_task_off) && p->num_tasks > 0) return fail(DISTCA_E_INVALID, "ca_bwd_tokens: null offset array");
  if (req_tok_bytes < 3 * row_bytes + lse_bytes || (req_tok_bytes & 15))
    return fail(DISTCA_E_INVALID, "ca_bwd_tokens: request token of %lld B (needs >= %lld, multiple of 16)", (long long)req_tok_bytes, (long long)(3 * row_bytes + lse_bytes));
  if (dq_tok_bytes < row_bytes || (dq_tok_bytes & 15))
    return fail(DISTCA_E_INVALID, "ca_bwd_tokens: dq token of %lld B (needs >= %lld, multiple of 16)", (long long)dq_tok_bytes, (long long)row_bytes);
  const uint8_t *r = (const uint8_t *)req_base;
  // [dO | O | lse | q | pad]
  const BwdQuerySide qs{r, r ? r + 2 * row_bytes + lse_bytes : nullptr, r ? r + row_bytes : nullptr, nullptr,
                        r ? r + 2 * row_bytes : nullptr, req_task_off, req_tok_bytes, dq_base, dq_task_off, dq_tok_bytes};
  return (p->dtype == DISTCA_DTYPE_F16 ? run_bwd_f16 : run_bwd)(qs, k, v, dk, dv, cu_q, cu_k, kv_off, kv_shards, p, workspace, workspace_bytes, stream);
}
#endif  // !DISTCA_F16

namespace distca {
int DISTCA_FN(run_bwd)(const BwdQuerySide &qs, const void *k, const void *v, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k,
                       const int32_t *kv_off, const distca_kv_shards *kv_shards, const distca_ca_params *p, void *workspace,
                       int64_t workspace_bytes, void *stream) {
  const void *dout = qs.dout, *q = qs.q, *out = qs.out;
  void *dq = qs.dq;
  if (!p) return fail(DISTCA_E_INVALID, "ca_bwd: null params");
  int rc = validate_params(p);
  if (rc) return rc;
  const bool alias = kv_off != nullptr;
  if (!dout || !q || !k || !v || !out || (!qs.lse && !qs.lse_tok) || !dq || !dk || !dv || !cu_q || !cu_k) {
    if (p->num_tasks == 0 || (p->total_q == 0 && p->total_k == 0)) return DISTCA_OK;
    return fail(DISTCA_E_INVALID, "ca_bwd: null pointer");
  }
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv))
    return fail(DISTCA_E_INVALID, "ca_bwd: tensors must be 16-byte aligned");
  // dK/dV go through fp32 accumulators (float atomics) only when key blocks are cut into pieces.  Tasks over shared
  // K/V rows otherwise have one work item per (group of tasks, key block), which sums in registers like any other.
  // With K/V shards read in place nothing is cut (the accumulators are dense tensors over stored rows).
  KvShards shards{};
  if (kv_shards) {
    rc = make_kv_shards(kv_shards, kv_off, true, &shards);
    if (rc) return rc;
  }
  const int32_t split = kv_shards ? 0 : bwd_split_target(p);
  const bool use_acc = split > 0;
  const bool shared = alias && !use_acc;
  const int64_t max_items_kv = split > 0 ? bwd_key_blocks_bound(p) + split : bwd_key_blocks_own_rows(p);
  const BwdWorkspace w = bwd_layout(p, use_acc, max_items_kv);
  if (!workspace || workspace_bytes < w.total)
    return fail(DISTCA_E_WORKSPACE, "ca_bwd: workspace %lld B < required %lld B", (long long)workspace_bytes, (long long)w.total);
  if (!aligned16(workspace)) return fail(DISTCA_E_INVALID, "ca_bwd: workspace must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  uint8_t *ws = (uint8_t *)workspace;
  const int64_t kv_elems = (int64_t)p->total_k * p->num_heads_kv * kHeadDim;
  const int64_t q_elems = (int64_t)p->total_q * p->num_heads_q * kHeadDim;

  // rows no task touches must come back as zero
  if (kv_elems > 0) {
    if (use_acc) {
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 2)), dim3(256), 0, s, (u32x4 *)(ws + w.dk_acc),
                         (w.total - w.dk_acc) / 16);
    } else if ((p->num_tasks == 0 || p->total_q == 0) && kv_shards) {
      return fail(DISTCA_E_UNSUPPORTED, "ca_bwd_buffers: a batch without tasks or queries (there is nothing to tell which rows to clear)");
    } else if (p->num_tasks == 0 || p->total_q == 0) {
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (u32x4 *)dk, kv_elems / 8);
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (u32x4 *)dv, kv_elems / 8);
    } else if (!shared) {
      // every task owns its rows and the dK/dV kernel writes each row of a task that has queries exactly once:
      // only the others need the fill (at 131 072 tokens that is 0.5 GB of writes not made); with shared rows the
      // fill follows the list builder below, which finds the rows no group of tasks covers
      hipLaunchKernelGGL(fill_unowned_rows_kernel, dim3((unsigned)p->num_tasks + 1, 16), dim3(256), 0, s, (u32x4 *)dk, (u32x4 *)dv,
                         cu_q, cu_k, p->num_tasks, p->total_k, (int64_t)p->num_heads_kv * kHeadDim / 8);
    }
  }
  if (p->num_tasks == 0 || p->total_q == 0) return check_launch("ca_bwd(clear)");

  BwdArgs a;
  a.q = (const elem_t *)q; a.k = (const elem_t *)k; a.v = (const elem_t *)v; a.dout = (const elem_t *)dout;
  a.lse2 = (const float *)(ws + w.lse2); a.dscaled = (const float *)(ws + w.delta);
  a.lse2_w = (float *)(ws + w.lse2); a.dscaled_w = (float *)(ws + w.delta);
  a.out = (const elem_t *)out; a.lse = qs.lse; a.lse_tok = (const uint8_t *)qs.lse_tok;
  a.dq = (elem_t *)dq; a.dk = (elem_t *)dk; a.dv = (elem_t *)dv;
  a.qs_task_off = qs.task_off; a.qs_tok_bytes = qs.tok_bytes; a.dq_task_off = qs.dq_task_off; a.dq_tok_bytes = qs.dq_tok_bytes;
  a.dk_acc = use_acc ? (float *)(ws + w.dk_acc) : nullptr;
  a.dv_acc = use_acc ? (float *)(ws + w.dv_acc) : nullptr;
  a.cu_q = cu_q; a.cu_k = cu_k; a.kv_off = kv_off;
  a.grp_first = a.grp_tasks = a.grp_off = a.grp_lmax = nullptr;
  a.shards = shards;
  a.sched_items_off = (int32_t)sched_header_ints(p->num_tasks);
  a.hq = p->num_heads_q; a.hkv = p->num_heads_kv; a.group = p->num_heads_q / p->num_heads_kv;
  a.total_q = p->total_q; a.causal = p->causal != 0; a.scale = p->softmax_scale;
  a.group_magic = a.group == 1 ? 0u : (uint32_t)(((1ull << 32) + a.group - 1) / a.group);
  if ((uint64_t)p->max_seqlen_q * a.group * a.group >= (1ull << 32))
    return fail(DISTCA_E_UNSUPPORTED, "ca_bwd: max_seqlen_q * (Hq/Hkv)^2 must stay below 2^32");

  // ---- dQ: one workgroup per (task, block of query rows, kv head).  It runs first: it also leaves the row
  // statistics (lse in the log2 domain, -delta) in the workspace, which the dK/dV kernel reads.
  {
    const SchedGeom geom = dq_geom(p);
    a.merge_tiles = geom.merge_tiles;
    const int64_t max_items = dq_max_items(p);
    rc = launch_build_schedule(0, cu_q, cu_k, p->num_tasks, geom, (int32_t *)(ws + w.sched_q), max_items, s);
    if (rc) return rc;
    const int64_t grid = max_items * p->num_heads_kv * kSchedOversubNum / kSchedOversubDen;
    if (grid > 0x7fffffff) return fail(DISTCA_E_INVALID, "ca_bwd: grid too large");
    a.sched = (const int32_t *)(ws + w.sched_q);
    a.zero_row = ws + w.sched_q + sched_zero_row_off(p->num_tasks, max_items);
    a.tickets = (int32_t *)(ws + w.sched_q + sched_ticket_off(p->num_tasks, max_items));
    ScopedTimer timer(DISTCA_TIMER_CA_BWD_DQ, s);
    rc = DISTCA_FN(launch_dq64)(a, grid, s);
    if (rc) return rc;
  }
  // ---- dK, dV: one workgroup per (task, 256-key block, kv head)
  {
    const int64_t max_items = max_items_kv;
    int32_t *list = (int32_t *)(ws + w.sched_kv);
    if (shared) {
      rc = launch_build_shared_schedule(cu_q, cu_k, kv_off, p->num_tasks, p->total_k, bwd_shared_geom(p), list, max_items, s);
      if (rc) return rc;
      const SharedGroups sg = shared_groups(list, p->num_tasks, max_items);
      a.grp_first = sg.first; a.grp_tasks = sg.tasks; a.grp_off = sg.off; a.grp_lmax = sg.lmax;
      if (kv_shards)
        hipLaunchKernelGGL(fill_gap_rows_shards_kernel, dim3((unsigned)p->num_tasks + 1, 64), dim3(256), 0, s, (uint8_t *)dk,
                           (uint8_t *)dv, sg.gap_lo, sg.gap_hi, p->total_k, (int64_t)p->num_heads_kv * kHeadDim * 2, shards);
      else
        hipLaunchKernelGGL(fill_gap_rows_kernel, dim3((unsigned)p->num_tasks + 1, 16), dim3(256), 0, s, (u32x4 *)dk, (u32x4 *)dv,
                           sg.gap_lo, sg.gap_hi, p->total_k, (int64_t)p->num_heads_kv * kHeadDim / 8);
    } else {
      rc = launch_build_schedule(1, cu_q, cu_k, p->num_tasks, bwd_geom(p), list, max_items, s);
      if (rc) return rc;
    }
    // when the list is sized for pieces of tasks over shared K/V rows but the tasks own their rows, the tighter bound
    // sizes the grid (a batch of many short documents and one long one would otherwise launch mostly workgroups
    // that find nothing to do)
    const int64_t grid_items = alias ? max_items : bwd_key_blocks_own_rows(p) + split;
    const int64_t grid = grid_items * p->num_heads_kv * kSchedOversubNum / kSchedOversubDen;
    if (grid > 0x7fffffff) return fail(DISTCA_E_INVALID, "ca_bwd: grid too large");
    a.sched = (const int32_t *)(ws + w.sched_kv);
    a.zero_row = ws + w.sched_kv + sched_zero_row_off(p->num_tasks, max_items);
    a.tickets = (int32_t *)(ws + w.sched_kv + sched_ticket_off(p->num_tasks, max_items));
    ScopedTimer timer(DISTCA_TIMER_CA_BWD, s);
    rc = DISTCA_FN(launch_dkdv64)(a, grid, use_acc, shared, s);
    if (rc) return rc;
  }
  if (use_acc) {
    hipLaunchKernelGGL(cvt_elem_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (const float *)(ws + w.dk_acc), (elem_t *)dk, kv_elems / 8);
    hipLaunchKernelGGL(cvt_elem_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (const float *)(ws + w.dv_acc), (elem_t *)dv, kv_elems / 8);
  }
  (void)q_elems;
  return check_launch("ca_bwd");
}
}  // namespace distca
