// Tile geometry of the attention kernels and the checks every entry point shares.
#pragma once
#include <math.h>
#include <stdlib.h>

#include "api_util.h"
#include "sched.h"

namespace distca {

constexpr int kHeadDim = 128;

// Forward kernel: each wave owns FWD_MSUB sub-tiles of 32 flattened query rows; KV tiles of 64 keys.  One
// sub-tile keeps a wave under 256 registers, so a compute unit holds eight waves.
#ifndef DISTCA_FWD_MSUB
#define DISTCA_FWD_MSUB 1
#endif
#ifndef DISTCA_FWD_WAVES
#define DISTCA_FWD_WAVES 8
#endif
constexpr int kFwdMsub = DISTCA_FWD_MSUB;
constexpr int kFwdWaves = DISTCA_FWD_WAVES;  // waves per workgroup of the forward kernel
constexpr int kFwdRows = kFwdWaves * 32 * kFwdMsub;
constexpr int kDqRows = 256;  // the dQ kernel: four waves of two 32-row sub-blocks
constexpr int kFwdKV = 64;

// dK/dV kernel: a workgroup owns 256 keys (four waves of 64, one per SIMD); query rows are streamed in blocks of
// 32 flattened rows.
constexpr int kBwdRows = 32;
constexpr int kBwdKV = 256;

inline int validate_params(const distca_ca_params *p) {
  if (p->head_dim != kHeadDim) return fail(DISTCA_E_UNSUPPORTED, "head_dim=%d: the kernels are built for head_dim 128 (smaller ones can be zero-padded to it)", p->head_dim);
  if (p->dtype != 0 && p->dtype != DISTCA_DTYPE_BF16 && p->dtype != DISTCA_DTYPE_F16)
    return fail(DISTCA_E_UNSUPPORTED, "dtype=%d: the attention kernels take bf16 (%d, or 0) or fp16 (%d) elements", p->dtype, DISTCA_DTYPE_BF16, DISTCA_DTYPE_F16);
  if (p->num_heads_q <= 0 || p->num_heads_kv <= 0 || p->num_heads_q % p->num_heads_kv)
    return fail(DISTCA_E_INVALID, "num_heads_q=%d must be a positive multiple of num_heads_kv=%d", p->num_heads_q, p->num_heads_kv);
  if (p->num_heads_kv > kSchedMaxHeads) return fail(DISTCA_E_UNSUPPORTED, "num_heads_kv=%d: at most %d kv heads", p->num_heads_kv, kSchedMaxHeads);
  if (p->num_tasks < 0 || p->total_q < 0 || p->total_k < 0 || p->max_seqlen_q < 0 || p->max_seqlen_k < 0)
    return fail(DISTCA_E_INVALID, "negative size in distca_ca_params");
  if (!(p->softmax_scale > 0.f) || !isfinite(p->softmax_scale)) return fail(DISTCA_E_INVALID, "softmax_scale must be positive and finite");
  const int64_t group = p->num_heads_q / p->num_heads_kv;
  if ((int64_t)p->max_seqlen_q * group >= (1ll << 30) || (int64_t)p->total_q * group >= (1ll << 31))
    return fail(DISTCA_E_INVALID, "query rows x heads-per-group exceeds 32-bit tile indexing");
  return DISTCA_OK;
}

// Batches of short tasks have the forward and dQ kernels work off several consecutive blocks of a task per work item
// (sched.h, fwd_merge).  Whether a batch is one is decided from host-known sizes, the mean task length: the kernels
// built for merged items carry a loop around their body, which the ones for long tasks are spared.
#ifndef DISTCA_MERGE_MEAN_TOKENS
#define DISTCA_MERGE_MEAN_TOKENS 2048
#endif
constexpr int32_t kMergeMeanTokens = DISTCA_MERGE_MEAN_TOKENS;  // batches whose tasks average fewer query tokens than this
#ifndef DISTCA_MERGE_TILES_FWD
#define DISTCA_MERGE_TILES_FWD 128
#endif
constexpr int32_t kMergeTilesFwd = DISTCA_MERGE_TILES_FWD;  // KV tiles (of 64 keys) a merged forward item aims for
#ifndef DISTCA_MERGE_TILES_DQ
#define DISTCA_MERGE_TILES_DQ 128
#endif
constexpr int32_t kMergeTilesDq = DISTCA_MERGE_TILES_DQ;    // the same for a merged dQ item (its list counts keys in the same unit)
inline bool merge_short_tasks(const distca_ca_params *p) {
  return p->num_tasks > 0 && (int64_t)p->total_q < (int64_t)kMergeMeanTokens * p->num_tasks;
}
inline SchedGeom fwd_geom(const distca_ca_params *p) {
  SchedGeom g;
  g.split_target = 0;
  g.walk_round = 0;
  g.merge_tiles = merge_short_tasks(p) ? kMergeTilesFwd : 0;
  g.rows_per_block = kFwdRows;
  g.kv_per_block = kFwdKV;
  g.group = p->num_heads_q / p->num_heads_kv;
  g.causal = p->causal != 0;
  const int64_t worst = (int64_t)p->max_seqlen_k / kFwdKV + 1;
  g.cost_shift = pick_cost_shift(worst > g.merge_tiles ? worst : g.merge_tiles);
  return g;
}
// Key blocks are cut into pieces (sched.h) when the batch has so few of them that they could not occupy the
// device twice over, unless the caller asked for a deterministic backward (the pieces' dK/dV are added up with
// float atomics).  Returns the number of pieces to aim for per kv head, 0 = no cutting.
constexpr int kSplitPiecesPerCU = 2;
// Upper bounds, from host-known sizes, of the number of key blocks = sum over tasks of ceil(Lk / kBwdKV).
// When every task has its own K/V rows the Lk add up to total_k at most; when tasks read shared rows
// (kv_task_offsets) only Lk <= max_seqlen_k is known.
inline int64_t bwd_key_blocks_own_rows(const distca_ca_params *p) { return (int64_t)p->total_k / kBwdKV + p->num_tasks + 1; }
inline int64_t bwd_key_blocks_bound(const distca_ca_params *p) {
  const int64_t by_total = bwd_key_blocks_own_rows(p);
  const int64_t by_max = ((int64_t)p->max_seqlen_k / kBwdKV + 1) * p->num_tasks + 1;
  return by_total > by_max ? by_total : by_max;
}
inline int32_t bwd_split_target(const distca_ca_params *p) {
  if (p->deterministic) return 0;
  const int cus = num_compute_units();  // of the current device; 256 when there is none (the host mirror on a CPU box)
  if (bwd_key_blocks_own_rows(p) * p->num_heads_kv >= 2 * cus) return 0;
  const int32_t t = kSplitPiecesPerCU * cus / p->num_heads_kv;
  return t > 0 ? t : 1;
}
inline SchedGeom dq_geom(const distca_ca_params *p) {
  SchedGeom g = fwd_geom(p);
  g.rows_per_block = kDqRows;
  g.merge_tiles = merge_short_tasks(p) ? kMergeTilesDq : 0;  // in the list's cost unit, visible keys / kFwdKV
  return g;
}
inline SchedGeom bwd_geom(const distca_ca_params *p) {
  SchedGeom g;
  g.merge_tiles = 0;
  g.rows_per_block = kBwdRows;
  g.kv_per_block = kBwdKV;
  g.group = p->num_heads_q / p->num_heads_kv;
  g.causal = p->causal != 0;
  g.cost_shift = pick_cost_shift((int64_t)p->max_seqlen_q * g.group / kBwdRows + 1);
  g.split_target = bwd_split_target(p);
  // one round of the dK/dV list per kv head: as many items as compute units serve that head (sched.h, kWalkUp)
  g.walk_round = num_compute_units() / p->num_heads_kv > 0 ? num_compute_units() / p->num_heads_kv : 1;
  return g;
}
// Upper bound of the item count that needs only host-known sizes.
inline int64_t fwd_max_items(const distca_ca_params *p) {
  const int64_t group = p->num_heads_q / p->num_heads_kv;
  return (int64_t)p->total_q * group / kFwdRows + p->num_tasks + 1;
}
inline int64_t dq_max_items(const distca_ca_params *p) {
  const int64_t group = p->num_heads_q / p->num_heads_kv;
  return (int64_t)p->total_q * group / kDqRows + p->num_tasks + 1;
}
inline int64_t bwd_max_items(const distca_ca_params *p) {
  // Without cutting, items are (task, key block) over rows the task owns, or (group of tasks that share rows, key
  // block): either way the blocks tile stored rows.  With cutting (small batches only) tasks over shared rows have an
  // item per task and key block, and cutting adds at most total cost / piece <= split_target pieces (piece_size rounds up).
  const int32_t split = bwd_split_target(p);
  return split > 0 ? bwd_key_blocks_bound(p) + split : bwd_key_blocks_own_rows(p);
}
// The dK/dV list over groups of tasks that share stored K/V rows: an item's cost is the sum over the group's tasks.
inline SchedGeom bwd_shared_geom(const distca_ca_params *p) {
  SchedGeom g = bwd_geom(p);
  g.split_target = 0;
  g.cost_shift = pick_cost_shift((int64_t)p->total_q * g.group / kBwdRows + p->num_tasks + 1);
  return g;
}

int launch_build_schedule(int kind, const int32_t *cu_q, const int32_t *cu_k, int32_t num_tasks, const SchedGeom &g,
                          int32_t *ws, int64_t max_items, hipStream_t stream);
// The dK/dV list over groups of tasks that share stored K/V rows (sched.h, SharedGroups); the region behind `ws` is
// sched_shared_region_bytes long.
int launch_build_shared_schedule(const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off, int32_t num_tasks, int32_t total_k,
                                 const SchedGeom &g, int32_t *ws, int64_t max_items, hipStream_t stream);

inline int64_t align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

}  // namespace distca
