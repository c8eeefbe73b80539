// Device builder and host mirror of the tile schedule described in sched.h.
#include <algorithm>
#include <vector>

#include "api_util.h"
#include "attn_cfg.h"
#include "sched.h"

namespace distca {
namespace {

constexpr int kSchedThreads = 1024;

__device__ __forceinline__ int32_t block_inclusive_scan_i32(int32_t v, int32_t *wave_sums) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int32_t o = __shfl_up(v, off, 64);
    if (lane >= off) v += o;
  }
  __syncthreads();
  if (lane == 63) wave_sums[wave] = v;
  __syncthreads();
  int32_t base = 0;
  for (int w = 0; w < wave; ++w) base += wave_sums[w];
  return v + base;
}

// What the list is made over.  TaskUnits: every task has its own blocks (query blocks in the forward and dQ lists, key
// blocks in the dK/dV list).  GroupUnits (the dK/dV list when tasks share stored K/V rows): a unit is a group of tasks
// that read prefixes of one stored document, its blocks are the document's key blocks, and a block's cost is the sum
// over the group's tasks of the query blocks that see it -- one work item owns a key block's dK/dV on behalf of every
// task, so that the sums need neither atomics nor a fixed-up order.
template <bool BWD>
struct TaskUnits {
  const int32_t *cu_q, *cu_k;
  SchedGeom g;
  __device__ __forceinline__ int32_t blocks(int32_t b) const {
    const int32_t lq = cu_q[b + 1] - cu_q[b], lk = cu_k[b + 1] - cu_k[b];
    const int32_t n = BWD ? bwd_num_blocks(g, lq, lk) : fwd_num_items(g, lq, lk);
    return n < 0 ? 0 : n;
  }
  __device__ __forceinline__ int32_t cost(int32_t b, int32_t i) const {
    const int32_t lq = cu_q[b + 1] - cu_q[b], lk = cu_k[b + 1] - cu_k[b];
    return BWD ? bwd_cost(g, lq, lk, i) : fwd_item_cost(g, lq, lk, i);
  }
};
struct GroupUnits {
  const int32_t *cu_q, *cu_k;
  SchedGeom g;
  const int32_t *grp_first, *grp_tasks, *grp_lmax;
  __device__ __forceinline__ int32_t blocks(int32_t u) const { return ceil_div(grp_lmax[u], g.kv_per_block); }
  __device__ __forceinline__ int32_t cost(int32_t u, int32_t i) const {
    int32_t c = 0;
    for (int32_t e = grp_first[u]; e < grp_first[u + 1]; ++e) {
      const int32_t b = grp_tasks[e];
      const int32_t lq = cu_q[b + 1] - cu_q[b], lk = cu_k[b + 1] - cu_k[b];
      if (i * g.kv_per_block < lk) c += bwd_cost(g, lq, lk, i);
    }
    return c;
  }
};

// Largest b in [0, B) with base[b] <= e.
__device__ __forceinline__ int32_t find_task(const int32_t *base, int32_t num_tasks, int32_t e) {
  int32_t lo = 0, hi = num_tasks;  // invariant: base[lo] <= e < base[hi]
  while (hi - lo > 1) {
    int32_t mid = (lo + hi) >> 1;
    if (base[mid] <= e) lo = mid; else hi = mid;
  }
  return lo;
}

// The sorted list over `num_units` units.  `hdr_units` sizes the header (the task count, whatever the units are).
template <bool BWD, class Units>
__device__ __forceinline__ void build_list(const Units &u, int32_t num_units, int32_t hdr_units, const SchedGeom &g,
                                           int32_t *__restrict__ ws, int32_t max_items) {
  __shared__ int32_t bins[kSchedBins];
  __shared__ int32_t wave_sums[kSchedThreads / 64];
  __shared__ int32_t carry;
  int32_t *base = ws + 4;
  int32_t *items = ws + sched_header_ints(hdr_units);
  const int tid = threadIdx.x;

  // 1. exclusive prefix of block counts per unit
  int32_t running = 0;
  for (int32_t c0 = 0; c0 < num_units; c0 += kSchedThreads) {
    const int32_t b = c0 + tid;
    const int32_t n = b < num_units ? u.blocks(b) : 0;
    const int32_t incl = block_inclusive_scan_i32(n, wave_sums);
    if (b < num_units) base[b] = running + incl - n;
    __syncthreads();
    if (tid == kSchedThreads - 1) carry = running + incl;
    __syncthreads();
    running = carry;
  }
  int32_t nitems = running < max_items ? running : max_items;
  if (tid == 0) base[num_units] = running;
  for (int i = tid; i < kSchedBins; i += kSchedThreads) bins[i] = 0;
  __syncthreads();

  // 1b. (backward, when asked for) the piece size that cuts expensive key blocks
  __shared__ unsigned long long total_cost;
  int32_t piece = 0;
  if (BWD && g.split_target > 0) {
    if (tid == 0) total_cost = 0;
    __syncthreads();
    unsigned long long local = 0;
    for (int32_t e = tid; e < nitems; e += kSchedThreads) {
      const int32_t b = find_task(base, num_units, e);
      local += (unsigned long long)u.cost(b, e - base[b]);
    }
    atomicAdd(&total_cost, local);
    __syncthreads();
    piece = piece_size(total_cost, g.split_target);
  }

  // 2. histogram of cost bins
  for (int32_t e = tid; e < nitems; e += kSchedThreads) {
    const int32_t b = find_task(base, num_units, e);
    const int32_t cost = u.cost(b, e - base[b]);
    const int32_t k = piece_count(cost, piece);
    for (int32_t j = 0; j < k; ++j) atomicAdd(&bins[cost_bin(g, piece_begin(cost, j + 1, k) - piece_begin(cost, j, k))], 1);
  }
  __syncthreads();

  // 3. start offset of each bin when bins are laid out from the most expensive down
  {
    constexpr int kPer = kSchedBins / kSchedThreads;
    int32_t cnt[kPer], local = 0;
#pragma unroll
    for (int v = 0; v < kPer; ++v) {
      cnt[v] = bins[kSchedBins - 1 - (tid * kPer + v)];
      local += cnt[v];
    }
    const int32_t incl = block_inclusive_scan_i32(local, wave_sums);
    int32_t start = incl - local;
    __syncthreads();
#pragma unroll
    for (int v = 0; v < kPer; ++v) {
      bins[kSchedBins - 1 - (tid * kPer + v)] = start;
      start += cnt[v];
    }
  }
  __syncthreads();

  // 4. scatter
  for (int32_t e = tid; e < nitems; e += kSchedThreads) {
    const int32_t b = find_task(base, num_units, e);
    const int32_t i = e - base[b];
    const int32_t cost = u.cost(b, i);
    const int32_t k = piece_count(cost, piece);
    for (int32_t j = 0; j < k; ++j) {
      const int32_t cj = piece_begin(cost, j + 1, k) - piece_begin(cost, j, k);
      const int32_t pos = atomicAdd(&bins[cost_bin(g, cj)], 1);
      if (pos < max_items) {
        int4 it = make_int4(b, i, cj, j | (k << 16));
        reinterpret_cast<int4 *>(items)[pos] = it;
      }
    }
  }
  __syncthreads();
  // 5. (backward) walk direction by rank.  The scatter above puts the entries of one cost bin in whatever order
  // the threads came; an entry's rank in the order (bin, unit, block, piece) is the start of its bin plus the
  // number of entries of the bin that precede it in that order, counted here, and is the same in every run.
  if (BWD && g.walk_round > 0) {
    const int32_t total = bins[0] < max_items ? bins[0] : max_items;
    for (int32_t pos = tid; pos < total; pos += kSchedThreads) {
      const int4 it = reinterpret_cast<const int4 *>(items)[pos];
      const int32_t bin = cost_bin(g, it.z);
      const int32_t seg0 = bin == kSchedBins - 1 ? 0 : bins[bin + 1];  // bins lie from the most expensive down
      const int32_t seg1 = bins[bin] < total ? bins[bin] : total;
      const int64_t key = ((int64_t)(base[it.x] + it.y) << 16) | item_piece(it.w);
      int32_t rank = seg0;
      for (int32_t o = seg0; o < seg1 && seg1 - seg0 <= kWalkTieLimit; ++o) {
        const int4 ot = reinterpret_cast<const int4 *>(items)[o];
        rank += (((int64_t)(base[ot.x] + ot.y) << 16) | item_piece(ot.w)) < key;
      }
      // only the flag bit changes, and the reads above look at the other bits only
      if ((rank / g.walk_round) & 1) items[4 * pos + 3] = it.w | kWalkUp;
    }
    __syncthreads();
  }
  if (tid == 0) {
    // after the scatter the counter of the cheapest bin holds the number of entries
    const int32_t total = bins[0];
    ws[0] = total < max_items ? total : max_items;
    ws[1] = running;
    // entries that found no room in the list (blocks beyond max_items count whole): never 0 < by construction
    // when the caller's sizes bound its sequence lengths; tests and debugging read it
    ws[2] = (total > max_items ? total - max_items : 0) + (running > max_items ? running - max_items : 0);
  }
  if (tid < kZeroRowBytes / 4) ws[sched_zero_row_off(hdr_units, max_items) / 4 + tid] = 0;
  if (tid < kTicketBytes / 4) ws[sched_ticket_off(hdr_units, max_items) / 4 + tid] = 0;
}

template <bool BWD>
__global__ __launch_bounds__(kSchedThreads) void build_schedule_kernel(const int32_t *__restrict__ cu_q,
                                                                     const int32_t *__restrict__ cu_k, int32_t num_tasks,
                                                                     SchedGeom g, int32_t *__restrict__ ws, int32_t max_items) {
  const TaskUnits<BWD> u{cu_q, cu_k, g};
  build_list<BWD>(u, num_tasks, num_tasks, g, ws, max_items);
  if (threadIdx.x == 0) ws[3] = 0;
}

// The dK/dV list over tasks that share stored K/V rows (see GroupUnits and, for the arrays, SharedGroups in sched.h).
// Tasks with queries form a group when they start at the same stored row.  Quadratic in the task count where a task
// looks for its group (a thousand tasks: a thousand comparisons per thread).
__global__ __launch_bounds__(kSchedThreads) void build_shared_schedule_kernel(const int32_t *__restrict__ cu_q,
                                                                            const int32_t *__restrict__ cu_k,
                                                                            const int32_t *__restrict__ kv_off, int32_t num_tasks,
                                                                            int32_t total_k, SchedGeom g, int32_t *__restrict__ ws,
                                                                            int32_t max_items) {
  __shared__ int32_t wave_sums2[kSchedThreads / 64];
  __shared__ int32_t carry2, violations;
  const SharedGroups sg = shared_groups(ws, num_tasks, max_items);
  int32_t *lead = sg.tmp, *gid = sg.tmp + num_tasks;
  const int tid = threadIdx.x;
  auto live = [&](int32_t b) { return cu_q[b + 1] > cu_q[b] && cu_k[b + 1] > cu_k[b]; };
  if (tid == 0) violations = 0;
  // a. the first live task that starts where task b starts
  for (int32_t b = tid; b < num_tasks; b += kSchedThreads) {
    int32_t l = -1;
    if (live(b)) {
      const int32_t off = kv_off[b];
      for (l = 0; l < b; ++l)
        if (kv_off[l] == off && live(l)) break;
    }
    lead[b] = l;
  }
  __syncthreads();
  // b. groups numbered in the order of their first tasks
  int32_t ngroups = 0;
  for (int32_t c0 = 0; c0 < num_tasks; c0 += kSchedThreads) {
    const int32_t b = c0 + tid;
    const int32_t is_lead = b < num_tasks && lead[b] == b ? 1 : 0;
    const int32_t incl = block_inclusive_scan_i32(is_lead, wave_sums2);
    if (is_lead) gid[b] = ngroups + incl - 1;
    __syncthreads();
    if (tid == kSchedThreads - 1) carry2 = ngroups + incl;
    __syncthreads();
    ngroups = carry2;
  }
  for (int32_t u = tid; u <= num_tasks; u += kSchedThreads) {
    sg.first[u] = 0;
    if (u < num_tasks) sg.lmax[u] = 0;
  }
  __syncthreads();
  // c. members, longest prefix and first row of every group
  for (int32_t b = tid; b < num_tasks; b += kSchedThreads)
    if (lead[b] >= 0) {
      const int32_t u = gid[lead[b]];
      atomicAdd(&sg.first[u + 1], 1);
      atomicMax(&sg.lmax[u], cu_k[b + 1] - cu_k[b]);
      if (lead[b] == b) sg.off[u] = kv_off[b];
    }
  __syncthreads();
  if (tid == 0) {  // counts -> exclusive prefix (first[u + 1] holds group u's count)
    int32_t acc = 0;
    for (int32_t u = 0; u < ngroups; ++u) {
      acc += sg.first[u + 1];
      sg.first[u + 1] = acc;
    }
  }
  __syncthreads();
  // d. a group's tasks in the order (prefix length, task): the order its work items walk them in, the same in every run
  for (int32_t b = tid; b < num_tasks; b += kSchedThreads)
    if (lead[b] >= 0) {
      const int32_t l = lead[b], lk = cu_k[b + 1] - cu_k[b];
      int32_t before = 0;
      for (int32_t o = l; o < num_tasks; ++o)
        if (o != b && lead[o] == l) {
          const int32_t lko = cu_k[o + 1] - cu_k[o];
          before += lko < lk || (lko == lk && o < b);
        }
      sg.tasks[sg.first[gid[l]] + before] = b;
    }
  // e. the stored rows no group covers: before the first group, and from the end of a group to the start of the next.
  // Groups must not overlap (tasks that share rows start at the same row); those that do are counted in word 3.
  for (int32_t u = tid; u <= ngroups; u += kSchedThreads) {
    const int32_t lo = u < ngroups ? sg.off[u] + sg.lmax[u] : 0;
    const int32_t from = u < ngroups ? sg.off[u] : -1;
    int32_t hi = total_k;
    for (int32_t o = 0; o < ngroups; ++o)
      if (sg.off[o] > from && sg.off[o] < hi) hi = sg.off[o];
    if (hi < lo) atomicAdd(&violations, 1);
    sg.gap_lo[u] = lo;
    sg.gap_hi[u] = hi;
  }
  for (int32_t u = ngroups + 1 + tid; u <= num_tasks; u += kSchedThreads) sg.gap_lo[u] = sg.gap_hi[u] = 0;
  __syncthreads();
  const GroupUnits u{cu_q, cu_k, g, sg.first, sg.tasks, sg.lmax};
  build_list<true>(u, ngroups, num_tasks, g, ws, max_items);
  if (tid == 0) ws[3] = violations;
}

}  // namespace

int launch_build_schedule(int kind, const int32_t *cu_q, const int32_t *cu_k, int32_t num_tasks, const SchedGeom &g,
                          int32_t *ws, int64_t max_items, hipStream_t stream) {
  if (max_items > 0x7fffffff) return fail(DISTCA_E_INVALID, "schedule: too many work items");
  if (kind == 0)
    hipLaunchKernelGGL((build_schedule_kernel<false>), dim3(1), dim3(kSchedThreads), 0, stream, cu_q, cu_k, num_tasks, g, ws,
                       (int32_t)max_items);
  else
    hipLaunchKernelGGL((build_schedule_kernel<true>), dim3(1), dim3(kSchedThreads), 0, stream, cu_q, cu_k, num_tasks, g, ws,
                       (int32_t)max_items);
  return check_launch("build_schedule");
}

int launch_build_shared_schedule(const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off, int32_t num_tasks, int32_t total_k,
                                 const SchedGeom &g, int32_t *ws, int64_t max_items, hipStream_t stream) {
  if (max_items > 0x7fffffff) return fail(DISTCA_E_INVALID, "schedule: too many work items");
  hipLaunchKernelGGL(build_shared_schedule_kernel, dim3(1), dim3(kSchedThreads), 0, stream, cu_q, cu_k, kv_off, num_tasks, total_k, g,
                     ws, (int32_t)max_items);
  return check_launch("build_shared_schedule");
}

}  // namespace distca

using namespace distca;

extern "C" int distca_ca_tile_shape(int kind, const distca_ca_params *p, int32_t out[2]) {
  if (!p || !out) return fail(DISTCA_E_INVALID, "tile_shape: null pointer");
  int rc = validate_params(p);
  if (rc) return rc;
  SchedGeom g = kind == 0 ? fwd_geom(p) : bwd_geom(p);
  out[0] = g.rows_per_block;  // flattened (token, head-in-group) rows
  out[1] = g.kv_per_block;
  return DISTCA_OK;
}

extern "C" int64_t distca_ca_schedule_capacity(int kind, const distca_ca_params *p) {
  if (!p) return fail(DISTCA_E_INVALID, "schedule_capacity: null params");
  int rc = validate_params(p);
  if (rc) return rc;
  if (kind == 0) return fwd_max_items(p);
  if (kind == 1) return bwd_max_items(p);
  if (kind == 2) return dq_max_items(p);
  return fail(DISTCA_E_INVALID, "schedule_capacity: kind must be 0 (fwd), 1 (bwd dK/dV) or 2 (bwd dQ)");
}

extern "C" int64_t distca_ca_schedule_host(int kind, const int32_t *cu_q, const int32_t *cu_k, const distca_ca_params *p,
                                           int32_t *items, int64_t max_items) {
  if (!p || !cu_q || !cu_k || (!items && max_items > 0)) return fail(DISTCA_E_INVALID, "schedule_host: null pointer");
  int rc = validate_params(p);
  if (rc) return rc;
  if (kind != 0 && kind != 1) return fail(DISTCA_E_INVALID, "schedule_host: kind must be 0 (fwd) or 1 (bwd)");
  const SchedGeom g = kind == 0 ? fwd_geom(p) : bwd_geom(p);
  struct It { int32_t task, block, cost, bin, piece; };
  std::vector<It> whole, v;
  unsigned long long total_cost = 0;
  for (int32_t b = 0; b < p->num_tasks; ++b) {
    const int32_t lq = cu_q[b + 1] - cu_q[b], lk = cu_k[b + 1] - cu_k[b];
    const int32_t n = kind == 0 ? fwd_num_items(g, lq, lk) : bwd_num_blocks(g, lq, lk);
    for (int32_t i = 0; i < n; ++i) {
      const int32_t c = kind == 0 ? fwd_item_cost(g, lq, lk, i) : bwd_cost(g, lq, lk, i);
      whole.push_back({b, i, c, 0, 0});
      total_cost += (unsigned long long)c;
    }
  }
  int32_t piece = 0;
  if (kind == 1 && g.split_target > 0) {
    piece = piece_size(total_cost, g.split_target);
  }
  for (const It &w : whole) {
    const int32_t k = piece_count(w.cost, piece);
    for (int32_t j = 0; j < k; ++j) {
      const int32_t cj = piece_begin(w.cost, j + 1, k) - piece_begin(w.cost, j, k);
      v.push_back({w.task, w.block, cj, cost_bin(g, cj), j | (k << 16)});
    }
  }
  std::stable_sort(v.begin(), v.end(), [](const It &a, const It &b) { return a.bin > b.bin; });
  const int64_t n = (int64_t)v.size();
  if (kind == 1 && g.walk_round > 0)
    for (int64_t s0 = 0, s1; s0 < n; s0 = s1) {  // one cost bin: entries [s0, s1)
      for (s1 = s0 + 1; s1 < n && v[s1].bin == v[s0].bin; ++s1) {}
      for (int64_t e = s0; e < s1; ++e)
        if (((s1 - s0 <= kWalkTieLimit ? e : s0) / g.walk_round) & 1) v[e].piece |= kWalkUp;
    }
  for (int64_t e = 0; e < n && e < max_items; ++e) {
    items[4 * e + 0] = v[e].task;
    items[4 * e + 1] = v[e].block;
    items[4 * e + 2] = v[e].cost;
    items[4 * e + 3] = v[e].piece;
  }
  return n;
}
