// Tile scheduler: turns (cu_seqlens_q, cu_seqlens_k) into a list of work items sorted by
// descending cost, from which the attention kernels' workgroups draw: every workgroup takes
// the next item of its home kv head (workgroup id % Hkv), so that a compute unit that frees up
// continues with the most expensive item left -- longest-processing-time-first balancing
// without a persistent kernel.  Workgroup ids are dealt round-robin over the 8 XCDs, so with
// Hkv = 8 every XCD works on one kv head and its L2 holds only that head's K/V, until that
// head's list is used up (see the ticket counters below).
//
// Cost unit = the causal-pair count the reference's planner balances across ranks
// (Item.get_flops, distca/planner/planner.py:366-378), here at tile granularity.
// The reference itself has no such component on the GPU: flash-attn launches a static
// (m-block, batch, head) grid sized by max_seqlen_q.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define DISTCA_HD __host__ __device__ __forceinline__
#else
#define DISTCA_HD inline
#endif

namespace distca {

struct SchedGeom {
  int32_t rows_per_block;  // flattened (token, head-in-group) query rows per m-block
  int32_t kv_per_block;    // keys per KV block
  int32_t group;           // Hq / Hkv
  int32_t causal;
  int32_t cost_shift;      // bin = min(kSchedBins-1, cost >> cost_shift)
  int32_t split_target;    // backward only, 0 = off: cut expensive key blocks into pieces so that about this
                           // many pieces exist per kv head (see piece_count)
  int32_t walk_round;      // backward only, 0 = off: items whose rank in the list is in an odd group of this many
                           // carry kWalkUp (below)
  int32_t merge_tiles;     // lists over blocks of query rows only, 0 = off: consecutive blocks of a short task form
                           // one work item, as many as bring it to about this many KV tiles (fwd_merge)
};

// Walk direction of a dK/dV item.  A key block streams the query rows that see it, and the compute units of one
// XCD, which share an L2, work on key blocks of one kv head at different places of that stream.  Taken in order
// of cost, the key blocks of a long document that start together from the document's end stay at the same rows
// until the cheapest of them is done; those that follow start one after another as the first ones end, 32 query
// blocks apart for neighbouring key blocks -- exactly the distance between their diagonals, so that a walk from the
// diagonal upwards puts each of them where the others already are, and all of them reach the document's end
// together.  Rounds of as many items as compute units serve one kv head therefore alternate: downwards from the
// end, upwards from the diagonal.  Measured on 131 072 tokens (27 documents, 8 kv heads): HBM reads of the
// kernel 33.6 GB with every walk downwards, 46.3 GB upwards, 22.3 GB alternating in rounds of 32 (16, 24, 40, 64:
// 42.9, 40.0, 38.2, 34.6 GB).  The rank that decides is the item's place in the order (cost bin descending, task,
// block, piece), which does not depend on how the builder's threads interleave, so that an item's sums are added
// in the same order in every run.
// Entries of one cost bin are ranked among themselves only when the bin holds at most this many (the count is
// quadratic in the bin); the entries of a larger bin all take the rank of its first one.  Their costs are equal, so
// they begin and end together round after round, which is the case a common direction suits.
constexpr int32_t kWalkTieLimit = 64;
constexpr int32_t kWalkUp = (int32_t)0x80000000u;  // flag in an item's fourth word, beside piece | pieces << 16
DISTCA_HD int32_t item_piece(int32_t w) { return w & 0xffff; }
DISTCA_HD int32_t item_pieces(int32_t w) { return (w >> 16) & 0x7fff; }

// Cutting key blocks: a batch of few tokens has fewer key blocks than the device has compute units, and
// the block at the start of a long document streams every query row below it, so without cuts the launch
// lasts as long as that one workgroup.  A block of cost c (query blocks to stream) is cut into
// ceil(c / piece) pieces of consecutive query blocks, piece = max(kMinPiece, ceil(total cost / split_target));
// the pieces are independent work items whose dK/dV are added up in fp32.
constexpr int32_t kMinPiece = 16;
constexpr int32_t kMaxPieces = 64;
// Piece size for a batch of `total_cost` query-block visits: the ceiling of total / target, so that the pieces
// of all blocks together number at most target + (number of blocks) -- the bound the work list is sized by
// (sum of ceil(c / piece) <= total / piece + blocks, and total / piece <= target only when piece is rounded up).
DISTCA_HD int32_t piece_size(unsigned long long total_cost, int32_t split_target) {
  if (split_target <= 0) return 0;
  const unsigned long long per = (total_cost + (unsigned long long)split_target - 1) / (unsigned long long)split_target;
  if (per <= (unsigned long long)kMinPiece) return kMinPiece;
  return per < 0x7fffffffull ? (int32_t)per : 0x7fffffff;
}
DISTCA_HD int32_t piece_count(int32_t cost, int32_t piece) {
  if (piece <= 0) return 1;
  int32_t k = (cost + piece - 1) / piece;
  return k < 1 ? 1 : (k > kMaxPieces ? kMaxPieces : k);
}
// query blocks [lo, hi) of piece j of k over n blocks, counted from the last block downwards
DISTCA_HD int32_t piece_begin(int32_t n, int32_t j, int32_t k) { return (int32_t)(((int64_t)n * j) / k); }

constexpr int kSchedBins = 4096;

DISTCA_HD int32_t ceil_div(int32_t a, int32_t b) { return (a + b - 1) / b; }

// forward: blocks of query rows
DISTCA_HD int32_t fwd_num_blocks(const SchedGeom &g, int32_t lq) { return ceil_div(lq * g.group, g.rows_per_block); }

// Keys visible to the last token of m-block i (0 when none): the KV extent the block streams.
DISTCA_HD int32_t fwd_visible_keys(const SchedGeom &g, int32_t lq, int32_t lk, int32_t i) {
  int32_t tok_end = ceil_div((i + 1) * g.rows_per_block, g.group);  // one past the last token
  if (tok_end > lq) tok_end = lq;
  int32_t nvis = g.causal ? tok_end + (lk - lq) : lk;
  if (nvis > lk) nvis = lk;
  return nvis > 0 ? nvis : 0;
}
DISTCA_HD int32_t fwd_cost(const SchedGeom &g, int32_t lq, int32_t lk, int32_t i) {
  return ceil_div(fwd_visible_keys(g, lq, lk, i), g.kv_per_block);
}

// Short tasks: a block of query rows that sees a handful of KV tiles spends a third of its workgroup's time outside the
// tile loop (drawing its ticket, loading the item and its bounds, waiting for Q and the first tile, draining the
// output).  With merge_tiles set, every work item of a task is `fwd_merge` consecutive blocks, which one workgroup
// works off one after the other: the ticket and the task's bounds are paid once, and what the next block needs can
// be requested while the present one finishes.  The number depends on the task alone (its most expensive block, the
// last one), so the kernel finds the blocks of item i without a table: blocks i * m .. min((i + 1) * m, blocks) - 1.
constexpr int32_t kMaxMerge = 8;
DISTCA_HD int32_t fwd_merge(const SchedGeom &g, int32_t lq, int32_t lk) {
  if (g.merge_tiles <= 0) return 1;
  const int32_t n = fwd_num_blocks(g, lq);
  if (n <= 1) return 1;
  const int32_t worst = fwd_cost(g, lq, lk, n - 1);
  int32_t m = g.merge_tiles / (worst > 0 ? worst : 1);
  return m < 1 ? 1 : (m > kMaxMerge ? kMaxMerge : m);
}
DISTCA_HD int32_t fwd_num_items(const SchedGeom &g, int32_t lq, int32_t lk) { return ceil_div(fwd_num_blocks(g, lq), fwd_merge(g, lq, lk)); }
DISTCA_HD int32_t fwd_item_cost(const SchedGeom &g, int32_t lq, int32_t lk, int32_t i) {
  const int32_t m = fwd_merge(g, lq, lk);
  if (m == 1) return fwd_cost(g, lq, lk, i);
  const int32_t n = fwd_num_blocks(g, lq);
  int32_t c = 0;
  for (int32_t b = i * m; b < (i + 1) * m && b < n; ++b) c += fwd_cost(g, lq, lk, b);
  return c;
}

// backward: blocks of keys
DISTCA_HD int32_t bwd_num_blocks(const SchedGeom &g, int32_t lq, int32_t lk) {
  return lq > 0 ? ceil_div(lk, g.kv_per_block) : 0;
}
// First m-block that sees any key of KV block n.
DISTCA_HD int32_t bwd_first_mblock(const SchedGeom &g, int32_t lq, int32_t lk, int32_t n) {
  if (!g.causal) return 0;
  int32_t t_first = n * g.kv_per_block - (lk - lq);
  if (t_first < 0) t_first = 0;
  return (int32_t)(((int64_t)t_first * g.group) / g.rows_per_block);
}
DISTCA_HD int32_t bwd_cost(const SchedGeom &g, int32_t lq, int32_t lk, int32_t n) {
  int32_t c = fwd_num_blocks(g, lq) - bwd_first_mblock(g, lq, lk, n);
  return c > 0 ? c : 0;
}

DISTCA_HD int32_t cost_bin(const SchedGeom &g, int32_t cost) {
  int32_t b = cost >> g.cost_shift;
  return b < kSchedBins - 1 ? b : kSchedBins - 1;
}

inline int32_t pick_cost_shift(int64_t max_cost) {
  int32_t s = 0;
  while ((max_cost >> s) >= kSchedBins) ++s;
  return s;
}

// Workspace layout of a schedule (all int32):
//   [0] item count   [1] blocks   [2] entries dropped for lack of room (0 unless the caller's sizes understate
//   its sequence lengths)   [3] reserved   [4 .. 4+B] exclusive block prefix per task
//   then items as (task, block, cost, piece | pieces << 16 [| kWalkUp]) quadruples, 16-byte aligned.
DISTCA_HD int64_t sched_header_ints(int32_t num_tasks) { return ((int64_t)4 + num_tasks + 1 + 3) / 4 * 4; }
DISTCA_HD int64_t sched_bytes(int32_t num_tasks, int64_t max_items) {
  return (sched_header_ints(num_tasks) + 4 * max_items) * (int64_t)sizeof(int32_t);
}
// A schedule region ends with 256 zero bytes, written by the builder: the attention kernels
// point the tile loads of rows that do not exist (past the end of a task) at them, so that such
// rows are finite whatever the neighbouring memory holds.
constexpr int64_t kZeroRowBytes = 256;
DISTCA_HD int64_t sched_zero_row_off(int32_t num_tasks, int64_t max_items) {
  return (sched_bytes(num_tasks, max_items) + 255) / 256 * 256;
}
// After the zero row: one ticket counter per kv head, zeroed by the builder.  The attention kernels
// are launched with 5/4 workgroups per (item, kv head) -- the surplus is what a fast XCD takes over from
// a slow one; the XCDs of a device were seen up to 8 % apart -- and a workgroup does not work on the
// item its id names: it draws the next ticket of its home head (id % Hkv), which is the rank of its
// item in the sorted list, and when that head's list is used up it draws from the other heads; it
// exits when all are used up.  Workgroup ids are dealt round-robin over the XCDs, and the XCDs of one
// device do not run at the same speed (several per cent apart on the same work): with one workgroup
// per item the kernel lasted as long as the slowest XCD took for its fixed eighth of the list,
// whereas now an XCD that finishes its own heads early takes items of the others.
constexpr int64_t kTicketBytes = 1024;
constexpr int32_t kSchedMaxHeads = (int32_t)(kTicketBytes / 4);
constexpr int32_t kSchedOversubNum = 5, kSchedOversubDen = 4;
DISTCA_HD int64_t sched_ticket_off(int32_t num_tasks, int64_t max_items) {
  return sched_zero_row_off(num_tasks, max_items) + kZeroRowBytes;
}
DISTCA_HD int64_t sched_region_bytes(int32_t num_tasks, int64_t max_items) {
  return sched_ticket_off(num_tasks, max_items) + kTicketBytes;
}

// The dK/dV list of a batch whose tasks share stored K/V rows (kv_task_offsets) is made over groups: the tasks
// (with queries) that start at one stored row read prefixes of one stored document, and a work item
// (group, key block) walks the query blocks of every task of the group whose prefix holds the block, so that the
// block's dK/dV are summed in registers and written once: no atomics, no accumulators in memory, the same bits in
// every run.  Tasks that start at different rows must not share rows (the builder counts the groups that run into
// the next one in word 3 of the list's header).  Behind the ticket counters the region then holds, all int32:
//   first [B + 1]   group u's tasks are tasks[first[u] .. first[u + 1]), by (prefix length, task index)
//   tasks [B]
//   off   [B]       first stored row of the group        lmax [B]   its longest prefix
//   gap_lo, gap_hi [B + 1]   stored rows [gap_lo[u], gap_hi[u]) belong to no group (zeroed by the backward): from the
//                            end of group u to the start of the next one; entry `number of groups`: the rows before
//                            the first group
//   tmp   [2 B]     scratch of the builder
struct SharedGroups {
  int32_t *first, *tasks, *off, *lmax, *gap_lo, *gap_hi, *tmp;
};
DISTCA_HD int64_t shared_groups_ints(int32_t num_tasks) { return ((int64_t)8 * ((int64_t)num_tasks + 1) + 63) / 64 * 64; }
DISTCA_HD int64_t sched_shared_region_bytes(int32_t num_tasks, int64_t max_items) {
  return sched_region_bytes(num_tasks, max_items) + shared_groups_ints(num_tasks) * (int64_t)sizeof(int32_t);
}
DISTCA_HD SharedGroups shared_groups(int32_t *ws, int32_t num_tasks, int64_t max_items) {
  int32_t *p = ws + sched_region_bytes(num_tasks, max_items) / (int64_t)sizeof(int32_t);
  const int64_t b = num_tasks;
  SharedGroups g;
  g.first = p;
  g.tasks = p + (b + 1);
  g.off = p + (2 * b + 1);
  g.lmax = p + (3 * b + 1);
  g.gap_lo = p + (4 * b + 1);
  g.gap_hi = p + (5 * b + 2);
  g.tmp = p + (6 * b + 3);
  return g;
}

#if defined(__HIPCC__)
// Draws this workgroup's (item rank, kv head); false when every list is used up.  `slot` is two ints
// of LDS that the caller may reuse afterwards.  All threads of the workgroup must call it.
__device__ __forceinline__ bool take_item(int32_t *tickets, int32_t nitems, int32_t hkv, int32_t *slot, int &item, int &kvh) {
  if (threadIdx.x < 64) {  // the first wave
    // One look at all the counters at once (a lane per head): a workgroup that comes when every list is used
    // up -- half of the launch's workgroups -- leaves after a single round trip to memory.  Counters only
    // grow: a list seen as used up stays so, and a stale smaller value only costs an atomic.
    const int lane = threadIdx.x;
    const int home = (int)(blockIdx.x % (unsigned)hkv);
    int t = -1, q = home;
    for (int base = 0; base < hkv && t < 0; base += 64) {
      int h = home + base + lane;
      while (h >= hkv) h -= hkv;
      const bool live = base + lane < hkv && __builtin_nontemporal_load(tickets + h) < nitems;
      unsigned long long avail = __ballot(live);
      // heads in the order home, home + 1, ...: lane d of this round looked at head home + base + d
      while (avail && t < 0) {
        const int d = __builtin_ctzll(avail);
        avail &= avail - 1;
        q = home + base + d;
        while (q >= hkv) q -= hkv;
        if (lane == 0) {
          t = atomicAdd(tickets + q, 1);
          if (t >= nitems) t = -1;
        }
        t = __shfl(t, 0, 64);
      }
    }
    if (lane == 0) {
      slot[0] = t;
      slot[1] = q;
    }
  }
  __syncthreads();
  item = __builtin_amdgcn_readfirstlane(slot[0]);
  kvh = __builtin_amdgcn_readfirstlane(slot[1]);
  __syncthreads();
  return item >= 0;
}
#endif

}  // namespace distca
