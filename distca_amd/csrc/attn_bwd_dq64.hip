// dQ of the varlen causal attention backward for gfx950, 64 query rows per wave.
//
// One workgroup of 4 waves per (task, block of 256 flattened query rows, kv head), one wave per SIMD with the
// SIMD's whole register file.  A wave owns two sub-blocks of 32 rows: their Q and dO stay in registers as MFMA B
// operands, their dQ^T accumulators in the accumulation registers.  K/V tiles of 32 keys stream through a ring of
// four LDS stages by LDS-direct loads, from key 0 up to the last key the block's rows see; every LDS fragment a
// wave reads (K rows, V rows, transposed K) feeds two MFMAs, one per sub-block: half the LDS bytes per MFMA of
// a wave that owns 32 rows.  With one wave per SIMD the arithmetic of a tile is written between the MFMAs of the
// same tile, as in the dK/dV kernel (attn_bwd_dkdv64.hip):
//
//   step 1   S^T  = K Q^T        16 MFMAs   A: rows of the K tile (LDS), B: Q registers
//   step 2   dP^T = V dO^T       16 MFMAs   A: rows of the V tile, B: dO registers      beside them: P from S
//   step 3   dQ^T += K^T dS^T    16 MFMAs   A: transposing reads of the K tile, B: dS   beside them: dS = P (dP - delta)
//                                           of the keys and sub-block whose MFMAs come later in the step
//
// The prologue also makes the row statistics of the backward (delta = <dO, O>, lse in the log2 domain) and leaves
// them in the workspace for the dK/dV kernel, which runs after this one.
#include "api_util.h"
#include "attn_bwd.h"
#include "attn_cfg.h"
#include "common.h"

#include <type_traits>

namespace distca {
namespace {

constexpr int kThreads = 256;
constexpr int kRowsWg = 256;            // flattened query rows per workgroup (kDqRows)
constexpr int kKeys = 32;               // keys per tile
constexpr int kRow = 256;               // bytes per tile row, chunks swizzled by tile_swz
constexpr int kTile = kKeys * kRow;
constexpr int kStageBytes = 2 * kTile;  // K tile, V tile
constexpr int kStages = 4;
constexpr int kLdsRing = kStages * kStageBytes;
constexpr int kRowsLds = 3 * kTile;        // per wave, behind the ring: 32 rows of Q, dO and O on their way in, 64 rows of dQ on their way out
constexpr int kLds = kLdsRing + 4 * kRowsLds;
static_assert(kLds <= 160 * 1024 && kRowsLds >= 64 * kRow, "LDS of a compute unit");
constexpr int kLoadsPerTile = 4;        // vector-memory instructions a wave issues per tile
constexpr float kLog2e = 1.4426950408889634f;
constexpr int kLead = 2;                // fragments by which sub-block 0 leads in the dQ step
constexpr int kFrags = 4;               // transposed K fragments held at a time
static_assert(kDqRows == kRowsWg, "the dQ work list is built for blocks of 256 rows");

template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void fence() { __builtin_amdgcn_sched_barrier(0); }
// The S and dP accumulators are read and overwritten by the vector ALU and must live in vector registers; this file
// is compiled with the compiler's default MFMA form (results in the accumulation registers, right for dQ), so
// these MFMAs are written as assembly.  The compiler does not space such an instruction from the vector
// instructions that read its result (an eight-pass MFMA: 11 quad-cycles from its issue): the order of a tile's
// instructions below, held in place by the scheduling fences, keeps between every such MFMA and the first read of its
// result either two later MFMAs, or one later MFMA (which cannot start before the pipe has finished the eight passes
// of the one in question) and at least four vector instructions; a change to the tile body has to keep that.
__device__ __forceinline__ void mfma32_v(f32x16 &acc, elemx8 a, elemx8 b) {
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_vc(f32x16 &acc, elemx8 a, elemx8 b, const f32x16 &c0) {  // acc = A B + c0
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "v"(b), "v"(c0));
}
// The same with the B operand in accumulation registers, where Q lives: a wave's 512 registers are 256 of each
// kind, and the vector half is what the tile arithmetic is short of.
typedef float accop_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ accop_t to_acc_regs(elemx8 v) {
  accop_t r;
  asm volatile("; operand to accumulation registers" : "=a"(r) : "0"(__builtin_bit_cast(accop_t, v)));
  return r;
}
__device__ __forceinline__ void mfma32_va(f32x16 &acc, elemx8 a, accop_t b) {
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(b));
}
__device__ __forceinline__ void mfma32_va0(f32x16 &acc, elemx8 a, accop_t b) {
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b));
}

// SEG: K/V rows are addressed through a table of shards (kv_shards.h) instead of as one dense tensor.
// MERGE: a work item is several consecutive blocks of a task's query rows (sched.h, fwd_merge), worked off one after the
// other; otherwise it is one block.
template <bool SEG, bool MERGE>
__global__ __launch_bounds__(kThreads, 1) void ca_bwd_dq64_kernel(BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int nitems = a.sched[0];
  int item, kvh;
  if (!take_item(a.tickets, nitems, a.hkv, reinterpret_cast<int32_t *>(lds), item, kvh)) return;
  int4 it4 = reinterpret_cast<const int4 *>(a.sched + a.sched_items_off)[item];
  it4.x = uniform_int(it4.x);
  it4.y = uniform_int(it4.y);
  const int task = it4.x;

  // The task's bounds and offsets: every load is issued before the first is used (the optional arrays are read
  // through a pointer that falls back to a place that is always readable, instead of under a branch each: with a
  // branch per array the loads went to memory one after the other, six trips before the kernel could start).
  const int32_t *cq = a.cu_q + task, *ck = a.cu_k + task;
  const int32_t *kvp = a.kv_off ? a.kv_off + task : ck;
  const int64_t *spare = reinterpret_cast<const int64_t *>(a.zero_row);
  const int64_t *qsp = a.qs_task_off ? a.qs_task_off + task : spare, *dqp = a.dq_task_off ? a.dq_task_off + task : spare;
  const int q0_ = cq[0], q1_ = cq[1], k0_ = ck[0], k1_ = ck[1], ks_ = *kvp;
  const int64_t qs_given_ = *qsp, dq_given_ = *dqp;
  fence();
  const int q0 = uniform_int(q0_), q1 = uniform_int(q1_), k0 = uniform_int(k0_), k1 = uniform_int(k1_), ks = uniform_int(ks_);
  const int64_t qs_given = uniform_int64(qs_given_), dq_given = uniform_int64(dq_given_);
  const int64_t qs_task = a.qs_task_off ? qs_given : (int64_t)q0 * a.qs_tok_bytes;
  const int64_t dq_task = a.dq_task_off ? dq_given : (int64_t)q0 * a.dq_tok_bytes;
  const int lq = q1 - q0;
  const int lk = k1 - k0;
  const int G = a.group;
  const int shift = lk - lq;

  const int nrows = lq * G;
  // the blocks of this item
  int mb_first = it4.y, mb_end = it4.y + 1;
  if constexpr (MERGE) {
    SchedGeom geom;
    geom.rows_per_block = kRowsWg; geom.kv_per_block = kFwdKV; geom.group = G; geom.causal = a.causal; geom.merge_tiles = a.merge_tiles;
    const int m = fwd_merge(geom, lq, lk), nblk = (nrows + kRowsWg - 1) / kRowsWg;
    mb_first = it4.y * m;
    mb_end = mb_first + m < nblk ? mb_first + m : nblk;
  }
  // (a jump back rather than a loop statement: without MERGE the body below is then straight-line code, exactly the
  // kernel that takes one block per item)
  int mblk = mb_first;
  bool requested = false;  // MERGE: the first sub-block's rows of this block are already on their way
next_block:
  // MERGE: the thread index is made opaque once per block, so that what derives from it is computed afresh for every
  // block instead of being carried, and partly spilled, across the whole body
  int tid_ = threadIdx.x;
  if constexpr (MERGE) asm volatile("" : "+v"(tid_));
  const int tid = tid_, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int row_wg = mblk * kRowsWg;

  int tok_end = (row_wg + kRowsWg + G - 1) / G;
  if (tok_end > lq) tok_end = lq;
  int nvis = a.causal ? tok_end + shift : lk;
  if (nvis > lk) nvis = lk;
  const int ntiles = nvis > 0 ? (nvis + kKeys - 1) / kKeys : 0;

  const uint32_t lds0 = (uint32_t)(uintptr_t)(DISTCA_LDS uint8_t *)lds;
  auto div_group = [&](int n) { return a.group_magic ? (int)__umulhi((uint32_t)n, a.group_magic) : n; };

  // ---- K/V tile fetch: this wave brings rows 8 w .. 8 w + 7 of the K tile and of the V tile, four rows per
  // instruction.  Tiles that lie wholly inside the prefix take a form without per-lane address arithmetic (a scalar
  // base that advances by one tile, per-lane offsets that never change); rows past the prefix read the zero row.
  const int64_t kv_stride = (int64_t)a.hkv * kHeadDim;
  const elem_t *kbase = a.k + (SEG ? 0 : (int64_t)ks * kv_stride) + kvh * kHeadDim;
  const elem_t *vbase = a.v + (SEG ? 0 : (int64_t)ks * kv_stride) + kvh * kHeadDim;
  ShardCursor cur;  // SEG: the shard that holds the rows of the tile requested next
  if constexpr (SEG) cur.open(a.shards, a.shards.task_shard[task]);
  uint32_t voff[2];
#pragma unroll
  for (int ii = 0; ii < 2; ++ii) {
    const int r = 8 * wave + 4 * ii + (lane >> 4);
    voff[ii] = (uint32_t)((r * kv_stride + (((lane & 15) ^ tile_swz(r)) * 8)) * 2);
  }
  // SEG: tiles that end at or before key run_lim lie in the present shard, key x of the prefix at kvirt / vvirt +
  // x * kv_stride; a tile past it looks for its shard first, so that a run of tiles inside one shard is requested
  // exactly as tiles of a dense tensor are.
  const elem_t *kvirt = kbase, *vvirt = vbase;
  int run_lim = SEG ? 0 : lk;
  auto issue_whole = [&](uint32_t dst, int j) {
    const elem_t *kt = kvirt + (int64_t)j * kKeys * kv_stride, *vt = vvirt + (int64_t)j * kKeys * kv_stride;
    lds_direct_load16(kt, voff[0], dst);
    lds_direct_load16(kt, voff[1], dst + 4 * kRow);
    lds_direct_load16(vt, voff[0], dst + kTile);
    lds_direct_load16(vt, voff[1], dst + kTile + 4 * kRow);
  };
  auto issue_tile = [&](int stage, int j) {
    const uint32_t dst = lds0 + stage * kStageBytes + 8 * wave * kRow;
    if constexpr (SEG) {
      if ((j + 1) * kKeys <= run_lim) {
        issue_whole(dst, j);
        return;
      }
      const int r0 = ks + j * kKeys;
      cur.seek(a.shards, r0);
      if ((j + 1) * kKeys <= lk && cur.holds(r0, kKeys)) {
        const int64_t back = (int64_t)(cur.lo - ks) * kv_stride * 2;
        kvirt = reinterpret_cast<const elem_t *>(static_cast<uintptr_t>(uniform_i64((int64_t)reinterpret_cast<uintptr_t>(kbase) + cur.k - back)));
        vvirt = reinterpret_cast<const elem_t *>(static_cast<uintptr_t>(uniform_i64((int64_t)reinterpret_cast<uintptr_t>(vbase) + cur.v - back)));
        run_lim = uniform_i32(cur.hi - ks < lk ? cur.hi - ks : lk);
        issue_whole(dst, j);
        return;
      }
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        const int r = 8 * wave + 4 * ii + (lane >> 4);
        const int key = j * kKeys + r;
        const int chunk = (lane & 15) ^ tile_swz(r);
        const bool ok = key < lk;
        const uint8_t *zero = reinterpret_cast<const uint8_t *>(a.zero_row);
        const uint8_t *kp = ok ? reinterpret_cast<const uint8_t *>(kbase) + shard_row_offset(a.shards, cur, ks + key, 0, kv_stride * 2) : zero;
        const uint8_t *vp = ok ? reinterpret_cast<const uint8_t *>(vbase) + shard_row_offset(a.shards, cur, ks + key, 1, kv_stride * 2) : zero;
        lds_direct_load16_ptr(kp + chunk * 16, dst + 4 * ii * kRow);
        lds_direct_load16_ptr(vp + chunk * 16, dst + kTile + 4 * ii * kRow);
      }
    } else {
      if ((j + 1) * kKeys <= lk) {
        const elem_t *kt = kbase + (int64_t)j * kKeys * kv_stride, *vt = vbase + (int64_t)j * kKeys * kv_stride;
        lds_direct_load16(kt, voff[0], dst);
        lds_direct_load16(kt, voff[1], dst + 4 * kRow);
        lds_direct_load16(vt, voff[0], dst + kTile);
        lds_direct_load16(vt, voff[1], dst + kTile + 4 * kRow);
        return;
      }
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        const int r = 8 * wave + 4 * ii + (lane >> 4);
        const int key = j * kKeys + r;
        const int chunk = (lane & 15) ^ tile_swz(r);
        const bool ok = key < lk;
        const elem_t *kp = ok ? kbase + (int64_t)key * kv_stride : reinterpret_cast<const elem_t *>(a.zero_row);
        const elem_t *vp = ok ? vbase + (int64_t)key * kv_stride : reinterpret_cast<const elem_t *>(a.zero_row);
        lds_direct_load16_ptr(kp + chunk * 8, dst + 4 * ii * kRow);
        lds_direct_load16_ptr(vp + chunk * 8, dst + kTile + 4 * ii * kRow);
      }
    }
  };

  // The first two tiles are requested before the block's own rows: they land in the ring while the rows pass through
  // the part of LDS behind it.
  if (ntiles > 0) {
    issue_tile(0, 0);
    issue_tile(1, 1);
  }

  // ---- this lane's two rows: Q and dO as B operands (row l32 of a sub-block, d = 16 s + 8 g .. +7), statistics
  int row[2], tok[2], lim[2];
  bool valid[2];
  float lse2[2], delta[2];
  accop_t qf[2][8];
  elemx8 dof[2][8];
  // The wave's 64 rows of Q, dO and O come through LDS: LDS-direct loads bring four whole rows of 256 bytes per
  // instruction, and the lanes then read their operand fragments (row l32 of a sub-block, chunk 2 s + g) from there.
  // Loaded straight into the operand layout, every load instruction touched 32 rows, 32 bytes of each, and the address
  // unit takes about a cycle per cache line it has to look up: 48 such loads per wave took 7.7 us to *issue*, a third
  // of what a block of a 1024-token document then spent in its tile loop.  The rows use the 24 KB per wave that lie
  // behind the tile ring (the 32 rows of a sub-block of Q, dO and O at a time), so the ring is free for the first tiles
  // meanwhile, and each wave reads only what it has loaded itself: no barrier.
  // Before that, and also in one batch, the lse of the lane's two rows (the opaque statements that move Q into the
  // accumulation registers order memory accesses around themselves: no load may be left between them).
  float lse_row[2];
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    row[m] = row_wg + (wave * 2 + m) * 32 + l32;
    valid[m] = row[m] < nrows;
    // A row past the task (the last block of a task only) reads the task's last row instead, without a branch: with
    // lse2 = +inf its P and dS are zero whatever Q and dO hold, as long as they are finite, and nothing of it is stored.
    const int rc = valid[m] ? row[m] : nrows - 1;
    tok[m] = div_group(rc);
    const int hg = rc - tok[m] * G;
    int lm = a.causal ? tok[m] + shift : lk - 1;
    if (lm > lk - 1) lm = lk - 1;
    lim[m] = lm;
    lse_row[m] = a.lse_tok ? reinterpret_cast<const float *>(a.lse_tok + qs_task + (int64_t)tok[m] * a.qs_tok_bytes)[kvh * G + hg]
                           : a.lse[(int64_t)(kvh * G + hg) * a.total_q + q0 + tok[m]];
  }
  const int wrow0 = row_wg + wave * 64;
  const uint32_t stg = lds0 + kLdsRing + wave * kRowsLds;  // [Q | dO | O] of one sub-block, 8 KB each
  // requests sub-block m of the wave's rows in block `blk` of the task: instruction i brings rows 32 m + 4 i + lane / 16
  // of the wave, lane % 16 being the position of the 16-byte chunk in the (swizzled) LDS row
  auto request_rows = [&](int blk, int m) {
    const int rw = blk * kRowsWg;
    const int tok0 = div_group(rw);
    const int64_t base = qs_task + (int64_t)tok0 * a.qs_tok_bytes + (int64_t)kvh * G * kHeadDim * 2;
    const uint8_t *qb = reinterpret_cast<const uint8_t *>(a.q) + base, *dob = reinterpret_cast<const uint8_t *>(a.dout) + base,
                  *ob = reinterpret_cast<const uint8_t *>(a.out) + base;
    uint32_t roff[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = 32 * m + 4 * i + (lane >> 4);
      int rg = rw + wave * 64 + r;
      if (rg > nrows - 1) rg = nrows - 1;
      const int t = div_group(rg);
      roff[i] = (uint32_t)((t - tok0) * a.qs_tok_bytes + (rg - t * G) * (kHeadDim * 2) + (((lane & 15) ^ tile_swz(r)) << 4));
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) lds_direct_load16(qb, roff[i], stg + i * 4 * kRow);
#pragma unroll
    for (int i = 0; i < 8; ++i) lds_direct_load16(dob, roff[i], stg + kTile + i * 4 * kRow);
#pragma unroll
    for (int i = 0; i < 8; ++i) lds_direct_load16(ob, roff[i], stg + 2 * kTile + i * 4 * kRow);
  };
  {
    const uint32_t frag = l32 * kRow + ((g ^ tile_swz(l32)) << 4);  // this lane's chunk 0 of row l32; ^ (s << 5)
    elemx8 qt[2][8], ot[2][8];
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      // MERGE: the first sub-block's rows were requested before the previous block of the item stored its results
      if (!(MERGE && m == 0 && requested)) request_rows(mblk, m);
      wait_vm<0>();  // (the first tiles, requested before, and lse as well)
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        qt[m][s] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(stg + (frag ^ (s << 5))));
        dof[m][s] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(stg + kTile + (frag ^ (s << 5))));
        ot[m][s] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(stg + 2 * kTile + (frag ^ (s << 5))));
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the reads are done before the place is filled again
    }
    fence();
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      float part = 0.f;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        qf[m][s] = to_acc_regs(qt[m][s]);
#pragma unroll
        for (int i = 0; i < 8; ++i) part += (float)dof[m][s][i] * (float)ot[m][s][i];
      }
      delta[m] = pair_sum(part);  // this lane's half of d, then the sum of the lane pair
      lse2[m] = valid[m] ? lse_row[m] * kLog2e : INFINITY;  // rows past the task: P = exp2(-inf) = 0
    }
  }
  // -delta of the lane's row in all 16 registers of a vector: the C operand of a tile's first dP MFMA, so that
  // dS = P * (what the MFMAs leave) costs one instruction per element
  f32x16 ndl[2];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int r = 0; r < 16; ++r) ndl[m][r] = -delta[m];
  int wrow1 = wrow0 + 63;
  if (wrow1 > nrows - 1) wrow1 = nrows - 1;
  const bool wave_live = wrow0 < nrows;
  int lim_first = 0x7fffffff, lim_last = -1;
  if (wave_live) {
    lim_first = a.causal ? wrow0 / G + shift : lk - 1;
    if (lim_first > lk - 1) lim_first = lk - 1;
    lim_last = a.causal ? wrow1 / G + shift : lk - 1;
    if (lim_last > lk - 1) lim_last = lk - 1;
  }

  f32x16 dqacc[2][4];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) dqacc[m][db][r] = 0.f;
  const float c = a.scale * kLog2e;
  const int k_rd = l32 * kRow + ((g ^ tile_swz(l32)) << 4);  // A operand rows of a tile, ^ 32*s
  // transposed K operand: lane points at (key 4g + i4 [+8 hi +16 t], chunk 8 b4 + h1 [+2 db], half lane&1);
  // tile_swz of that row is (i4<<1) | (g<<3) | hi
  const int i4 = (lane & 15) >> 2, b4 = (lane >> 4) & 1, h1 = (lane & 3) >> 1;
  const int t_rd = (4 * g + i4) * kRow + ((((b4 ^ g) << 3) | (i4 << 1) | h1) << 4) + 8 * (lane & 1);  // ^ 32*db ^ 16*hi

  // Absolute LDS addresses of this lane's operand reads in stage 0, the eight swizzled variants of each read shape,
  // kept in registers: where the stage is a constant (the unrolled loop below) stage and tile sit in the read
  // instruction's offset field and no address arithmetic is left between the MFMAs.
  uint32_t k_ad[8], t_ad[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    k_ad[i] = lds0 + (k_rd ^ (i << 5));
    t_ad[i] = lds0 + ((t_rd ^ ((i & 3) << 5) ^ ((i >> 2) << 4)) + (i >> 2) * 8 * kRow);
    asm volatile("" : "+v"(k_ad[i]), "+v"(t_ad[i]));
  }


  // One tile.  MASKED: the tile straddles the diagonal or the end of the prefix, compare and select per element.
  auto tile = [&](auto stage, int key0, auto masked) __attribute__((always_inline)) {  // stage: an int or a constant
    constexpr bool kMasked = decltype(masked)::value;
    const uint32_t so = (uint32_t)stage * kStageBytes;
    f32x16 sacc[2], dpacc[2];
    elemx8 kf[2], vf[2];
    elemx4 ct[kFrags][2];
    auto load_k = [&](int s, int buf) { kf[buf] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(k_ad[s] + so)); };
    auto load_v = [&](int s, int buf) { vf[buf] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(k_ad[s] + so + kTile)); };
    auto load_t = [&](int n, int buf) {  // n = 4 t + db: keys 16 t .. 16 t + 15, d block db
      ct[buf][0] = lds_read_tr(lds_ptr(t_ad[n & 3] + so + 16 * (n >> 2) * kRow));
      ct[buf][1] = lds_read_tr(lds_ptr(t_ad[4 + (n & 3)] + so + 16 * (n >> 2) * kRow));
    };
    // ---- step 1: S^T = K Q^T
    load_k(0, 0);
    load_k(1, 1);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      fence();
      if (s == 0) {
        mfma32_va0(sacc[0], kf[0], qf[0][0]);
        mfma32_va0(sacc[1], kf[0], qf[1][0]);
      } else {
        mfma32_va(sacc[0], kf[s & 1], qf[0][s]);
        mfma32_va(sacc[1], kf[s & 1], qf[1][s]);
      }
      fence();
      if (s + 2 < 8) load_k(s + 2, s & 1);
      if (s >= 6) load_v(s - 6, s - 6);  // the first operands of step 2
    }
    // ---- step 2: dP^T = V dO^T; beside the MFMAs, P = exp2(S c - lse2) of two elements per MFMA
    auto p_elem = [&](int m, int r) {
      float p = fast_exp2(__builtin_fmaf(sacc[m][r], c, -lse2[m]));
      if constexpr (kMasked) {
        if (key0 + acc_row(r, g) > lim[m]) p = 0.f;
      }
      sacc[m][r] = p;
    };
    auto ds_elem = [&](int m, int r) { dpacc[m][r] = sacc[m][r] * dpacc[m][r]; };  // dP accumulated on top of -delta
    elemx8 dsf[2][2];
    auto ds_cvt = [&](int m, int t) {
      const int r0 = 8 * t;
      dsf[m][t] = cvt8(dpacc[m][r0], dpacc[m][r0 + 1], dpacc[m][r0 + 2], dpacc[m][r0 + 3], dpacc[m][r0 + 4], dpacc[m][r0 + 5],
                       dpacc[m][r0 + 6], dpacc[m][r0 + 7]);
    };
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      fence();
      if (s == 0) mfma32_vc(dpacc[0], vf[0], dof[0][0], ndl[0]);
      else mfma32_v(dpacc[0], vf[s & 1], dof[0][s]);
      fence();
      p_elem(0, 2 * s);
      p_elem(0, 2 * s + 1);
      fence();
      if (s == 0) mfma32_vc(dpacc[1], vf[0], dof[1][0], ndl[1]);
      else mfma32_v(dpacc[1], vf[s & 1], dof[1][s]);
      fence();
      p_elem(1, 2 * s);
      p_elem(1, 2 * s + 1);
      if (s + 2 < 8) load_v(s + 2, s & 1);
      if (s >= 8 - kFrags) load_t(s - (8 - kFrags), s - (8 - kFrags));  // the first operands of step 3
    }
    fence();
    // dS of the first 16 keys of sub-block 0: dP is complete only now
#pragma unroll
    for (int r = 0; r < 8; ++r) ds_elem(0, r);
    ds_cvt(0, 0);
    // ---- step 3: dQ^T += K^T dS^T.  Sub-block 0 leads by kLead fragments: dS of sub-block 1's first 16 keys stands
    // behind its first MFMAs, dS of the other 16 keys of both behind the MFMAs that follow
    static_assert(kLead == 2 && kFrags == 4, "the portions below are laid out for a lead of two fragments");
#pragma unroll
    for (int n = 0; n < kLead; ++n) {
      const elemx8 kt = cat4(ct[n % kFrags][0], ct[n % kFrags][1]);
      fence();
      dqacc[0][n & 3] = mfma32(kt, dsf[0][0], dqacc[0][n & 3]);
      fence();
#pragma unroll
      for (int r = 4 * n; r < 4 * n + 4; ++r) ds_elem(1, r);
    }
    ds_cvt(1, 0);
#pragma unroll
    for (int n = 0; n < 8; ++n) {
      const elemx8 kt1 = cat4(ct[n % kFrags][0], ct[n % kFrags][1]);
      fence();
      dqacc[1][n & 3] = mfma32(kt1, dsf[1][n >> 2], dqacc[1][n & 3]);
      fence();
      if (n + kFrags < 8) load_t(n + kFrags, n % kFrags);
      if (n == 0) {
#pragma unroll
        for (int r = 8; r < 12; ++r) ds_elem(0, r);
      }
      if (n == 1) {
#pragma unroll
        for (int r = 12; r < 16; ++r) ds_elem(0, r);
        ds_cvt(0, 1);
      }
      if (n == 2) {
#pragma unroll
        for (int r = 8; r < 12; ++r) ds_elem(1, r);
      }
      if (n == 3) {
#pragma unroll
        for (int r = 12; r < 16; ++r) ds_elem(1, r);
        ds_cvt(1, 1);
      }
      if (n + kLead < 8) {
        const int n0 = n + kLead;
        const elemx8 kt0 = cat4(ct[n0 % kFrags][0], ct[n0 % kFrags][1]);
        fence();
        dqacc[0][n0 & 3] = mfma32(kt0, dsf[0][n0 >> 2], dqacc[0][n0 & 3]);
        fence();
      }
    }
  };

  // Tiles are walked from key 0 up, so the first key of a tile only grows: first come tiles that every row of the
  // wave sees whole (no masking), then tiles on the diagonal or at the end of the prefix (masked), then, for waves
  // whose rows end below those of the block's last wave, tiles that none of their rows sees.  Each kind has a loop
  // of its own with one body; every wave passes the same barriers and makes the same requests in all of them.
  auto advance = [&](int p) {
    wait_vm<kLoadsPerTile>();
    fence();
    asm volatile("s_barrier" ::: "memory");
    fence();
    issue_tile((p + 2) % kStages, p + 2);
  };
  int p = 0;
  // four unmasked tiles per round, one per ring stage, as long as the fourth is still unmasked
  for (; p + 3 < ntiles; p += 4) {
    if (!wave_live || (p + 3) * kKeys + kKeys - 1 > lim_first) break;
    advance(p);
    tile(std::integral_constant<int, 0>{}, p * kKeys, std::false_type{});
    advance(p + 1);
    tile(std::integral_constant<int, 1>{}, (p + 1) * kKeys, std::false_type{});
    advance(p + 2);
    tile(std::integral_constant<int, 2>{}, (p + 2) * kKeys, std::false_type{});
    advance(p + 3);
    tile(std::integral_constant<int, 3>{}, (p + 3) * kKeys, std::false_type{});
  }
  for (; p < ntiles; ++p) {
    if (!wave_live || p * kKeys + kKeys - 1 > lim_first) break;
    advance(p);
    tile(p % kStages, p * kKeys, std::false_type{});
  }
  for (; p < ntiles; ++p) {
    if (!wave_live || p * kKeys > lim_last) break;
    advance(p);
    tile(p % kStages, p * kKeys, std::true_type{});
  }
  for (; p < ntiles; ++p) advance(p);
  wait_vm<0>();  // nothing may still be on its way into LDS when the workgroup ends

  // MERGE: the next block's first rows are requested now and arrive while this block's results are stored; the dQ rows
  // then leave through the wave's stage of the ring, which every wave has left (the barrier), instead of through the
  // rows' place.
  if constexpr (MERGE) {
    requested = mblk + 1 < mb_end;
    __syncthreads();
    if (requested) request_rows(mblk + 1, 0);
  }

  // ---- epilogue: the row statistics for the dK/dV kernel, which runs after this one (stored here rather than where
  // they are made: the wait that precedes the tile loop would have to see the stores through as well), and the dQ rows.
  // A lane holds half of each of its two rows in pieces of 8 bytes (registers 4*cq..+3 of block db hold d0..d0+3):
  // stored from there, an instruction touched 32 rows.  The pieces go to the wave's 16 KB behind the ring instead, in
  // the tiles' swizzled row layout, and leave from there four whole rows per instruction.
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    if (valid[m] && g == 0) {
      const int hg = row[m] - tok[m] * G;
      const int64_t so = (int64_t)(kvh * G + hg) * a.total_q + q0 + tok[m];
      a.lse2_w[so] = lse2[m];
      a.dscaled_w[so] = ndl[m][0];  // -delta: the start value of the dP accumulators in the dK/dV kernel
    }
  }
  {
    const uint32_t out_b = MERGE ? lds0 + wave * kStageBytes : stg;
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int cq = 0; cq < 4; ++cq) {
          const int chunk = 2 * db + 8 * (cq >> 1) + (cq & 1);  // d0 / 8 with d0 = 16 db + 64 (cq >> 1) + 8 (cq & 1) + 4 g
          *static_cast<DISTCA_LDS elemx4 *>(const_cast<DISTCA_LDS void *>(lds_ptr(out_b + (32 * m + l32) * kRow + ((chunk ^ tile_swz(l32)) << 4) + 8 * g))) =
              cvt4(dqacc[m][db][4 * cq] * a.scale, dqacc[m][db][4 * cq + 1] * a.scale, dqacc[m][db][4 * cq + 2] * a.scale,
                   dqacc[m][db][4 * cq + 3] * a.scale);
        }
    // (LDS operations of one wave complete in order: the reads below see the writes above)
    uint8_t *dq_blk = reinterpret_cast<uint8_t *>(a.dq) + dq_task + (int64_t)kvh * G * kHeadDim * 2;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int r = 4 * i + (lane >> 4);
      const int rg = wrow0 + r;
      const elemx8 v = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(out_b + r * kRow + ((lane & 15) << 4)));
      if (rg < nrows) {
        const int t = div_group(rg);
        *reinterpret_cast<elemx8 *>(dq_blk + (int64_t)t * a.dq_tok_bytes + (rg - t * G) * (kHeadDim * 2) + (((lane & 15) ^ tile_swz(r)) << 4)) = v;
      }
    }
  }
  if constexpr (MERGE) {
    if (++mblk < mb_end) {
      __syncthreads();  // every wave has left the ring's stages before the next block's first tiles are requested
      goto next_block;
    }
  }
}

}  // namespace

int DISTCA_FN(launch_dq64)(const BwdArgs &a, int64_t grid, hipStream_t stream) {
  if (device_setup_pending(kSlotBwdDq64)) {
    const void *kernels[] = {(const void *)ca_bwd_dq64_kernel<false, false>, (const void *)ca_bwd_dq64_kernel<true, false>,
                             (const void *)ca_bwd_dq64_kernel<false, true>, (const void *)ca_bwd_dq64_kernel<true, true>};
    for (const void *kf : kernels) {
      hipError_t e = hipFuncSetAttribute(kf, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
      if (e != hipSuccess) return fail(DISTCA_E_LAUNCH, "ca_bwd: cannot reserve %d B of LDS: %s", kLds, hipGetErrorString(e));
    }
    device_setup_done(kSlotBwdDq64);
  }
  const dim3 g((unsigned)grid), b(kThreads);
  const bool seg = a.shards.num_shards > 0, merge = a.merge_tiles > 0;
  if (seg && merge) hipLaunchKernelGGL((ca_bwd_dq64_kernel<true, true>), g, b, kLds, stream, a);
  else if (seg) hipLaunchKernelGGL((ca_bwd_dq64_kernel<true, false>), g, b, kLds, stream, a);
  else if (merge) hipLaunchKernelGGL((ca_bwd_dq64_kernel<false, true>), g, b, kLds, stream, a);
  else hipLaunchKernelGGL((ca_bwd_dq64_kernel<false, false>), g, b, kLds, stream, a);
  return DISTCA_OK;
}

}  // namespace distca
