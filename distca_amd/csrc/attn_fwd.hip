// Varlen causal flash-attention forward for gfx950 (wave64, bf16 MFMA 32x32x16).
//
// Stands where the reference calls flash-attn's varlen forward
// (distca/runtime/megatron/ops/fused_comm_attn.py:151-197).
//
// Work decomposition.  The G = Hq/Hkv query heads that share a kv head are flattened with
// the tokens into one row axis: row R of a task = (token R / G, head R % G), so one K/V
// tile in LDS serves all heads of its group.  A workgroup (8 waves) owns kRows consecutive
// flattened rows of one task and one kv head and streams that task's visible KV prefix in
// tiles of 64 keys; tiles entirely above the diagonal are never visited and only tiles
// that straddle it are masked.  With 8 waves a workgroup covers 256 rows per K/V tile it pulls
// through the vector memory unit, whose throughput (about 64 bytes per clock per compute unit)
// is what a 128-row workgroup ran into.
//
// Per wave: MSUB sub-tiles of 32 rows.  Scores are produced transposed, S^T = K Q^T, so a
// lane holds one query row (column lane%32) and 16 keys per 32x32 block: the online-softmax
// row reductions are in-register plus one lane-pair exchange, and the fp32 accumulator
// registers are, after conversion to bf16, already laid out as the B operand of
// O^T += V^T P^T.  Q stays in registers for the whole KV loop; K is read from LDS row-major
// (16-byte reads), V through the transposing LDS read.
//
// K/V tiles go from global memory straight into LDS (LDS-direct loads, four 256-byte rows per
// instruction, rows unpadded with swizzled 16-byte chunks, see tile_swz), one period ahead of
// their use.
#include <type_traits>
#include <mutex>

#include "api_util.h"
#include "attn_bwd.h"
#include "attn_cfg.h"
#include "common.h"
#include "kv_shards.h"

namespace distca {
namespace {

constexpr int kRowB = 256;    // bytes per K or V row in LDS (unpadded; chunk c of row r sits at c ^ tile_swz(r))
constexpr int kKTile = kFwdKV * kRowB;
constexpr int kVTile = kFwdKV * kRowB;
constexpr int kKOff = 0, kVOff = 2 * kKTile;  // two K stages, then two V stages
constexpr int kFwdLds = 2 * kKTile + 2 * kVTile;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

struct FwdArgs {
  const elem_t *q, *k, *v;
  elem_t *out;
  float *lse;
  const int32_t *cu_q, *cu_k, *kv_off;
  const int32_t *sched;  // schedule workspace
  const void *zero_row;  // 256 zero bytes: source of tile rows past the end of the prefix
  int32_t sched_items_off;  // int32 offset of the item array
  int32_t hq, hkv, group, total_q;
  int32_t causal;
  float scale;
  // Where the query and output tokens live.  Token t of task b starts at base + off[b] + t * tok_bytes
  // (off == nullptr: the packed tensor, off[b] = cu_q[b] * tok_bytes); head h at + h * 256 bytes.
  int32_t *tickets;  // one counter per kv head (sched.h)
  const int64_t *q_task_off, *out_task_off;
  int64_t q_tok_bytes, out_tok_bytes;
  int32_t merge_tiles;   // MERGE kernels: the list's merge_tiles (sched.h)
  int32_t lse_in_token;  // 1: lse of (token, head) as fp32 at token + hq * 256 + h * 4 (the [out | lse] reply), 0: lse[h][token]
  KvShards shards;       // SEG kernels: k and v are the bases of a buffer that holds the stored rows shard by shard
};

// SEG: K/V rows are addressed through a table of shards (kv_shards.h) instead of as one dense tensor.
// MERGE: a work item is several consecutive blocks of a task's query rows (sched.h, fwd_merge), worked off one after the
// other; otherwise it is one block.
template <int MSUB, bool SEG, bool MERGE>
__global__ __launch_bounds__(kFwdWaves * 64, (MSUB == 1 && kFwdWaves == 4 ? 2 : 1)) void ca_fwd_kernel(FwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int nitems = a.sched[0];
  int item, kvh;
  if (!take_item(a.tickets, nitems, a.hkv, reinterpret_cast<int32_t *>(lds), item, kvh)) return;
  // (the item's fields and the task's bounds are moved to scalar registers as they are read: what derives from them,
  // base pointers, loop limits and tile addresses, is then scalar arithmetic)
  int4 it = reinterpret_cast<const int4 *>(a.sched + a.sched_items_off)[item];
  it.x = uniform_int(it.x);
  it.y = uniform_int(it.y);
  const int task = it.x;

  const int q0 = uniform_int(a.cu_q[task]);
  const int lq = uniform_int(a.cu_q[task + 1]) - q0;
  const int lk = uniform_int(a.cu_k[task + 1]) - uniform_int(a.cu_k[task]);
  const int ks = uniform_int(a.kv_off ? a.kv_off[task] : a.cu_k[task]);
  const int G = a.group;
  const int shift = lk - lq;

  constexpr int kRows = kFwdWaves * 32 * MSUB;
  const int nrows = lq * G;
  // the blocks of this item
  int mb_first = it.y, mb_end = it.y + 1;
  if constexpr (MERGE) {
    SchedGeom geom;
    geom.rows_per_block = kRows; geom.kv_per_block = kFwdKV; geom.group = G; geom.causal = a.causal; geom.merge_tiles = a.merge_tiles;
    const int m = fwd_merge(geom, lq, lk), nblk = (nrows + kRows - 1) / kRows;
    mb_first = it.y * m;
    mb_end = mb_first + m < nblk ? mb_first + m : nblk;
  }
  // (a jump back rather than a loop statement: without MERGE the body below is then straight-line code, exactly the
  // kernel that takes one block per item)
  int mblk = mb_first;
  // MERGE: the Q rows and the first K tile of a block are requested while the block before it finishes (below)
  elemx8 qf[MSUB][8];
  bool requested = false;
next_block:
  // MERGE: the thread index is made opaque once per block, so that what derives from it (the lanes' LDS and global
  // offsets, a few dozen registers) is computed afresh for every block instead of being carried, and partly spilled,
  // across the whole body: a reload from scratch memory waits for every request in flight, those made for the next
  // block included.
  int tid_ = threadIdx.x;
  if constexpr (MERGE) asm volatile("" : "+v"(tid_));
  const int tid = tid_, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int row_wg = mblk * kRows;

  // ---- KV extent of this workgroup
  int tok_end = (row_wg + kRows + G - 1) / G;
  if (tok_end > lq) tok_end = lq;
  int nvis = a.causal ? tok_end + shift : lk;
  if (nvis > lk) nvis = lk;
  const int ntiles = nvis > 0 ? (nvis + kFwdKV - 1) / kFwdKV : 0;

  // ---- per-lane rows
  const uint8_t *qbytes = reinterpret_cast<const uint8_t *>(a.q) + uniform_int64(a.q_task_off ? a.q_task_off[task] : (int64_t)q0 * a.q_tok_bytes);
  uint8_t *obytes = reinterpret_cast<uint8_t *>(a.out) + uniform_int64(a.out_task_off ? a.out_task_off[task] : (int64_t)q0 * a.out_tok_bytes);
  int row[MSUB], tok[MSUB], lim[MSUB];
  bool valid[MSUB];
  const elem_t *qptr[MSUB];
#pragma unroll
  for (int m = 0; m < MSUB; ++m) {
    row[m] = row_wg + (wave * MSUB + m) * 32 + l32;
    valid[m] = row[m] < nrows;
    tok[m] = row[m] / G;
    const int hg = row[m] - tok[m] * G;
    int lm = a.causal ? tok[m] + shift : lk - 1;
    if (lm > lk - 1) lm = lk - 1;
    lim[m] = lm;
    qptr[m] = reinterpret_cast<const elem_t *>(qbytes + (int64_t)tok[m] * a.q_tok_bytes) + (kvh * G + hg) * kHeadDim;
  }
  // wave-uniform limits: first row's limit decides whether a tile needs masking, last row's
  // whether the wave has anything to do in it.
  const int wrow0 = row_wg + wave * MSUB * 32;
  int wrow1 = wrow0 + MSUB * 32 - 1;
  if (wrow1 > nrows - 1) wrow1 = nrows - 1;
  const bool wave_live = wrow0 < nrows;
  int lim_first = 0x7fffffff, lim_last = -1;
  if (wave_live) {
    lim_first = a.causal ? wrow0 / G + shift : lk - 1;
    if (lim_first > lk - 1) lim_first = lk - 1;
    lim_last = a.causal ? wrow1 / G + shift : lk - 1;
    if (lim_last > lk - 1) lim_last = lk - 1;
  }

  // ---- Q fragments (B operand of S^T = K Q^T): lane holds row l32, d = 16*s + 8*g .. +7
  if (!MERGE || !requested) {
#pragma unroll
    for (int m = 0; m < MSUB; ++m) {
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        if (valid[m]) qf[m][s] = *reinterpret_cast<const elemx8 *>(qptr[m] + 16 * s + 8 * g);
        else qf[m][s] = elemx8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  }

  // ---- K/V tile fetch: wave w brings rows 16w .. 16w+15 of the K tile and of the V tile, four
  // rows per instruction; lane p fetches the chunk that belongs at chunk position p%16 of row p/16
  const int64_t kv_stride = (int64_t)a.hkv * kHeadDim;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(DISTCA_LDS uint8_t *)lds;
  const int uwave = __builtin_amdgcn_readfirstlane(wave);
  const elem_t *kbase = a.k + (SEG ? 0 : (int64_t)ks * kv_stride) + kvh * kHeadDim;
  const elem_t *vbase = a.v + (SEG ? 0 : (int64_t)ks * kv_stride) + kvh * kHeadDim;
  // SEG: the shards that hold the rows of the K tile and of the V tile requested next (the K requests run a tile ahead)
  ShardCursor kcur, vcur;
  if constexpr (SEG) {
    kcur.open(a.shards, a.shards.task_shard[task]);
    vcur = kcur;
  }
  // a wave brings kRowsW rows of a K tile or of a V tile, four rows per instruction
  constexpr int kRowsW = kFwdKV / kFwdWaves, kLdW = kRowsW / 4;
  auto issue_rows = [&](const elem_t *base, int j, uint32_t tile_off, const ShardCursor &cur, int which) {
#pragma unroll
    for (int i = 0; i < kLdW; ++i) {
      const int r = kRowsW * uwave + 4 * i + (lane >> 4);
      const int key = j * kFwdKV + r;
      const int chunk = (lane & 15) ^ tile_swz(r);
      const elem_t *src;
      if constexpr (SEG) {
        src = reinterpret_cast<const elem_t *>(reinterpret_cast<const uint8_t *>(base) +
                                               (key < lk ? shard_row_offset(a.shards, cur, ks + key, which, kv_stride * 2) : 0));
      } else {
        src = base + (int64_t)key * kv_stride;
      }
      if (key >= lk) src = reinterpret_cast<const elem_t *>(a.zero_row);
      lds_direct_load16_ptr(src + chunk * 8, lds0 + tile_off + (kRowsW * uwave + 4 * i) * kRowB);
    }
  };
  // Tiles that lie wholly inside the prefix (all but the last one; SEG: and inside one shard) take a form without
  // per-lane address arithmetic: a scalar base that advances by one tile, plus a per-lane offset that never changes.
  uint32_t voff[kLdW];
#pragma unroll
  for (int i = 0; i < kLdW; ++i) {
    const int r = kRowsW * uwave + 4 * i + (lane >> 4);
    voff[i] = (uint32_t)((r * kv_stride + (((lane & 15) ^ tile_swz(r)) * 8)) * 2);
  }
  auto issue_rows_fast = [&](const elem_t *tb, uint32_t tile_off) {
#pragma unroll
    for (int i = 0; i < kLdW; ++i) lds_direct_load16(tb, voff[i], lds0 + tile_off + (kRowsW * uwave + 4 * i) * kRowB);
  };
  // Key j * kFwdKV + r of a tile that ends at or before key `lim` lies at virt + (j * kFwdKV + r) * kv_stride.  Without
  // SEG that is the whole prefix but for its last, partial tile; with SEG the tiles inside the present shard: a tile
  // past `lim` looks for its shard (which moves virt and lim on) and only takes the per-lane form when it straddles
  // two shards or the end of the prefix, so that a run of tiles inside one shard costs what it costs without SEG.
  struct Run {
    const elem_t *virt;
    int lim;
  };
  Run krun{kbase, SEG ? 0 : lk}, vrun{vbase, SEG ? 0 : lk};
  auto issue_kv = [&](const elem_t *base, int j, uint32_t tile_off, Run &run, ShardCursor &cur, int which) __attribute__((always_inline)) {
    if ((j + 1) * kFwdKV <= run.lim) {
      issue_rows_fast(run.virt + (int64_t)j * kFwdKV * kv_stride, tile_off);
      return;
    }
    if constexpr (SEG) {
      const int r0 = ks + j * kFwdKV;
      cur.seek(a.shards, r0);
      if ((j + 1) * kFwdKV <= lk && cur.holds(r0, kFwdKV)) {
        run.virt = reinterpret_cast<const elem_t *>(static_cast<uintptr_t>(uniform_i64(
            (int64_t)reinterpret_cast<uintptr_t>(base) + (which ? cur.v : cur.k) - (int64_t)(cur.lo - ks) * kv_stride * 2)));
        run.lim = uniform_i32(cur.hi - ks < lk ? cur.hi - ks : lk);
        issue_rows_fast(run.virt + (int64_t)j * kFwdKV * kv_stride, tile_off);
        return;
      }
    }
    issue_rows(base, j, tile_off, cur, which);
  };
  auto issue_k = [&](int j) __attribute__((always_inline)) { issue_kv(kbase, j, kKOff + (j & 1) * kKTile, krun, kcur, 0); };
  auto issue_v = [&](int j) __attribute__((always_inline)) { issue_kv(vbase, j, kVOff + (j & 1) * kVTile, vrun, vcur, 1); };

  // ---- accumulators
  f32x16 oacc[MSUB][4];
  float m_run[MSUB], l_run[MSUB];
#pragma unroll
  for (int m = 0; m < MSUB; ++m) {
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[m][db][r] = 0.f;
    m_run[m] = -INFINITY;
    l_run[m] = 0.f;
  }
  const float c = a.scale * kLog2e;
  constexpr float kLazy = 8.f, kRedo = 32.f * 256.f;

  // LDS read offsets (bytes) that do not depend on the tile
  const int k_rd = l32 * kRowB + ((g ^ tile_swz(l32)) << 4);  // + kb*32*kRowB, ^ 32*s
  // transposed V operand: lane points at (key 4g + i4 [+8 hi +16 t], chunk 8 b4 + h1 [+2 db], half lane&1);
  // tile_swz of that row is (i4<<1) | (g<<3) | hi
  const int i4 = (lane & 15) >> 2, b4 = (lane >> 4) & 1, h1 = (lane & 3) >> 1;
  const int v_rd = (4 * g + i4) * kRowB + ((((b4 ^ g) << 3) | (i4 << 1) | h1) << 4) + 8 * (lane & 1);  // ^ 32*db ^ 16*hi

  // Absolute LDS addresses of this lane's operand reads in stage 0, the eight swizzled variants of each,
  // kept in registers: with the stage and the row block in the instruction's offset field, no address
  // arithmetic is left between the MFMAs.
  uint32_t k_ad[8], v_ad[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    k_ad[i] = lds0 + kKOff + (k_rd ^ (i << 5));
    v_ad[i] = lds0 + kVOff + (v_rd ^ ((i & 3) << 5) ^ ((i >> 2) << 4));
    asm volatile("" : "+v"(k_ad[i]), "+v"(v_ad[i]));
  }
  f32x16 sacc[MSUB][2];
  elemx8 pf[MSUB][4];
  auto tile_active = [&](int j) { return wave_live && j * kFwdKV <= lim_last; };

  // ---- S^T = K Q^T : [64 keys] x [32*MSUB rows]
  auto phase_s = [&](int j, auto par) __attribute__((always_inline)) {  // par: parity of j, known at compile time
#pragma unroll
    for (int m = 0; m < MSUB; ++m)
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[m][kb][r] = 0.f;
    constexpr int kPf = 2;  // K fragments are requested kPf steps before the MFMAs that use them
    elemx8 kf[kPf][2];
    auto load_k = [&](int s, int buf) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) kf[buf][kb] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(k_ad[s] + decltype(par)::value * kKTile + kb * 32 * kRowB));
    };
#pragma unroll
    for (int s = 0; s < kPf; ++s) load_k(s, s);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int m = 0; m < MSUB; ++m) sacc[m][kb] = mfma32(kf[s % kPf][kb], qf[m][s], sacc[m][kb]);
      __builtin_amdgcn_sched_barrier(0);
      if (s + kPf < 8) load_k(s + kPf, s % kPf);
    }
  };
  // ---- mask, online softmax (log2 domain, one query row per lane pair), P as bf16 B operand
  auto phase_x = [&](int j) __attribute__((always_inline)) {
    const int key0 = j * kFwdKV;
    if (key0 + kFwdKV - 1 > lim_first) {  // the tile straddles the diagonal or the end of the prefix
#pragma unroll
      for (int m = 0; m < MSUB; ++m)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const int key = key0 + kb * 32 + acc_row(r, g);
            if (key > lim[m]) sacc[m][kb][r] = -INFINITY;
          }
    }
#pragma unroll
    for (int m = 0; m < MSUB; ++m) {
      // P = 2^(S c + mc) as bf16 B operand; returns this lane's share of the row sums
      auto exp_tile = [&](float mc) __attribute__((always_inline)) {
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int kb = t >> 1, r0 = 8 * (t & 1);
          float e[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            e[i] = fast_exp2(__builtin_fmaf(sacc[m][kb][r0 + i], c, mc));
            sum += e[i];
          }
          pf[m][t] = cvt8(e[0], e[1], e[2], e[3], e[4], e[5], e[6], e[7]);
        }
        return sum;
      };
      // The running reference m_run of a row need not be its maximum: any value within 2^kLazy of
      // it gives the same O / l.  So first try the tile against the old reference, without looking
      // for the maximum at all; only when a lane's 32 exponentials add up to more than 32 * 2^kLazy
      // (or the row has no reference yet) is the maximum taken, the row rescaled if it moved by
      // more than 2^kLazy, and the tile done again.
      bool exact = __any(m_run[m] == -INFINITY);
      float sum = 0.f;
      if (!exact) {
        sum = exp_tile(-m_run[m] * c);
        exact = __any(sum > kRedo);
      }
      if (exact) {
        float mx = sacc[m][0][0];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) mx = __builtin_fmaxf(mx, sacc[m][kb][r]);
        mx = pair_max(mx);
        const float m_new = __builtin_fmaxf(m_run[m], mx);
        if (__any((m_new - m_run[m]) * c > kLazy)) {
          const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
          const float alpha = fast_exp2((m_run[m] - m_use) * c);
          l_run[m] *= alpha;
#pragma unroll
          for (int db = 0; db < 4; ++db)
#pragma unroll
            for (int r = 0; r < 16; ++r) oacc[m][db][r] *= alpha;
          m_run[m] = m_new;
        }
        sum = exp_tile((m_run[m] == -INFINITY) ? 0.f : -m_run[m] * c);
      }
      l_run[m] += sum;
    }
  };
  // ---- O^T += V^T P^T : [128 d] x [32*MSUB rows], contraction over the 64 keys
  auto phase_pv = [&](int j, auto par) __attribute__((always_inline)) {
    constexpr int kPfV = 4;  // V^T fragments are requested four MFMAs ahead
    elemx4 vf[kPfV][2];
    auto load_v = [&](int u, int buf) {  // u = 4*t + db
      const uint32_t vo = decltype(par)::value * kVTile + 16 * (u >> 2) * kRowB;
      vf[buf][0] = lds_read_tr(lds_ptr(v_ad[u & 3] + vo));
      vf[buf][1] = lds_read_tr(lds_ptr(v_ad[4 + (u & 3)] + vo + 8 * kRowB));
    };
#pragma unroll
    for (int u = 0; u < kPfV; ++u) load_v(u, u);
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int m = 0; m < MSUB; ++m) oacc[m][u & 3] = mfma32(cat4(vf[u % kPfV][0], vf[u % kPfV][1]), pf[m][u >> 2], oacc[m][u & 3]);
      __builtin_amdgcn_sched_barrier(0);
      if (u + kPfV < 16) load_v(u + kPfV, u % kPfV);
    }
  };

  // The waves form two groups (0-3, 4-7; a SIMD holds one wave of each) that run half a period
  // apart, so that one group's MFMA phases coincide with the other's softmax arithmetic instead
  // of both queueing for the same pipe.  Between consecutive workgroup barriers b0, b1, b2, ...
  //   [b(2p),   b(2p+1)):  group 0: PV(p-1), S(p)     group 1: softmax(p-1)
  //   [b(2p+1), b(2p+2)):  group 0: softmax(p)        group 1: PV(p-1), S(p)
  // Tile p of K is read between b(2p) and b(2p+2), tile p of V between b(2p+2) and b(2p+4); every
  // wave requests K(p+1) and V(p) at the start of its softmax half of period p (group 1 right after
  // b(2p), group 0 right after b(2p+1)), into the stages whose last readers finished before b(2p), and
  // waits for its own requests before b(2p+2).  The MFMA halves are the critical path of a period (one
  // group's, then the other's); a request holds its wave for a hundred cycles or so, and in front of
  // group 0's MFMA half that time showed in the period (-3 % with the requests behind it).
  // MERGE: what the item's next block starts with is requested when this block's tile loop is over, so that it
  // arrives while the results are normalised and stored: its Q rows (the Q registers are free: every S of this block
  // is done) and its first K tile (no wave reads a K stage any more: the last barrier of the loop lies behind every S
  // phase; tile 0 is the same for every block of a task).  The run and cursor objects the request goes through are
  // set up afresh by the next block, which also finds its tile 0 request made.  (Made from inside the loop's last
  // period instead, the requests cost the loop its register allocation: six hundred spills.)
  const bool more = MERGE && mblk + 1 < mb_end;
  auto request_next_block = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < MSUB; ++m) {
      const int nrow = row[m] + kRows;
      const int ntok = nrow / G;
      const elem_t *np = reinterpret_cast<const elem_t *>(qbytes + (int64_t)ntok * a.q_tok_bytes) + (kvh * G + (nrow - ntok * G)) * kHeadDim;
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        if (nrow < nrows) qf[m][s] = *reinterpret_cast<const elemx8 *>(np + 16 * s + 8 * g);
        else qf[m][s] = elemx8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
    krun = Run{kbase, SEG ? 0 : lk};
    if constexpr (SEG) kcur.open(a.shards, a.shards.task_shard[task]);
    issue_k(0);  // (the next block has rows, hence at least one tile)
  };
  const int grp = uwave >> 2;
  if (ntiles > 0 && (!MERGE || !requested)) issue_k(0);
  wait_vm0();
  __syncthreads();  // b0
  // The period loop is unrolled by two so that the LDS stage of every operand read is a constant folded into
  // the instruction's offset field instead of an addition per read between the MFMAs.
  using P0 = std::integral_constant<int, 0>;
  using P1 = std::integral_constant<int, 1>;
  auto period0 = [&](int p, auto par) __attribute__((always_inline)) {   // par = parity of p
    using Same = std::integral_constant<int, decltype(par)::value>;
    using Other = std::integral_constant<int, 1 - decltype(par)::value>;
    if (p > 0 && tile_active(p - 1)) phase_pv(p - 1, Other{});
    const bool act = p < ntiles && tile_active(p);
    if (act) phase_s(p, Same{});
    __syncthreads();
    if (p + 1 < ntiles) issue_k(p + 1);
    if (p < ntiles) issue_v(p);
    if (act) phase_x(p);
    wait_vm0();
    __syncthreads();
  };
  auto period1 = [&](int p, auto par) __attribute__((always_inline)) {
    using Same = std::integral_constant<int, decltype(par)::value>;
    using Other = std::integral_constant<int, 1 - decltype(par)::value>;
    if (p + 1 < ntiles) issue_k(p + 1);
    if (p < ntiles) issue_v(p);
    const bool act_prev = p > 0 && tile_active(p - 1);
    if (act_prev) phase_x(p - 1);
    __syncthreads();
    if (act_prev) phase_pv(p - 1, Other{});
    if (p < ntiles && tile_active(p)) phase_s(p, Same{});
    wait_vm0();
    __syncthreads();
  };
  if (grp == 0) {
    for (int p = 0; p <= ntiles; p += 2) {
      period0(p, P0{});
      if (p + 1 <= ntiles) period0(p + 1, P1{});
    }
  } else {
    for (int p = 0; p <= ntiles; p += 2) {
      period1(p, P0{});
      if (p + 1 <= ntiles) period1(p + 1, P1{});
    }
  }

  // (Where the results go is worked out ahead of those requests: should the compiler have parked a pointer in scratch
  // memory, fetching it back afterwards would wait for the requests as well.)
  uint8_t *otok_m[MSUB];
#pragma unroll
  for (int m = 0; m < MSUB; ++m) {
    otok_m[m] = obytes + (int64_t)tok[m] * a.out_tok_bytes;
    if constexpr (MERGE) asm volatile("" : "+v"(otok_m[m]));
  }
  if constexpr (MERGE) {
    requested = more;
    if (more) request_next_block();
  }

  // ---- epilogue: normalise, write O (bf16) and LSE (fp32, natural log)
#pragma unroll
  for (int m = 0; m < MSUB; ++m) {
    const float l_tot = pair_sum(l_run[m]);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (valid[m]) {
      const int hg = row[m] - tok[m] * G;
      uint8_t *otok = otok_m[m];
      elem_t *op = reinterpret_cast<elem_t *>(otok) + (kvh * G + hg) * kHeadDim;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int cq = 0; cq < 4; ++cq) {
          // registers 4*cq .. 4*cq+3 of block db hold d0 .. d0+3
          const int d0 = 16 * db + 64 * (cq >> 1) + 8 * (cq & 1) + 4 * g;
          const elemx4 o4 = cvt4(oacc[m][db][4 * cq] * inv, oacc[m][db][4 * cq + 1] * inv, oacc[m][db][4 * cq + 2] * inv,
                                 oacc[m][db][4 * cq + 3] * inv);
          *reinterpret_cast<elemx4 *>(op + d0) = o4;
        }
      if (g == 0) {
        const float lse = l_tot > 0.f ? (m_run[m] * c + fast_log2(l_tot)) * kLn2 : -INFINITY;
        const int head = kvh * G + hg;
        if (a.lse_in_token) {
          float *lp = reinterpret_cast<float *>(otok + (int64_t)a.hq * kHeadDim * 2);
          lp[head] = lse;
          if (head == a.hq - 1) {  // zero the padding that rounds the token up to 16 bytes
            for (int64_t b = (int64_t)a.hq * (kHeadDim * 2 + 4); b < (((int64_t)a.hq * (kHeadDim * 2 + 4) + 15) & ~(int64_t)15); b += 4) *reinterpret_cast<float *>(otok + b) = 0.f;
          }
        } else {
          a.lse[(int64_t)head * a.total_q + q0 + tok[m]] = lse;
        }
      }
    }
  }
  if constexpr (MERGE) {
    if (++mblk < mb_end) goto next_block;
  }
}

}  // namespace
}  // namespace distca

using namespace distca;

#ifndef DISTCA_F16
// Scratch memory of distca_ca_fwd_noalloc: the forward's work list, zero row and ticket counters, which every other
// entry point takes from the caller's workspace.  One copy per GPU, held until the process ends.  The name below is
// a host-side stand-in, never a device address: host code uses the per-device address from hipGetSymbolAddress.
constexpr int64_t kNoAllocScratchBytes = 1 << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {
// Device address of `scratch` on the current device, resolved once per device with that device current.
int noalloc_scratch(void **out) {
  static std::mutex mu;
  static void *ptr[64] = {nullptr};
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(DISTCA_E_LAUNCH, "ca_fwd_noalloc: hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= 64) return fail(DISTCA_E_UNSUPPORTED, "ca_fwd_noalloc: device id %d (at most 64 devices)", dev);
  std::lock_guard<std::mutex> lock(mu);
  if (!ptr[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail(DISTCA_E_LAUNCH, "ca_fwd_noalloc: hipGetSymbolAddress: %s", hipGetErrorString(e));
    ptr[dev] = p;
  }
  *out = ptr[dev];
  return DISTCA_OK;
}
}  // namespace

extern "C" int64_t distca_ca_fwd_noalloc_max_bytes(void) { return kNoAllocScratchBytes; }

extern "C" int64_t distca_ca_fwd_workspace_bytes(const distca_ca_params *p) {
  if (!p) return fail(DISTCA_E_INVALID, "fwd_workspace_bytes: null params");
  int rc = validate_params(p);
  if (rc) return rc;
  return sched_region_bytes(p->num_tasks, fwd_max_items(p));
}

extern "C" int distca_ca_fwd_tokens(const void *q_base, const int64_t *q_task_off, int64_t q_tok_bytes, const void *k,
                                    const void *v, void *out_base, const int64_t *out_task_off, int64_t out_tok_bytes,
                                    float *lse, const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off,
                                    const distca_ca_params *p, void *workspace, int64_t workspace_bytes, void *stream) {
  if (!p) return fail(DISTCA_E_INVALID, "ca_fwd: null params");
  return (p->dtype == DISTCA_DTYPE_F16 ? run_fwd_tokens_f16 : run_fwd_tokens)(q_base, q_task_off, q_tok_bytes, k, v, nullptr, out_base,
                                                                              out_task_off, out_tok_bytes, lse, cu_q, cu_k, kv_off, p,
                                                                              workspace, workspace_bytes, stream);
}

extern "C" int distca_ca_fwd_buffers(const void *q_base, const int64_t *q_task_off, int64_t q_tok_bytes, const void *k,
                                     const void *v, const distca_kv_shards *kv_shards, void *out_base, const int64_t *out_task_off,
                                     int64_t out_tok_bytes, float *lse, const int32_t *cu_q, const int32_t *cu_k,
                                     const int32_t *kv_off, const distca_ca_params *p, void *workspace, int64_t workspace_bytes,
                                     void *stream) {
  if (!p) return fail(DISTCA_E_INVALID, "ca_fwd: null params");
  if (!kv_shards) return fail(DISTCA_E_INVALID, "ca_fwd_buffers: null table of K/V shards");
  return (p->dtype == DISTCA_DTYPE_F16 ? run_fwd_tokens_f16 : run_fwd_tokens)(q_base, q_task_off, q_tok_bytes, k, v, kv_shards, out_base,
                                                                              out_task_off, out_tok_bytes, lse, cu_q, cu_k, kv_off, p,
                                                                              workspace, workspace_bytes, stream);
}

namespace distca {
int make_kv_shards(const distca_kv_shards *in, const int32_t *kv_off, bool backward, KvShards *out) {
  if (in->num_shards <= 0) return fail(DISTCA_E_INVALID, "kv_shards: num_shards=%d", in->num_shards);
  if (!in->row_start || !in->k_offset || !in->v_offset || !in->task_shard) return fail(DISTCA_E_INVALID, "kv_shards: null array");
  if (backward && (!in->dk_offset || !in->dv_offset)) return fail(DISTCA_E_INVALID, "kv_shards: the backward needs dk_offset and dv_offset");
  if (!kv_off) return fail(DISTCA_E_INVALID, "kv_shards: kv_task_offsets is required (tasks name stored rows)");
  out->row_start = in->row_start; out->k_off = in->k_offset; out->v_off = in->v_offset;
  out->dk_off = in->dk_offset; out->dv_off = in->dv_offset; out->task_shard = in->task_shard;
  out->num_shards = in->num_shards;
  return DISTCA_OK;
}
}  // namespace distca

extern "C" int distca_ca_fwd(const void *q, const void *k, const void *v, void *out, float *lse, const int32_t *cu_q,
                             const int32_t *cu_k, const int32_t *kv_off, const distca_ca_params *p, void *workspace,
                             int64_t workspace_bytes, void *stream) {
  if (!p) return fail(DISTCA_E_INVALID, "ca_fwd: null params");
  const int rc = validate_params(p);
  if (rc) return rc;
  if (p->num_tasks == 0 || p->total_q == 0) return DISTCA_OK;
  if (!lse) return fail(DISTCA_E_INVALID, "ca_fwd: null pointer");
  return distca_ca_fwd_tokens(q, nullptr, 0, k, v, out, nullptr, 0, lse, cu_q, cu_k, kv_off, p, workspace, workspace_bytes, stream);
}

extern "C" int distca_ca_fwd_noalloc(const void *q, const void *k, const void *v, void *out, float *lse, const int32_t *cu_q,
                                     const int32_t *cu_k, const int32_t *kv_off, const distca_ca_params *p, void *stream) {
  if (!p) return fail(DISTCA_E_INVALID, "ca_fwd_noalloc: null params");
  const int64_t need = distca_ca_fwd_workspace_bytes(p);
  if (need < 0) return (int)need;
  if (need > kNoAllocScratchBytes)
    return fail(DISTCA_E_WORKSPACE,
                "ca_fwd_noalloc: this batch needs %lld B of scratch, the static array holds %lld B (about %lld work items: "
                "query rows x heads per kv head / %d + tasks); use distca_ca_fwd with a workspace",
                (long long)need, (long long)kNoAllocScratchBytes, (long long)(kNoAllocScratchBytes / 16), kFwdRows);
  void *ws = nullptr;
  const int rc = noalloc_scratch(&ws);
  if (rc) return rc;
  return distca_ca_fwd(q, k, v, out, lse, cu_q, cu_k, kv_off, p, ws, kNoAllocScratchBytes, stream);
}

#endif  // !DISTCA_F16

namespace distca {
int DISTCA_FN(run_fwd_tokens)(const void *q_base, const int64_t *q_task_off, int64_t q_tok_bytes, const void *k, const void *v,
                              const distca_kv_shards *kv_shards, void *out_base, const int64_t *out_task_off, int64_t out_tok_bytes,
                              float *lse, const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off, const distca_ca_params *p,
                              void *workspace, int64_t workspace_bytes, void *stream) {
  const void *q = q_base;
  void *out = out_base;
  if (!p) return fail(DISTCA_E_INVALID, "ca_fwd: null params");
  int rc = validate_params(p);
  if (rc) return rc;
  if (p->num_tasks == 0 || p->total_q == 0) return DISTCA_OK;
  if (!q || !k || !v || !out || !cu_q || !cu_k) return fail(DISTCA_E_INVALID, "ca_fwd: null pointer");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out)) return fail(DISTCA_E_INVALID, "ca_fwd: q/k/v/out must be 16-byte aligned");
  if (!lse && !out_task_off) return fail(DISTCA_E_INVALID, "ca_fwd: lse is null and the output is not in token layout");
  const int64_t row_bytes = (int64_t)p->num_heads_q * kHeadDim * 2;
  if (!q_task_off) q_tok_bytes = row_bytes;
  if (!out_task_off) out_tok_bytes = row_bytes;
  if (q_tok_bytes < row_bytes || (q_tok_bytes & 15)) return fail(DISTCA_E_INVALID, "ca_fwd: query token of %lld B (needs >= %lld, multiple of 16)", (long long)q_tok_bytes, (long long)row_bytes);
  const int64_t out_need = row_bytes + (lse ? 0 : (int64_t)p->num_heads_q * 4);
  if (out_tok_bytes < out_need || (out_tok_bytes & 15)) return fail(DISTCA_E_INVALID, "ca_fwd: output token of %lld B (needs >= %lld, multiple of 16)", (long long)out_tok_bytes, (long long)out_need);
  const int64_t need = distca_ca_fwd_workspace_bytes(p);
  if (!workspace || workspace_bytes < need) return fail(DISTCA_E_WORKSPACE, "ca_fwd: workspace %lld B < required %lld B", (long long)workspace_bytes, (long long)need);
  if (!aligned16(workspace)) return fail(DISTCA_E_INVALID, "ca_fwd: workspace must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const SchedGeom geom = fwd_geom(p);
  const int64_t max_items = fwd_max_items(p);
  rc = launch_build_schedule(0, cu_q, cu_k, p->num_tasks, geom, (int32_t *)workspace, max_items, s);
  if (rc) return rc;

  FwdArgs a;
  a.q = (const elem_t *)q; a.k = (const elem_t *)k; a.v = (const elem_t *)v;
  a.out = (elem_t *)out; a.lse = lse;
  a.cu_q = cu_q; a.cu_k = cu_k; a.kv_off = kv_off;
  a.sched = (const int32_t *)workspace;
  a.zero_row = (const uint8_t *)workspace + sched_zero_row_off(p->num_tasks, max_items);
  a.sched_items_off = (int32_t)sched_header_ints(p->num_tasks);
  a.tickets = (int32_t *)((uint8_t *)workspace + sched_ticket_off(p->num_tasks, max_items));
  a.hq = p->num_heads_q; a.hkv = p->num_heads_kv; a.group = p->num_heads_q / p->num_heads_kv;
  a.total_q = p->total_q; a.causal = p->causal != 0; a.scale = p->softmax_scale;
  a.q_task_off = q_task_off; a.out_task_off = out_task_off; a.q_tok_bytes = q_tok_bytes; a.out_tok_bytes = out_tok_bytes;
  a.lse_in_token = lse ? 0 : 1;
  a.merge_tiles = geom.merge_tiles;
  a.shards = KvShards{};
  if (kv_shards) {
    rc = make_kv_shards(kv_shards, kv_off, false, &a.shards);
    if (rc) return rc;
  }
  const int64_t grid = max_items * p->num_heads_kv * kSchedOversubNum / kSchedOversubDen;
  if (grid > 0x7fffffff) return fail(DISTCA_E_INVALID, "ca_fwd: grid too large");
  if (device_setup_pending(kSlotFwdLds)) {
    const void *kernels[] = {(const void *)ca_fwd_kernel<kFwdMsub, false, false>, (const void *)ca_fwd_kernel<kFwdMsub, true, false>,
                             (const void *)ca_fwd_kernel<kFwdMsub, false, true>, (const void *)ca_fwd_kernel<kFwdMsub, true, true>};
    for (const void *kf : kernels) {
      hipError_t e = hipFuncSetAttribute(kf, hipFuncAttributeMaxDynamicSharedMemorySize, kFwdLds);
      if (e != hipSuccess) return fail(DISTCA_E_LAUNCH, "ca_fwd: cannot reserve %d B of LDS: %s", kFwdLds, hipGetErrorString(e));
    }
    device_setup_done(kSlotFwdLds);
  }
  {
    ScopedTimer timer(DISTCA_TIMER_CA_FWD, s);
    const dim3 g((unsigned)grid), b(kFwdWaves * 64);
    const bool merge = geom.merge_tiles > 0;
    if (kv_shards && merge) hipLaunchKernelGGL((ca_fwd_kernel<kFwdMsub, true, true>), g, b, kFwdLds, s, a);
    else if (kv_shards) hipLaunchKernelGGL((ca_fwd_kernel<kFwdMsub, true, false>), g, b, kFwdLds, s, a);
    else if (merge) hipLaunchKernelGGL((ca_fwd_kernel<kFwdMsub, false, true>), g, b, kFwdLds, s, a);
    else hipLaunchKernelGGL((ca_fwd_kernel<kFwdMsub, false, false>), g, b, kFwdLds, s, a);
  }
  return check_launch("ca_fwd");
}
}  // namespace distca
