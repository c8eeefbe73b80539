// dK / dV of the varlen causal attention backward for gfx950, 64 keys per wave.
//
// One workgroup of 4 waves per (task, block of 256 keys, kv head), one wave per SIMD, so that a wave may use the
// SIMD's whole register file: the dK^T / dV^T accumulators of its 64 keys (2 key blocks x 4 blocks over d x 2
// matrices x 16 registers) fill the 256 accumulation registers, K of its keys stays in 64 vector registers as MFMA
// B operand, V of the workgroup's keys in LDS (and, as far as registers allow, in registers too: kVRegSlices).  The query side (Q, dO and the row statistics of every head of the
// kv group, flattened into rows) streams through LDS in blocks of 32 rows, by LDS-direct loads into a ring of
// four stages, from the last block down to the first one the causal mask lets see these keys, or from that one up.
//
// With one wave per SIMD nothing else can use the SIMD's vector ALU while the wave waits for the matrix pipe, and
// a wave issues in order: an MFMA that finds the pipe busy holds up everything behind it.  So the arithmetic of a
// block (P = exp2(S c - lse2), dS = P (dP - delta), conversions to bf16) is written between the MFMAs of the same
// block, a few instructions behind each one, where it runs while the pipe works:
//
//   step 1   S  = Q K^T        16 MFMAs   A: rows of the Q tile (LDS), B: K registers
//   step 2   dP = dO V^T       16 MFMAs   A: rows of the dO tile, B: V (LDS)        beside them: P from S
//   step 3   dV^T += dO^T P    16 MFMAs   A: transposing reads of the dO tile, B: P  beside them: dS from P, dP
//   step 4   dK^T += Q^T dS    16 MFMAs   A: transposing reads of the Q tile, B: dS
//
// Every LDS fragment a wave reads feeds two MFMAs (one per key block of the wave): half the LDS traffic per MFMA of
// a 32-key wave: with eight waves of 32 keys, two per SIMD, the LDS reads bounded the kernel.
#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

#include "api_util.h"
#include "attn_bwd.h"
#include "attn_cfg.h"
#include "common.h"

#include <type_traits>

namespace distca {
namespace {

constexpr int kThreads = 256;
constexpr int kBN = kBwdKV;    // keys per workgroup
constexpr int kBM = kBwdRows;  // flattened query rows per block
static_assert(kBN == 256 && kBM == 32, "tile geometry of this kernel");
constexpr int kRow = 256;      // bytes per tile row, chunks swizzled by tile_swz
constexpr int kStages = 4;
constexpr int kTileQ = 0, kTileDO = kBM * kRow;
constexpr int kTileBytes = 2 * kBM * kRow;
constexpr int kStatBytes = 3 * kBM * 4;  // lse2, -delta, lim per row
constexpr int kStatOff = kStages * kTileBytes;
constexpr int kVPitch = 272;             // resident V rows (padded: 128-bit row reads without bank conflicts)
constexpr int kVOff = kStatOff + kStages * kStatBytes;
// Of the eight 16-element slices over d of a wave's V rows, the first kVRegSlices stay in registers as B operands
// beside K (as many as fit without spills inside the block loops: 12 fewer of a block's 72 LDS reads, -2 %); the
// rest is read from LDS every block.
constexpr int kVRegSlices = 6;
constexpr int kLds = kVOff + kBN * kVPitch;
static_assert(kLds <= 160 * 1024, "LDS budget");
#ifndef DISTCA_RAWBAR
#define DISTCA_RAWBAR 1
#endif
constexpr int kLoadsPerBlock = 5;        // vector-memory instructions a wave issues per block
constexpr float kLog2e = 1.4426950408889634f;

template <int N>
__device__ __forceinline__ void wait_vm() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}
__device__ __forceinline__ void fence() { __builtin_amdgcn_sched_barrier(0); }
// This file is compiled with the compiler's default choice of MFMA form, which at 512 registers per wave keeps
// every MFMA result in the accumulation registers: right for the 256 dK / dV accumulators, which only MFMAs touch
// and which fill that file exactly.  The S and dP accumulators, which the vector ALU reads and overwrites, must
// live in the ordinary vector registers instead, and the only way to say so per instruction is to write those
// MFMAs as assembly with vector-register operands.  The compiler does not know what such a statement executes and
// so does not space its result from the vector instructions that read it (11 quad-cycles for this MFMA): the
// order of a block's instructions below keeps at least one later MFMA, which cannot start before the pipe has
// finished with the one in question, between every such MFMA and the first read of its result.
__device__ __forceinline__ void mfma32_v(f32x16 &acc, elemx8 a, elemx8 b) {
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_v0(f32x16 &acc, elemx8 a, elemx8 b) {  // acc = A B
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_vc(f32x16 &acc, elemx8 a, elemx8 b, const f32x16 &c0) {  // acc = A B + c0
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "v"(b), "v"(c0));
}

template <bool ALIAS>
__global__ __launch_bounds__(kThreads, 1) void ca_bwd_dkdv64_kernel(BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int nitems = a.sched[0];
  int item, kvh;
  if (!take_item(a.tickets, nitems, a.hkv, reinterpret_cast<int32_t *>(lds), item, kvh)) return;
  const int4 it4 = reinterpret_cast<const int4 *>(a.sched + a.sched_items_off)[item];
  const int task = it4.x, nblk = it4.y;

  const int q0 = a.cu_q[task];
  const int lq = a.cu_q[task + 1] - q0;
  const int lk = a.cu_k[task + 1] - a.cu_k[task];
  const int ks = a.kv_off ? a.kv_off[task] : a.cu_k[task];
  const int G = a.group;
  const int shift = lk - lq;
  const int nrows = lq * G;
  const int nmb = (nrows + kBM - 1) / kBM;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, g = lane >> 5;
  const int kb0 = nblk * kBN;        // first key of the workgroup
  const int kw0 = kb0 + wave * 64;   // first key of the wave

  int mb0 = 0;
  if (a.causal) {
    int t_first = kb0 - shift;
    if (t_first < 0) t_first = 0;
    mb0 = (int)(((int64_t)t_first * G) / kBM);
  }
  // the query blocks of this item, visited from block top - 1 down to block bot: all that see the key block,
  // or one piece of them (sched.h)
  int top = nmb, bot = mb0;
  {
    const int piece = item_piece(it4.w), pieces = item_pieces(it4.w);
    if (pieces > 1) {
      const int n = nmb > mb0 ? nmb - mb0 : 0;
      top = nmb - piece_begin(n, piece, pieces);
      bot = nmb - piece_begin(n, piece + 1, pieces);
    }
  }
  const int niter = top > bot ? top - bot : 0;

  const int64_t kv_stride = (int64_t)a.hkv * kHeadDim;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(DISTCA_LDS uint8_t *)lds;
  auto div_group = [&](int n) { return a.group_magic ? (int)__umulhi((uint32_t)n, a.group_magic) : n; };

  // ---- K of the wave's keys as B operands (lane holds key 32 kb + l32, d = 16 s + 8 g .. +7); V of the same keys
  // into LDS, read back by this wave only, and its first kVRegSlices slices into registers as well
  elemx8 kreg[2][8], vreg[2][kVRegSlices];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb) {
    const int key = kw0 + 32 * kb + l32;
    const int64_t off = (int64_t)(ks + key) * kv_stride + kvh * kHeadDim + 8 * g;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      elemx8 kf = elemx8{0, 0, 0, 0, 0, 0, 0, 0}, vf = elemx8{0, 0, 0, 0, 0, 0, 0, 0};
      if (key < lk) {
        kf = *reinterpret_cast<const elemx8 *>(a.k + off + 16 * s);
        vf = *reinterpret_cast<const elemx8 *>(a.v + off + 16 * s);
      }
      kreg[kb][s] = kf;
      if (s < kVRegSlices) vreg[kb][s] = vf;
      *reinterpret_cast<elemx8 *>(lds + kVOff + (wave * 64 + 32 * kb + l32) * kVPitch + 32 * s + 16 * g) = vf;
    }
  }
  const int v_rd = kVOff + (wave * 64 + l32) * kVPitch + 16 * g;  // + 32*kb*kVPitch + 32*s

  f32x16 dkacc[2][4], dvacc[2][4];
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        dkacc[kb][db][r] = 0.f;
        dvacc[kb][db][r] = 0.f;
      }

  // byte offset of (token 0 of the task, first head of the group) in the query-side region
  const int64_t qbase = (a.qs_task_off ? a.qs_task_off[task] : (int64_t)q0 * a.qs_tok_bytes) + (int64_t)kvh * G * kHeadDim * 2;

  // ---- query-side tile fetch: this wave brings rows 8 w .. 8 w + 7 of a block, two LDS-direct loads each for its
  // rows of Q and of dO, and (every wave, to the same place) the 64 row statistics of the block with one load: lane L
  // fetches lse2 of row L % 32 for L < 32 and -delta of that row for L >= 32, which is the order they have in LDS.
  // kLoadsPerBlock vector-memory instructions per wave and block in every form, which the counted waits rely on.
  // Rows that do not exist (past the task, or a block below the item's last) read the zero row and get lim = -1
  // (every key masked).  Blocks whose 32 rows all exist take a form without per-lane address arithmetic when the
  // group size divides 32 (a block then starts at a token boundary): scalar bases, per-lane offsets that never change.
  const float *stat_lo = a.lse2 < a.dscaled ? a.lse2 : a.dscaled;  // the two arrays lie in one workspace
  const int64_t stat_span = a.lse2 < a.dscaled ? a.dscaled - a.lse2 : a.lse2 - a.dscaled;
  const bool fast_ok = (kBM % G) == 0 && ((int64_t)G * a.total_q + stat_span) * 4 < (1ll << 32) && 32 * a.qs_tok_bytes < (1ll << 32);
  const int tok_per_blk = kBM / G;
  uint32_t voff_q[2], voff_s;
  int tok_l;  // token, within a block that starts at a token boundary, of row l32
  {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int rl = wave * 8 + 4 * i + (lane >> 4);
      const int tq = div_group(rl);
      voff_q[i] = (uint32_t)(tq * a.qs_tok_bytes + (rl - tq * G) * (kHeadDim * 2) + (((lane & 15) ^ tile_swz(rl)) << 4));
    }
    tok_l = div_group(l32);
    const int64_t which = (g == 0) == (a.lse2 < a.dscaled) ? 0 : stat_span;  // lanes < 32: lse2, the others: -delta
    voff_s = (uint32_t)((((int64_t)(l32 - tok_l * G)) * a.total_q + tok_l + which) * 4);
  }
  const uint8_t *q_task = reinterpret_cast<const uint8_t *>(a.q) + qbase;     // token 0 of the task, first head of the group
  const uint8_t *do_task = reinterpret_cast<const uint8_t *>(a.dout) + qbase;
  const float *stat_task = stat_lo + (int64_t)kvh * G * a.total_q + q0;
  const uint32_t m0_wave = lds0 + wave * 8 * kRow;  // + stage * kTileBytes [+ kTileDO] [+ 4 * kRow]
  auto block_is_fast = [&](int mbx) { return fast_ok && mbx >= bot && mbx < top && (mbx + 1) * kBM <= nrows; };
  auto issue_fast = [&](int stage, int mbx) {
    const int tok0 = mbx * tok_per_blk;
    const uint32_t stat = kStatOff + stage * kStatBytes;
    int lm = a.causal ? tok0 + tok_l + shift : lk - 1;
    if (lm > lk - 1) lm = lk - 1;
    reinterpret_cast<int *>(lds + stat + 2 * kBM * 4)[l32] = lm;
    const int64_t tb = (int64_t)tok0 * a.qs_tok_bytes;
    const uint32_t m0 = m0_wave + stage * kTileBytes;
    lds_direct_load16(q_task + tb, voff_q[0], m0 + kTileQ);
    lds_direct_load16(do_task + tb, voff_q[0], m0 + kTileDO);
    lds_direct_load16(q_task + tb, voff_q[1], m0 + kTileQ + 4 * kRow);
    lds_direct_load16(do_task + tb, voff_q[1], m0 + kTileDO + 4 * kRow);
    lds_direct_load4_base(stat_task + tok0, voff_s, lds0 + stat);
  };
  auto issue_slow = [&](int stage, int mbx) {
    const int tile = stage * kTileBytes;
    const int stat = kStatOff + stage * kStatBytes;
    const bool blk_ok = mbx >= bot && mbx < top;
    {  // row statistics and limits
      const int rho = mbx * kBM + l32;
      const bool ok = blk_ok && rho < nrows;
      const int rc = ok ? rho : nrows - 1;
      const int tok = div_group(rc);
      const int hg = rc - tok * G;
      int lm = a.causal ? tok + shift : lk - 1;
      if (lm > lk - 1) lm = lk - 1;
      reinterpret_cast<int *>(lds + stat + 2 * kBM * 4)[l32] = ok ? lm : -1;
      const int64_t so = (int64_t)(kvh * G + hg) * a.total_q + q0 + tok;
      lds_direct_load4((g == 0 ? a.lse2 : a.dscaled) + so, lds0 + stat);
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int rl = wave * 8 + 4 * i + (lane >> 4);
      const int rho = mbx * kBM + rl;
      const bool ok = blk_ok && rho < nrows;
      const int tok = div_group(ok ? rho : 0);
      const int hg = (ok ? rho : 0) - tok * G;
      const int chunk = (lane & 15) ^ tile_swz(rl);
      const int64_t eo = qbase + (int64_t)tok * a.qs_tok_bytes + hg * (kHeadDim * 2);
      const elem_t *qs = reinterpret_cast<const elem_t *>(ok ? reinterpret_cast<const uint8_t *>(a.q) + eo : reinterpret_cast<const uint8_t *>(a.zero_row));
      const elem_t *ds = reinterpret_cast<const elem_t *>(ok ? reinterpret_cast<const uint8_t *>(a.dout) + eo : reinterpret_cast<const uint8_t *>(a.zero_row));
      const uint32_t dst = lds0 + tile + (wave * 8 + 4 * i) * kRow;
      lds_direct_load16_ptr(qs + chunk * 8, dst + kTileQ);
      lds_direct_load16_ptr(ds + chunk * 8, dst + kTileDO);
    }
  };
  auto issue_tile = [&](int stage, int mbx) {
    if (block_is_fast(mbx)) issue_fast(stage, mbx);
    else issue_slow(stage, mbx);
  };

  const float c = a.scale * kLog2e;
  const int a_rd = l32 * kRow + ((g ^ tile_swz(l32)) << 4);  // A operand rows of the query tile, ^ 32*s
  // transposed A operand: lane points at (row 4g + i4 [+8 hi +16 (j>>2)], chunk 8 b4 + h1 [+2 (j&3)], half lane&1);
  // tile_swz of that row is (i4<<1) | (g<<3) | hi
  const int i4 = (lane & 15) >> 2, b4 = (lane >> 4) & 1, h1 = (lane & 3) >> 1;
  const int t_rd = (4 * g + i4) * kRow + ((((b4 ^ g) << 3) | (i4 << 1) | h1) << 4) + 8 * (lane & 1);  // ^ 32*(j&3) ^ 16*hi

  wait_vm<0>();  // K and V have arrived; the counted waits below cover the tile loads only
  // The item's blocks are walked downwards from block top - 1 or upwards from block bot, as the schedule says
  // (sched.h, kWalkUp: items of alternate rounds meet at the same query rows, which their XCD's L2 then serves).
  const bool walk_up = (it4.w & kWalkUp) != 0;
  auto block_at = [&](int p) { return walk_up ? bot + p : top - 1 - p; };
  if (niter > 0) {
    issue_tile(0, block_at(0));
    issue_tile(1, block_at(1));
  }

  // One block.  MASKED: the block straddles the diagonal or the end of the task, compare and select per element.
  auto block = [&](int stage, auto masked) __attribute__((always_inline)) {
    constexpr bool kMasked = decltype(masked)::value;
    const uint8_t *tile = lds + stage * kTileBytes;
    const uint8_t *stat = lds + kStatOff + stage * kStatBytes;
    f32x16 sacc[2], dpacc[2];
    // row statistics of this lane's accumulator rows (register 4 cq + rr is query row 8 cq + 4 g + rr), fetched
    // from LDS a little ahead of their use rather than held for the whole block; dP accumulates on top of -delta
    // of its rows, so that dS = P * (what the MFMAs leave)
    f32x4 lse_buf[2];
    i32x4 lim_buf[2];
    auto load_stat = [&](int cq) {
      const int qr = 8 * cq + 4 * g;
      lse_buf[cq & 1] = *reinterpret_cast<const f32x4 *>(stat + qr * 4);
      if constexpr (kMasked) lim_buf[cq & 1] = *reinterpret_cast<const i32x4 *>(stat + 2 * kBM * 4 + qr * 4);
    };
    // -delta of the rows, loaded into the registers of the first key half's dP accumulator, is also the C operand of
    // the first dP MFMA of the second key half, which is issued first (no copy)
#pragma unroll
    for (int cq = 0; cq < 4; ++cq) {
      const f32x4 nd = *reinterpret_cast<const f32x4 *>(stat + kBM * 4 + (8 * cq + 4 * g) * 4);
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) dpacc[0][4 * cq + rr] = nd[rr];
    }
    // ---- step 1: S = Q K^T
    elemx8 qa[2], da[2], vb[2][2];
    auto load_q = [&](int s, int buf) { qa[buf] = *reinterpret_cast<const elemx8 *>(tile + kTileQ + (a_rd ^ (s << 5))); };
    auto load_dv = [&](int s, int buf) {
      da[buf] = *reinterpret_cast<const elemx8 *>(tile + kTileDO + (a_rd ^ (s << 5)));
      if (s >= kVRegSlices) {
        vb[buf][0] = *reinterpret_cast<const elemx8 *>(lds + v_rd + 32 * s);
        vb[buf][1] = *reinterpret_cast<const elemx8 *>(lds + v_rd + 32 * kVPitch + 32 * s);
      }
    };
    load_q(0, 0);
    load_q(1, 1);
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      fence();
      if (s == 0) {
        mfma32_v0(sacc[0], qa[0], kreg[0][0]);
        mfma32_v0(sacc[1], qa[0], kreg[1][0]);
      } else {
        mfma32_v(sacc[0], qa[s & 1], kreg[0][s]);
        mfma32_v(sacc[1], qa[s & 1], kreg[1][s]);
      }
      fence();
      if (s + 2 < 8) load_q(s + 2, s & 1);
      if (s >= 6) load_dv(s - 6, s - 6);  // the first operands of step 2
      if (s == 7) load_stat(0);
    }

    // ---- step 2: dP = dO V^T; beside the MFMAs, P = exp2(S c - lse2) of two elements per MFMA
    elemx8 pb[2][2], dsb[2][2];
    auto p_elem = [&](int kb, int r) {
      float p = fast_exp2(__builtin_fmaf(sacc[kb][r], c, -lse_buf[(r >> 2) & 1][r & 3]));
      if constexpr (kMasked) {
        if (kw0 + 32 * kb + l32 > lim_buf[(r >> 2) & 1][r & 3]) p = 0.f;
      }
      sacc[kb][r] = p;
    };
    auto p_cvt = [&](int kb, int t) {
      const int r0 = 8 * t;
      pb[kb][t] = cvt8(sacc[kb][r0], sacc[kb][r0 + 1], sacc[kb][r0 + 2], sacc[kb][r0 + 3], sacc[kb][r0 + 4], sacc[kb][r0 + 5],
                       sacc[kb][r0 + 6], sacc[kb][r0 + 7]);
    };
    elemx4 ct[2][2];  // transposed fragments [buffer][lo, hi]
    auto load_t = [&](int which, int j, int buf) {
      const int lo = (16 * (j >> 2)) * kRow + (t_rd ^ ((j & 3) << 5));
      const int hi = (16 * (j >> 2) + 8) * kRow + (t_rd ^ ((j & 3) << 5) ^ 16);
      ct[buf][0] = lds_read_tr((const DISTCA_LDS void *)(tile + which + lo));
      ct[buf][1] = lds_read_tr((const DISTCA_LDS void *)(tile + which + hi));
    };
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      fence();
      if (s == 0) {
        mfma32_vc(dpacc[1], da[0], vreg[1][0], dpacc[0]);
        mfma32_v(dpacc[0], da[0], vreg[0][0]);
      } else {
        mfma32_v(dpacc[0], da[s & 1], s < kVRegSlices ? vreg[0][s < kVRegSlices ? s : 0] : vb[s & 1][0]);
      }
      fence();
      p_elem(0, 2 * s);
      p_elem(0, 2 * s + 1);
      if (s == 4) p_cvt(0, 0);
      fence();
      if (s > 0) mfma32_v(dpacc[1], da[s & 1], s < kVRegSlices ? vreg[1][s < kVRegSlices ? s : 0] : vb[s & 1][1]);
      fence();
      p_elem(1, 2 * s);
      p_elem(1, 2 * s + 1);
      if (s == 4) p_cvt(1, 0);
      if (s + 2 < 8) load_dv(s + 2, s & 1);
      if (s >= 6) load_t(kTileDO, s - 6, s - 6);  // the first operands of step 3
      if ((s & 1) == 0 && s < 6) load_stat(s / 2 + 1);  // statistics of the rows of steps s + 2, s + 3
    }
    fence();
    p_cvt(0, 1);
    p_cvt(1, 1);

    // ---- step 3: dV^T += dO^T P; beside the MFMAs, dS = P (dP - delta) of two elements per MFMA
    auto ds_elem = [&](int kb, int r) { dpacc[kb][r] = sacc[kb][r] * dpacc[kb][r]; };
    auto ds_cvt = [&](int kb, int t) {
      const int r0 = 8 * t;
      dsb[kb][t] = cvt8(dpacc[kb][r0], dpacc[kb][r0 + 1], dpacc[kb][r0 + 2], dpacc[kb][r0 + 3], dpacc[kb][r0 + 4], dpacc[kb][r0 + 5],
                        dpacc[kb][r0 + 6], dpacc[kb][r0 + 7]);
    };
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const elemx8 dot = cat4(ct[j & 1][0], ct[j & 1][1]);
      fence();
      dvacc[0][j & 3] = mfma32(dot, pb[0][j >> 2], dvacc[0][j & 3]);
      fence();
      ds_elem(0, 2 * j);
      ds_elem(0, 2 * j + 1);
      if (j == 4) ds_cvt(0, 0);
      fence();
      dvacc[1][j & 3] = mfma32(dot, pb[1][j >> 2], dvacc[1][j & 3]);
      fence();
      ds_elem(1, 2 * j);
      ds_elem(1, 2 * j + 1);
      if (j == 4) ds_cvt(1, 0);
      if (j + 2 < 8) load_t(kTileDO, j + 2, j & 1);
      else load_t(kTileQ, j - 6, j & 1);  // the first operands of step 4
    }
    fence();
    ds_cvt(0, 1);
    ds_cvt(1, 1);

    // ---- step 4: dK^T += Q^T dS
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const elemx8 qt = cat4(ct[j & 1][0], ct[j & 1][1]);
      fence();
      dkacc[0][j & 3] = mfma32(qt, dsb[0][j >> 2], dkacc[0][j & 3]);
      dkacc[1][j & 3] = mfma32(qt, dsb[1][j >> 2], dkacc[1][j & 3]);
      fence();
      if (j + 2 < 8) load_t(kTileQ, j + 2, j & 1);
    }
  };

  // Along a walk the furthest key a block's rows see only falls (downwards) or only grows (upwards) from block to
  // block: blocks that see all of this wave's keys from every row (no masking), blocks on the diagonal (masked)
  // and, for waves whose keys lie past the diagonal of some blocks, blocks that see none of them come in that
  // order or in the reverse.  Each kind has a loop of its own with one body (with the two bodies and a skip in one loop the
  // register allocator moved the 256 accumulators between the register files in every iteration); every wave
  // passes the same barriers and makes the same requests in all of them.  A block cut off by the end of the task
  // needs no masking on that account: its missing rows are zero rows of Q and dO, which add nothing to dK or dV
  // whatever P and dS come out as (their statistics are those of the task's last row, so both stay finite).
  auto row_limit = [&](int rho) {  // the last key that flattened row rho sees
    int lm = a.causal ? div_group(rho) + shift : lk - 1;
    return lm > lk - 1 ? lk - 1 : lm;
  };
  auto advance = [&](int p) {
    // block p has landed when at most the loads of block p + 1 are still on their way (requests are made for blocks
    // past the end as well, from the zero row, which keeps that count fixed)
    wait_vm<kLoadsPerBlock>();
#if DISTCA_RAWBAR
    // the bare barrier instruction: what it orders are the LDS-direct loads, which the counted wait above covers;
    // __syncthreads() would also wait for this wave's own LDS reads in flight
    fence();
    asm volatile("s_barrier" ::: "memory");
    fence();
#else
    __syncthreads();
#endif
    // stage (p + 2) % 4 was last read for block p - 2, which every wave left before this barrier
    issue_tile((p + 2) % kStages, block_at(p + 2));
  };
  // 2: every row of the block sees all of this wave's keys; 1: some rows see some; 0: none does
  auto block_kind = [&](int p) {
    const int mbx = block_at(p);
    if (kw0 + 63 <= row_limit(mbx * kBM)) return 2;
    int rho_last = (mbx + 1) * kBM - 1;
    if (rho_last > nrows - 1) rho_last = nrows - 1;
    return kw0 <= row_limit(rho_last) ? 1 : 0;
  };
  // Along a walk the kinds come in the order 2, 1, 0 (downwards) or 0, 1, 2 (upwards): five loops in a row, of
  // which a walk uses three.
  int p = 0;
  for (; p < niter && block_kind(p) == 0; ++p) advance(p);
  for (; p < niter && block_kind(p) == 1; ++p) {
    advance(p);
    block(p % kStages, std::true_type{});
  }
  for (; p < niter && block_kind(p) == 2; ++p) {
    advance(p);
    block(p % kStages, std::false_type{});
  }
  for (; p < niter && block_kind(p) == 1; ++p) {
    advance(p);
    block(p % kStages, std::true_type{});
  }
  for (; p < niter; ++p) advance(p);
  wait_vm<0>();  // nothing may still be on its way into LDS when the workgroup ends

  // ---- epilogue: dK, dV of this wave's keys (registers 4*cq..+3 of block db hold d0..d0+3)
#pragma unroll
  for (int kb = 0; kb < 2; ++kb)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) dkacc[kb][db][r] *= a.scale;
  if (ALIAS) {
    // Work items that share K/V rows (tasks over one stored prefix, pieces of one key block) add up in fp32; the
    // order of these additions is the one source of run-to-run variation.  A lane holds one key's values, 2 KB apart
    // from its neighbour's in memory: the sums pass through LDS so that one atomic instruction covers 64
    // consecutive floats of a row instead of 64 rows.
    constexpr int kEpiPitch = (kHeadDim + 4) * 4;  // bytes per key row in LDS; the 16 spare bytes spread the banks
    static_assert(kBN * kEpiPitch <= kLds, "the epilogue stages one 256 x 128 fp32 matrix in LDS");
    __syncthreads();  // every wave has finished with the V rows and the tile ring
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      float *dst = which == 0 ? a.dk_acc : a.dv_acc;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const int wkey0 = wave * 64 + 32 * kb;  // this wave's rows of the staging matrix: written and read by it alone
        const int nkeys = lk - (kw0 + 32 * kb) < 32 ? lk - (kw0 + 32 * kb) : 32;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int cq = 0; cq < 4; ++cq) {
            const int d0 = 16 * db + 64 * (cq >> 1) + 8 * (cq & 1) + 4 * g;
            const f32x16 &acc = which == 0 ? dkacc[kb][db] : dvacc[kb][db];
            *reinterpret_cast<f32x4 *>(lds + (wkey0 + l32) * kEpiPitch + d0 * 4) = f32x4{acc[4 * cq], acc[4 * cq + 1], acc[4 * cq + 2], acc[4 * cq + 3]};
          }
        // LDS operations of one wave complete in order: the reads below see the writes above
        for (int kk = 0; kk < nkeys; ++kk) {
          const float *row = reinterpret_cast<const float *>(lds + (wkey0 + kk) * kEpiPitch);
          float *out = dst + (int64_t)(ks + kw0 + 32 * kb + kk) * kv_stride + kvh * kHeadDim;
          unsafeAtomicAdd(out + lane, row[lane]);
          unsafeAtomicAdd(out + 64 + lane, row[64 + lane]);
        }
      }
    }
  } else {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int key = kw0 + 32 * kb + l32;
      if (key < lk) {
        const int64_t off = (int64_t)(ks + key) * kv_stride + kvh * kHeadDim;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int cq = 0; cq < 4; ++cq) {
            const int d0 = 16 * db + 64 * (cq >> 1) + 8 * (cq & 1) + 4 * g;
            *reinterpret_cast<elemx4 *>(a.dk + off + d0) =
                cvt4(dkacc[kb][db][4 * cq], dkacc[kb][db][4 * cq + 1], dkacc[kb][db][4 * cq + 2], dkacc[kb][db][4 * cq + 3]);
            *reinterpret_cast<elemx4 *>(a.dv + off + d0) =
                cvt4(dvacc[kb][db][4 * cq], dvacc[kb][db][4 * cq + 1], dvacc[kb][db][4 * cq + 2], dvacc[kb][db][4 * cq + 3]);
          }
      }
    }
  }
}

}  // namespace

#ifndef DISTCA_F16
int dkdv64_lds_bytes() { return kLds; }
#endif

int DISTCA_FN(launch_dkdv64)(const BwdArgs &a, int64_t grid, bool alias, hipStream_t stream) {
  if (device_setup_pending(kSlotBwdLds64)) {
    hipError_t e1 = hipFuncSetAttribute((const void *)ca_bwd_dkdv64_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    hipError_t e2 = hipFuncSetAttribute((const void *)ca_bwd_dkdv64_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e1 != hipSuccess || e2 != hipSuccess) return fail(DISTCA_E_LAUNCH, "ca_bwd: cannot reserve %d B of LDS", kLds);
    device_setup_done(kSlotBwdLds64);
  }
  if (alias)
    hipLaunchKernelGGL((ca_bwd_dkdv64_kernel<true>), dim3((unsigned)grid), dim3(kThreads), kLds, stream, a);
  else
    hipLaunchKernelGGL((ca_bwd_dkdv64_kernel<false>), dim3((unsigned)grid), dim3(kThreads), kLds, stream, a);
  return DISTCA_OK;
}

}  // namespace distca
