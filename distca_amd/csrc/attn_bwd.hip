// Varlen causal flash-attention backward (dQ, dK, dV) for gfx950.
//
// Stands where the reference calls flash-attn's varlen backward
// (distca/runtime/megatron/ops/fused_comm_attn.py:259-272).
//
// The backward runs as two kernels that both recompute P from (Q, K, LSE), so that neither
// needs floating-point atomics and the result is bit-reproducible (the `deterministic` switch
// of the reference's FlashAttnArgs holds by construction).  A single-kernel form that added
// dQ partial sums with fp32 atomics was measured first: the atomics alone (4 bytes per
// (row, key) pair per 128 keys, 124 GB at 128K tokens) took as long as the rest of the kernel.
//
//   1. ca_bwd_dq_kernel: one workgroup of 8 waves per (task, block of 256 flattened query
//      rows, kv head), in the order of the forward tile schedule; the mirror image of the
//      forward kernel.  Q and dO stay in registers as B operands, K/V tiles of 64 keys are
//      streamed through LDS:
//        S^T = K Q^T, dP^T = V dO^T        A from LDS rows, B from registers
//        P, dS as above (one query row per lane: lse2 and delta are per-lane scalars)
//        dQ^T += K^T dS^T                  A by transposing LDS reads of the K tile, B = dS registers
//      Its prologue, which reads a row's dO anyway, also makes the row statistics both kernels need
//      (delta = <dO, O>, lse * log2(e)) and leaves them in the workspace.
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

constexpr float kLog2e = 1.4426950408889634f;

// ------------------------------------------------------------------------------------------
// dQ
// ------------------------------------------------------------------------------------------
constexpr int kDqKV = kFwdKV;  // 64 keys per tile
constexpr int kDqRowB = 256;                   // unpadded rows, chunks swizzled by tile_swz
constexpr int kDqTile = kDqKV * kDqRowB;
constexpr int kDqStage = 2 * kDqTile;          // K tile + V tile
constexpr int kDqLds = 2 * kDqStage;

template <int MSUB>
__global__ __launch_bounds__(kWaves * 64, (MSUB == 1 && kWaves == 4 ? 2 : 1)) void ca_bwd_dq_kernel(BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int nitems = a.sched[0];
  int item, kvh;
  if (!take_item(a.tickets, nitems, a.hkv, reinterpret_cast<int32_t *>(lds), item, kvh)) return;
  const int4 it4 = reinterpret_cast<const int4 *>(a.sched + a.sched_items_off)[item];
  const int task = it4.x, mblk = it4.y;

  const int q0 = a.cu_q[task];
  const int64_t qs_task = a.qs_task_off ? a.qs_task_off[task] : (int64_t)q0 * a.qs_tok_bytes;
  const int64_t dq_task = a.dq_task_off ? a.dq_task_off[task] : (int64_t)q0 * a.dq_tok_bytes;
  const int lq = a.cu_q[task + 1] - q0;
  const int lk = a.cu_k[task + 1] - a.cu_k[task];
  const int ks = a.kv_off ? a.kv_off[task] : a.cu_k[task];
  const int G = a.group;
  const int shift = lk - lq;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  constexpr int kRows = kWaves * 32 * MSUB;
  const int row_wg = mblk * kRows;
  const int nrows = lq * G;

  int tok_end = (row_wg + kRows + G - 1) / G;
  if (tok_end > lq) tok_end = lq;
  int nvis = a.causal ? tok_end + shift : lk;
  if (nvis > lk) nvis = lk;
  const int ntiles = nvis > 0 ? (nvis + kDqKV - 1) / kDqKV : 0;

  int row[MSUB], tok[MSUB], lim[MSUB];
  bool valid[MSUB];
  float lse2[MSUB], dsc[MSUB];
  elemx8 qf[MSUB][8], dof[MSUB][8];
#pragma unroll
  for (int m = 0; m < MSUB; ++m) {
    row[m] = row_wg + (wave * MSUB + m) * 32 + l32;
    valid[m] = row[m] < nrows;
    tok[m] = row[m] / G;
    const int hg = row[m] - tok[m] * G;
    int lm = a.causal ? tok[m] + shift : lk - 1;
    if (lm > lk - 1) lm = lk - 1;
    lim[m] = lm;
    const int64_t ro = qs_task + (int64_t)tok[m] * a.qs_tok_bytes + ((kvh * G + hg) * kHeadDim + 8 * g) * 2;  // bytes
    lse2[m] = INFINITY;  // rows past the task: P = exp2(-inf) = 0
    dsc[m] = 0.f;
    // The row statistics of the backward are made here, where the row's dO is read anyway, and left in the
    // workspace for the dK/dV kernel, which runs after this one: delta = <dO, O> over the row (this lane's half of
    // d, then the sum of the lane pair) and lse in the log2 domain.
    float part = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      if (valid[m]) {
        qf[m][s] = *reinterpret_cast<const elemx8 *>(reinterpret_cast<const uint8_t *>(a.q) + ro + 32 * s);
        dof[m][s] = *reinterpret_cast<const elemx8 *>(reinterpret_cast<const uint8_t *>(a.dout) + ro + 32 * s);
        const elemx8 of = *reinterpret_cast<const elemx8 *>(reinterpret_cast<const uint8_t *>(a.out) + ro + 32 * s);
#pragma unroll
        for (int i = 0; i < 8; ++i) part += (float)dof[m][s][i] * (float)of[i];
      } else {
        qf[m][s] = elemx8{0, 0, 0, 0, 0, 0, 0, 0};
        dof[m][s] = elemx8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
    const float delta = pair_sum(part);
    if (valid[m]) {
      const int64_t so = (int64_t)(kvh * G + hg) * a.total_q + q0 + tok[m];
      const float l = a.lse_tok ? reinterpret_cast<const float *>(a.lse_tok + qs_task + (int64_t)tok[m] * a.qs_tok_bytes)[kvh * G + hg]
                                : a.lse[so];
      lse2[m] = l * kLog2e;
      dsc[m] = delta * a.scale;
      if (g == 0) {
        a.lse2_w[so] = lse2[m];
        a.dscaled_w[so] = -delta;  // the start value of the dP accumulators in the dK/dV kernel
      }
    }
  }
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

  // ---- K/V tile fetch by LDS-direct loads, as in the forward kernel: a wave brings kRowsW rows of
  // the K tile and of the V tile, four rows per instruction
  const int64_t kv_stride = (int64_t)a.hkv * kHeadDim;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(DISTCA_LDS uint8_t *)lds;
  const int uwave = __builtin_amdgcn_readfirstlane(wave);
  const elem_t *kbase = a.k + (int64_t)ks * kv_stride + kvh * kHeadDim;
  const elem_t *vbase = a.v + (int64_t)ks * kv_stride + kvh * kHeadDim;
  constexpr int kRowsW = kDqKV / kWaves, kLdW = 2 * (kRowsW / 4);
  auto issue_kv = [&](int j, int stage, int i) {
    const bool is_k = i < kLdW / 2;
    const int ii = is_k ? i : i - kLdW / 2;
    const int r = kRowsW * uwave + 4 * ii + (lane >> 4);
    const int key = j * kDqKV + r;
    const int chunk = (lane & 15) ^ tile_swz(r);
    const elem_t *src = (is_k ? kbase : vbase) + (int64_t)key * kv_stride;
    if (key >= lk) src = reinterpret_cast<const elem_t *>(a.zero_row);
    const uint32_t dst = lds0 + stage * kDqStage + (is_k ? 0 : kDqTile) + (kRowsW * uwave + 4 * ii) * kDqRowB;
    lds_direct_load16_ptr(src + chunk * 8, dst);
  };
  // Tiles that lie wholly inside the prefix (all but the last one) take a form without per-lane address
  // arithmetic: a scalar base that advances by one tile, plus a per-lane offset that never changes.
  uint32_t voff[kLdW / 2];
#pragma unroll
  for (int ii = 0; ii < kLdW / 2; ++ii) {
    const int r = kRowsW * uwave + 4 * ii + (lane >> 4);
    voff[ii] = (uint32_t)((r * kv_stride + (((lane & 15) ^ tile_swz(r)) * 8)) * 2);
  }
  auto issue_kv_whole = [&](int j, int stage, int i) {
    const bool is_k = i < kLdW / 2;
    const int ii = is_k ? i : i - kLdW / 2;
    const elem_t *tb = (is_k ? kbase : vbase) + (int64_t)j * kDqKV * kv_stride;
    lds_direct_load16(tb, voff[ii], lds0 + stage * kDqStage + (is_k ? 0 : kDqTile) + (kRowsW * uwave + 4 * ii) * kDqRowB);
  };

  f32x16 dqacc[MSUB][4];
#pragma unroll
  for (int m = 0; m < MSUB; ++m)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) dqacc[m][db][r] = 0.f;
  const float c = a.scale * kLog2e;
  const int k_rd = l32 * kDqRowB + ((g ^ tile_swz(l32)) << 4);  // + kb*32*kDqRowB, ^ 32*s
  // transposed K operand: lane points at (key 4g + i4 [+8 hi +16 t], chunk 8 b4 + h1 [+2 db], half lane&1)
  const int i4 = (lane & 15) >> 2, b4 = (lane >> 4) & 1, h1 = (lane & 3) >> 1;
  const int t_rd = (4 * g + i4) * kDqRowB + ((((b4 ^ g) << 3) | (i4 << 1) | h1) << 4) + 8 * (lane & 1);  // ^ 32*db ^ 16*hi

  if (ntiles > 0) {
#pragma unroll
    for (int i = 0; i < kLdW; ++i) issue_kv(0, 0, i);
  }
  wait_vm0();
  __syncthreads();

  // Absolute LDS addresses of this lane's operand reads in stage 0, the eight swizzled variants of each, kept
  // in registers; the tile loop is unrolled by two so that the stage is a constant in the instruction's offset
  // field: no address arithmetic is left between the MFMAs.
  uint32_t k_ad[8], t_ad[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    k_ad[i] = lds0 + (k_rd ^ (i << 5));
    t_ad[i] = lds0 + (t_rd ^ ((i & 3) << 5) ^ ((i >> 2) << 4));
    asm volatile("" : "+v"(k_ad[i]), "+v"(t_ad[i]));
  }
  auto tile_step = [&](int j, auto par) __attribute__((always_inline)) {
    constexpr int stage = decltype(par)::value;
    const bool has_next = j + 1 < ntiles;

    const int key0 = j * kDqKV;
    const bool active = wave_live && key0 <= lim_last;
    // the next tile: whole tiles are requested one instruction per MFMA step below; the one the end of the
    // prefix cuts off (the last) needs per-lane addresses and is requested here
    const bool next_whole = has_next && (j + 2) * kDqKV <= lk;
    if (has_next && (!next_whole || !active)) {
#pragma unroll
      for (int i = 0; i < kLdW; ++i) issue_kv(j + 1, stage ^ 1, i);
    }
    if (active) {
      // ---- S^T = K Q^T, dP^T = V dO^T : [64 keys] x [32*MSUB rows]
      f32x16 sacc[MSUB][2], dpacc[MSUB][2];
#pragma unroll
      for (int m = 0; m < MSUB; ++m)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            sacc[m][kb][r] = 0.f;
            dpacc[m][kb][r] = 0.f;
          }
      // operand fragments are requested kPf steps before the MFMAs that use them; the next tile's
      // loads go out one instruction per step
      constexpr int kPf = 1;
      elemx8 kf[kPf][2], vf[kPf][2];
      auto load_kv = [&](int s, int buf) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          kf[buf][kb] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(k_ad[s] + stage * kDqStage + kb * 32 * kDqRowB));
          vf[buf][kb] = *static_cast<const DISTCA_LDS elemx8 *>(lds_ptr(k_ad[s] + stage * kDqStage + kDqTile + kb * 32 * kDqRowB));
        }
      };
#pragma unroll
      for (int s = 0; s < kPf; ++s) load_kv(s, s);
#pragma unroll
      for (int s = 0; s < 8; ++s) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int m = 0; m < MSUB; ++m) {
            sacc[m][kb] = mfma32(kf[s % kPf][kb], qf[m][s], sacc[m][kb]);
            dpacc[m][kb] = mfma32(vf[s % kPf][kb], dof[m][s], dpacc[m][kb]);
          }
        __builtin_amdgcn_sched_barrier(0);
        if (s + kPf < 8) load_kv(s + kPf, s % kPf);
        if (next_whole && s < kLdW) issue_kv_whole(j + 1, stage ^ 1, s);
      }
      // ---- P, dS (one query row per lane) and the bf16 B operand of the dQ product
      const bool need_mask = key0 + kDqKV - 1 > lim_first;
      elemx8 dsf[MSUB][4];
#pragma unroll
      for (int m = 0; m < MSUB; ++m) {
        // the masked form only for tiles that straddle the diagonal or the end of the prefix (uniform branch)
        auto body = [&](auto masked) __attribute__((always_inline)) {
#pragma unroll
          for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              float p = fast_exp2(__builtin_fmaf(sacc[m][kb][r], c, -lse2[m]));
              if constexpr (decltype(masked)::value) {
                if (key0 + kb * 32 + acc_row(r, g) > lim[m]) p = 0.f;
              }
              dpacc[m][kb][r] = p * __builtin_fmaf(dpacc[m][kb][r], a.scale, -dsc[m]);
            }
        };
        if (need_mask) body(std::true_type{});
        else body(std::false_type{});
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int kb = t >> 1, r0 = 8 * (t & 1);
          dsf[m][t] = cvt8(dpacc[m][kb][r0], dpacc[m][kb][r0 + 1], dpacc[m][kb][r0 + 2], dpacc[m][kb][r0 + 3], dpacc[m][kb][r0 + 4],
                           dpacc[m][kb][r0 + 5], dpacc[m][kb][r0 + 6], dpacc[m][kb][r0 + 7]);
        }
      }
      // ---- dQ^T += K^T dS^T : [128 d] x [32*MSUB rows], contraction over the 64 keys
      constexpr int kPfT = 4;
      elemx4 ktf[kPfT][2];
      auto load_t = [&](int u, int buf) {  // u = 4*t + db
        const uint32_t ko = stage * kDqStage + 16 * (u >> 2) * kDqRowB;
        ktf[buf][0] = lds_read_tr(lds_ptr(t_ad[u & 3] + ko));
        ktf[buf][1] = lds_read_tr(lds_ptr(t_ad[4 + (u & 3)] + ko + 8 * kDqRowB));
      };
#pragma unroll
      for (int u = 0; u < kPfT; ++u) load_t(u, u);
#pragma unroll
      for (int u = 0; u < 16; ++u) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int m = 0; m < MSUB; ++m) dqacc[m][u & 3] = mfma32(cat4(ktf[u % kPfT][0], ktf[u % kPfT][1]), dsf[m][u >> 2], dqacc[m][u & 3]);
        __builtin_amdgcn_sched_barrier(0);
        if (u + kPfT < 16) load_t(u + kPfT, u % kPfT);
      }
    }
    wait_vm0();
    __syncthreads();
  };
  for (int j = 0; j < ntiles; j += 2) {
    tile_step(j, std::integral_constant<int, 0>{});
    if (j + 1 < ntiles) tile_step(j + 1, std::integral_constant<int, 1>{});
  }

  // ---- epilogue: dQ rows (bf16)
#pragma unroll
  for (int m = 0; m < MSUB; ++m) {
    if (valid[m]) {
      const int hg = row[m] - tok[m] * G;
      elem_t *op = reinterpret_cast<elem_t *>(reinterpret_cast<uint8_t *>(a.dq) + dq_task + (int64_t)tok[m] * a.dq_tok_bytes) + (kvh * G + hg) * kHeadDim;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int cq = 0; cq < 4; ++cq) {
          const int d0 = 16 * db + 64 * (cq >> 1) + 8 * (cq & 1) + 4 * g;
          *reinterpret_cast<elemx4 *>(op + d0) =
              cvt4(dqacc[m][db][4 * cq], dqacc[m][db][4 * cq + 1], dqacc[m][db][4 * cq + 2], dqacc[m][db][4 * cq + 3]);
        }
    }
  }
}

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
BwdWorkspace bwd_layout(const distca_ca_params *p, bool alias) {
  BwdWorkspace w;
  int64_t o = 0;
  w.sched_kv = o; o += sched_region_bytes(p->num_tasks, bwd_max_items(p));
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
  // sized for the aliased-KV form so one query serves both call shapes
  return bwd_layout(p, true).total;
}

extern "C" int distca_ca_bwd(const void *dout, const void *q, const void *k, const void *v, const void *out, const float *lse,
                             void *dq, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off,
                             const distca_ca_params *p, void *workspace, int64_t workspace_bytes, void *stream) {
  if (!p) return fail(DISTCA_E_INVALID, "ca_bwd: null params");
  const int64_t row_bytes = (int64_t)p->num_heads_q * kHeadDim * 2;
  const BwdQuerySide qs{dout, q, out, lse, nullptr, nullptr, row_bytes, dq, nullptr, row_bytes};
  return (p->dtype == DISTCA_DTYPE_F16 ? run_bwd_f16 : run_bwd)(qs, k, v, dk, dv, cu_q, cu_k, kv_off, p, workspace, workspace_bytes, stream);
}

extern "C" int distca_ca_bwd_tokens(const void *req_base, const int64_t *req_task_off, int64_t req_tok_bytes, const void *k,
                                    const void *v, void *dq_base, const int64_t *dq_task_off, int64_t dq_tok_bytes, void *dk,
                                    void *dv, const int32_t *cu_q, const int32_t *cu_k, const int32_t *kv_off,
                                    const distca_ca_params *p, void *workspace, int64_t workspace_bytes, void *stream) {
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
  return (p->dtype == DISTCA_DTYPE_F16 ? run_bwd_f16 : run_bwd)(qs, k, v, dk, dv, cu_q, cu_k, kv_off, p, workspace, workspace_bytes, stream);
}
#endif  // !DISTCA_F16

namespace distca {
int DISTCA_FN(run_bwd)(const BwdQuerySide &qs, const void *k, const void *v, void *dk, void *dv, const int32_t *cu_q, const int32_t *cu_k,
                       const int32_t *kv_off, const distca_ca_params *p, void *workspace, int64_t workspace_bytes, void *stream) {
  const void *dout = qs.dout, *q = qs.q, *out = qs.out;
  void *dq = qs.dq;
  if (!p) return fail(DISTCA_E_INVALID, "ca_bwd: null params");
  int rc = validate_params(p);
  if (rc) return rc;
  const bool alias = kv_off != nullptr;
  if (p->deterministic && alias)
    return fail(DISTCA_E_UNSUPPORTED, "ca_bwd: deterministic=1 with kv_task_offsets (dK/dV of aliased rows are summed with float atomics)");
  if (!dout || !q || !k || !v || !out || (!qs.lse && !qs.lse_tok) || !dq || !dk || !dv || !cu_q || !cu_k) {
    if (p->num_tasks == 0 || (p->total_q == 0 && p->total_k == 0)) return DISTCA_OK;
    return fail(DISTCA_E_INVALID, "ca_bwd: null pointer");
  }
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv))
    return fail(DISTCA_E_INVALID, "ca_bwd: tensors must be 16-byte aligned");
  // dK/dV go through fp32 accumulators when tasks alias K/V rows or when key blocks are cut into pieces
  const bool use_acc = alias || bwd_split_target(p) > 0;
  const BwdWorkspace w = bwd_layout(p, use_acc);
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
    } else if (p->num_tasks == 0 || p->total_q == 0) {
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (u32x4 *)dk, kv_elems / 8);
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (u32x4 *)dv, kv_elems / 8);
    } else {
      // every task owns its rows and the dK/dV kernel writes each row of a task that has queries exactly once:
      // only the others need the fill (at 131 072 tokens that is 0.5 GB of writes not made)
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
  a.sched_items_off = (int32_t)sched_header_ints(p->num_tasks);
  a.hq = p->num_heads_q; a.hkv = p->num_heads_kv; a.group = p->num_heads_q / p->num_heads_kv;
  a.total_q = p->total_q; a.causal = p->causal != 0; a.scale = p->softmax_scale;
  a.group_magic = a.group == 1 ? 0u : (uint32_t)(((1ull << 32) + a.group - 1) / a.group);
  if ((uint64_t)p->max_seqlen_q * a.group * a.group >= (1ull << 32))
    return fail(DISTCA_E_UNSUPPORTED, "ca_bwd: max_seqlen_q * (Hq/Hkv)^2 must stay below 2^32");

  if (device_setup_pending(kSlotBwdLds)) {
    hipError_t e = hipFuncSetAttribute((const void *)ca_bwd_dq_kernel<kFwdMsub>, hipFuncAttributeMaxDynamicSharedMemorySize, kDqLds);
    if (e != hipSuccess) return fail(DISTCA_E_LAUNCH, "ca_bwd: cannot reserve %d B of LDS: %s", kDqLds, hipGetErrorString(e));
    device_setup_done(kSlotBwdLds);
  }

  // ---- dQ: one workgroup per (task, block of query rows, kv head).  It runs first: it also leaves the row
  // statistics (lse in the log2 domain, -delta) in the workspace, which the dK/dV kernel reads.
  {
    const SchedGeom geom = dq_geom(p);
    const int64_t max_items = dq_max_items(p);
    rc = launch_build_schedule(0, cu_q, cu_k, p->num_tasks, geom, (int32_t *)(ws + w.sched_q), max_items, s);
    if (rc) return rc;
    const int64_t grid = max_items * p->num_heads_kv * kSchedOversubNum / kSchedOversubDen;
    if (grid > 0x7fffffff) return fail(DISTCA_E_INVALID, "ca_bwd: grid too large");
    a.sched = (const int32_t *)(ws + w.sched_q);
    a.zero_row = ws + w.sched_q + sched_zero_row_off(p->num_tasks, max_items);
    a.tickets = (int32_t *)(ws + w.sched_q + sched_ticket_off(p->num_tasks, max_items));
    ScopedTimer timer(DISTCA_TIMER_CA_BWD_DQ, s);
    hipLaunchKernelGGL((ca_bwd_dq_kernel<kFwdMsub>), dim3((unsigned)grid), dim3(kWaves * 64), kDqLds, s, a);
  }
  // ---- dK, dV: one workgroup per (task, 256-key block, kv head)
  {
    const SchedGeom geom = bwd_geom(p);
    const int64_t max_items = bwd_max_items(p);
    rc = launch_build_schedule(1, cu_q, cu_k, p->num_tasks, geom, (int32_t *)(ws + w.sched_kv), max_items, s);
    if (rc) return rc;
    // the list is sized for tasks over shared K/V rows; without them the tighter bound sizes the grid (a batch of
    // many short documents and one long one would otherwise launch mostly workgroups that find nothing to do)
    const int64_t grid_items = alias ? max_items : bwd_key_blocks_own_rows(p) + bwd_split_target(p);
    const int64_t grid = grid_items * p->num_heads_kv * kSchedOversubNum / kSchedOversubDen;
    if (grid > 0x7fffffff) return fail(DISTCA_E_INVALID, "ca_bwd: grid too large");
    a.sched = (const int32_t *)(ws + w.sched_kv);
    a.zero_row = ws + w.sched_kv + sched_zero_row_off(p->num_tasks, bwd_max_items(p));
    a.tickets = (int32_t *)(ws + w.sched_kv + sched_ticket_off(p->num_tasks, max_items));
    ScopedTimer timer(DISTCA_TIMER_CA_BWD, s);
    rc = DISTCA_FN(launch_dkdv64)(a, grid, use_acc, s);
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
