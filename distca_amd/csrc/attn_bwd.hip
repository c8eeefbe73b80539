// Varlen causal flash-attention backward (dQ, dK, dV) for gfx950.
//
// Stands where the reference calls flash-attn's varlen backward
// (distca/runtime/megatron/ops/fused_comm_attn.py:259-272).
//
// Three launches on the caller's stream:
//   1. bwd_prepare:  delta[h][t] = <dO, O> per (token, head), and zero the fp32 dQ accumulator.
//   2. ca_bwd_kernel: one workgroup per (task, block of kBwdKV keys, kv head), in the order
//      of the tile schedule.  Each wave keeps K and V of its 32*KSUB keys as MFMA B operands in
//      registers together with the fp32 dK^T / dV^T accumulators, and the workgroup streams
//      the query side (Q, dO, LSE, delta of every head of the group, flattened like the
//      forward) through LDS in blocks of 32*MSUB rows, starting at the first block the causal
//      mask lets see these keys.  Per block: S = Q K^T and dP = dO V^T (A from LDS, B from
//      registers); P = exp2(S*c - LSE), dS = P (dP - delta) * scale in registers;
//      dV^T += dO^T P and dK^T += Q^T dS with the A operand fetched by transposing LDS reads
//      of the same row-major tiles and the B operand being the accumulator registers
//      converted to bf16 in place; dS goes through LDS once so that each wave can form a
//      32-column slice of dQ = dS K over all keys of the workgroup, which is added to the
//      fp32 accumulator with hardware float atomics.
//   3. bwd_finish: dQ accumulator -> bf16 (and dK/dV when tasks alias KV rows).
#include <hip/amd_detail/amd_hip_unsafe_atomics.h>

#include "api_util.h"
#include "attn_cfg.h"
#include "common.h"

namespace distca {
namespace {

constexpr int kPitch = 272;  // bytes per 128-element bf16 row in LDS
constexpr float kLog2e = 1.4426950408889634f;

struct BwdArgs {
  const __bf16 *q, *k, *v, *dout;
  const float *lse, *delta;
  float *dq_acc;
  __bf16 *dk, *dv;
  float *dk_acc, *dv_acc;  // used instead of dk/dv when tasks may alias KV rows
  const int32_t *cu_q, *cu_k, *kv_off;
  const int32_t *sched;
  int32_t sched_items_off;
  int32_t hq, hkv, group, total_q;
  int32_t causal;
  float scale;
};

template <int KSUB, int MSUB>
struct BwdLds {
  static constexpr int kBN = kWaves * 32 * KSUB;
  static constexpr int kBM = 32 * MSUB;
  static constexpr int kDsPitch = kBN * 2 + 16;
  static constexpr int kKs = 0;
  static constexpr int kQs = kKs + kBN * kPitch;
  static constexpr int kDOs = kQs + kBM * kPitch;
  static constexpr int kDSs = kDOs + kBM * kPitch;
  static constexpr int kLse = kDSs + kBM * kDsPitch;
  static constexpr int kDelta = kLse + kBM * 4;
  static constexpr int kLim = kDelta + kBM * 4;
  static constexpr int kRowOff = kLim + kBM * 4;
  static constexpr int kTotal = kRowOff + kBM * 4;
};

template <int KSUB, int MSUB, bool ALIAS>
__global__ __launch_bounds__(256, 1) void ca_bwd_kernel(BwdArgs a) {
  using L = BwdLds<KSUB, MSUB>;
  constexpr int kBN = L::kBN, kBM = L::kBM;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const int nitems = a.sched[0];
  const int item = blockIdx.x / a.hkv;
  if (item >= nitems) return;
  const int kvh = blockIdx.x - item * a.hkv;
  const int4 it = reinterpret_cast<const int4 *>(a.sched + a.sched_items_off)[item];
  const int task = it.x, nblk = it.y;

  const int q0 = a.cu_q[task];
  const int lq = a.cu_q[task + 1] - q0;
  const int lk = a.cu_k[task + 1] - a.cu_k[task];
  const int ks = a.kv_off ? a.kv_off[task] : a.cu_k[task];
  const int G = a.group;
  const int shift = lk - lq;
  const int nrows = lq * G;
  const int nmb = (nrows + kBM - 1) / kBM;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, g = lane >> 5;
  const int kb0 = nblk * kBN;            // first key of the workgroup
  const int kw0 = kb0 + wave * 32 * KSUB;  // first key of the wave

  int mb0 = 0;
  if (a.causal) {
    int t_first = kb0 - shift;
    if (t_first < 0) t_first = 0;
    mb0 = (int)(((int64_t)t_first * G) / kBM);
  }

  const int64_t kv_stride = (int64_t)a.hkv * kHeadDim;
  const int64_t q_stride = (int64_t)a.hq * kHeadDim;

  // ---- K tile of the workgroup into LDS (row-major; read transposed for dQ)
  {
    const int col = tid & 15, row = tid >> 4;
#pragma unroll
    for (int i = 0; i < kBN / 16; ++i) {
      const int r = row + 16 * i;
      const int key = kb0 + r;
      u32x4 val = u32x4{0, 0, 0, 0};
      if (key < lk) val = *reinterpret_cast<const u32x4 *>(a.k + (int64_t)(ks + key) * kv_stride + kvh * kHeadDim + col * 8);
      *reinterpret_cast<u32x4 *>(lds + L::kKs + r * kPitch + col * 16) = val;
    }
  }
  // ---- K, V of this wave's keys as B operands (lane: key l32, d = 16s + 8g ..)
  bf16x8 kfr[KSUB][8], vfr[KSUB][8];
#pragma unroll
  for (int kk = 0; kk < KSUB; ++kk) {
    const int key = kw0 + kk * 32 + l32;
    const bool ok = key < lk;
    const int64_t off = (int64_t)(ks + key) * kv_stride + kvh * kHeadDim + 8 * g;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      if (ok) {
        kfr[kk][s] = *reinterpret_cast<const bf16x8 *>(a.k + off + 16 * s);
        vfr[kk][s] = *reinterpret_cast<const bf16x8 *>(a.v + off + 16 * s);
      } else {
        kfr[kk][s] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
        vfr[kk][s] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
      }
    }
  }

  f32x16 dkacc[KSUB][4], dvacc[KSUB][4];
#pragma unroll
  for (int kk = 0; kk < KSUB; ++kk)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        dkacc[kk][db][r] = 0.f;
        dvacc[kk][db][r] = 0.f;
      }

  // ---- query-side tile staging: kBM rows x 16 chunks of 16 B for Q and for dO
  constexpr int kChunks = kBM * 16 / 256;  // per thread, per tensor
  const int ld_col = tid & 15, ld_row = tid >> 4;
  u32x4 qreg[kChunks], doreg[kChunks];
  float lse_reg[kChunks], delta_reg[kChunks];
  int lim_reg[kChunks], off_reg[kChunks];
  const int64_t qbase = ((int64_t)q0 * a.hq + kvh * G) * kHeadDim;
  auto load_tile = [&](int mb) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int r = mb * kBM + ld_row + 16 * i;
      const int tok = r / G;
      const int hg = r - tok * G;
      const bool ok = r < nrows;
      const int ro = tok * a.hq + hg;
      if (ok) {
        qreg[i] = *reinterpret_cast<const u32x4 *>(a.q + qbase + (int64_t)ro * kHeadDim + ld_col * 8);
        doreg[i] = *reinterpret_cast<const u32x4 *>(a.dout + qbase + (int64_t)ro * kHeadDim + ld_col * 8);
      } else {
        qreg[i] = u32x4{0, 0, 0, 0};
        doreg[i] = u32x4{0, 0, 0, 0};
      }
      if (ld_col == 0) {
        int lm = a.causal ? tok + shift : lk - 1;
        if (lm > lk - 1) lm = lk - 1;
        if (ok) {
          const int64_t so = (int64_t)(kvh * G + hg) * a.total_q + q0 + tok;
          lse_reg[i] = a.lse[so] * kLog2e;
          delta_reg[i] = a.delta[so];
          lim_reg[i] = lm;
          off_reg[i] = ro;
        } else {
          lse_reg[i] = INFINITY;  // P = exp2(-inf) = 0 for rows past the task
          delta_reg[i] = 0.f;
          lim_reg[i] = 0x7fffffff;
          off_reg[i] = -1;
        }
      }
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int r = ld_row + 16 * i;
      *reinterpret_cast<u32x4 *>(lds + L::kQs + r * kPitch + ld_col * 16) = qreg[i];
      *reinterpret_cast<u32x4 *>(lds + L::kDOs + r * kPitch + ld_col * 16) = doreg[i];
      if (ld_col == 0) {
        reinterpret_cast<float *>(lds + L::kLse)[r] = lse_reg[i];
        reinterpret_cast<float *>(lds + L::kDelta)[r] = delta_reg[i];
        reinterpret_cast<int *>(lds + L::kLim)[r] = lim_reg[i];
        reinterpret_cast<int *>(lds + L::kRowOff)[r] = off_reg[i];
      }
    }
  };

  const float c = a.scale * kLog2e;
  // tile-independent LDS offsets
  const int a_rd = l32 * kPitch + 16 * g;  // A operand rows (Q / dO / dS), + 32*s
  const int t_rd = (4 * g + ((lane & 15) >> 2)) * kPitch + (64 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;  // transposed A
  const int kt_rd = (8 * g + ((lane & 15) >> 2)) * kPitch + (16 * wave + 64 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  const int ds_rd = l32 * L::kDsPitch + 16 * g;
  const int dq_col = 16 * wave + 64 * (l32 >> 4) + (l32 & 15);

  if (mb0 < nmb) {
    load_tile(mb0);
    store_tile();
  }
  __syncthreads();

  for (int mb = mb0; mb < nmb; ++mb) {
    const bool has_next = mb + 1 < nmb;
    if (has_next) load_tile(mb + 1);

    // ---- S = Q K^T, dP = dO V^T   (rows: queries, cols: this wave's keys)
    f32x16 sacc[MSUB][KSUB], dpacc[MSUB][KSUB];
#pragma unroll
    for (int m = 0; m < MSUB; ++m)
#pragma unroll
      for (int kk = 0; kk < KSUB; ++kk)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sacc[m][kk][r] = 0.f;
          dpacc[m][kk][r] = 0.f;
        }
#pragma unroll
    for (int s = 0; s < 8; ++s) {
#pragma unroll
      for (int m = 0; m < MSUB; ++m) {
        const bf16x8 qa = *reinterpret_cast<const bf16x8 *>(lds + L::kQs + m * 32 * kPitch + a_rd + 32 * s);
        const bf16x8 da = *reinterpret_cast<const bf16x8 *>(lds + L::kDOs + m * 32 * kPitch + a_rd + 32 * s);
#pragma unroll
        for (int kk = 0; kk < KSUB; ++kk) {
          sacc[m][kk] = mfma32(qa, kfr[kk][s], sacc[m][kk]);
          dpacc[m][kk] = mfma32(da, vfr[kk][s], dpacc[m][kk]);
        }
      }
    }

    // ---- P and dS in registers; dS also to LDS for the dQ product
    const int lim_first = reinterpret_cast<const int *>(lds + L::kLim)[0];
    const bool need_mask = kw0 + 32 * KSUB - 1 > lim_first;
    bf16x8 pb[MSUB][KSUB][2], dsb[MSUB][KSUB][2];
#pragma unroll
    for (int m = 0; m < MSUB; ++m) {
#pragma unroll
      for (int cq = 0; cq < 4; ++cq) {
        const int qr = m * 32 + 8 * cq + 4 * g;
        const f32x4 lse4 = *reinterpret_cast<const f32x4 *>(lds + L::kLse + qr * 4);
        const f32x4 del4 = *reinterpret_cast<const f32x4 *>(lds + L::kDelta + qr * 4);
#pragma unroll
        for (int kk = 0; kk < KSUB; ++kk) {
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            const int r = 4 * cq + rr;
            float p = fast_exp2(__builtin_fmaf(sacc[m][kk][r], c, -lse4[rr]));
            if (need_mask) {
              const int lm = reinterpret_cast<const int *>(lds + L::kLim)[qr + rr];
              if (kw0 + kk * 32 + l32 > lm) p = 0.f;
            }
            const float ds = p * (dpacc[m][kk][r] - del4[rr]) * a.scale;
            sacc[m][kk][r] = p;
            dpacc[m][kk][r] = ds;
          }
        }
      }
#pragma unroll
      for (int kk = 0; kk < KSUB; ++kk) {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const int r0 = 8 * t;
          pb[m][kk][t] = cvt8(sacc[m][kk][r0], sacc[m][kk][r0 + 1], sacc[m][kk][r0 + 2], sacc[m][kk][r0 + 3], sacc[m][kk][r0 + 4],
                              sacc[m][kk][r0 + 5], sacc[m][kk][r0 + 6], sacc[m][kk][r0 + 7]);
          dsb[m][kk][t] = cvt8(dpacc[m][kk][r0], dpacc[m][kk][r0 + 1], dpacc[m][kk][r0 + 2], dpacc[m][kk][r0 + 3],
                               dpacc[m][kk][r0 + 4], dpacc[m][kk][r0 + 5], dpacc[m][kk][r0 + 6], dpacc[m][kk][r0 + 7]);
        }
        // dS[q][key] -> LDS, one bf16 per (lane, register)
        __bf16 *dsp = reinterpret_cast<__bf16 *>(lds + L::kDSs) + (wave * 32 * KSUB + kk * 32 + l32);
#pragma unroll
        for (int r = 0; r < 16; ++r) dsp[(m * 32 + acc_row(r, g)) * (L::kDsPitch / 2)] = dsb[m][kk][r >> 3][r & 7];
      }
    }

    // ---- dV^T += dO^T P,  dK^T += Q^T dS   (contraction over the query rows)
#pragma unroll
    for (int m = 0; m < MSUB; ++m) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const int off = (m * 32 + 16 * t) * kPitch + t_rd + 32 * db;
          const bf16x8 dot = cat4(lds_read_tr((const DISTCA_LDS void *)(lds + L::kDOs + off)),
                                  lds_read_tr((const DISTCA_LDS void *)(lds + L::kDOs + off + 8 * kPitch)));
          const bf16x8 qt = cat4(lds_read_tr((const DISTCA_LDS void *)(lds + L::kQs + off)),
                                 lds_read_tr((const DISTCA_LDS void *)(lds + L::kQs + off + 8 * kPitch)));
#pragma unroll
          for (int kk = 0; kk < KSUB; ++kk) {
            dvacc[kk][db] = mfma32(dot, pb[m][kk][t], dvacc[kk][db]);
            dkacc[kk][db] = mfma32(qt, dsb[m][kk][t], dkacc[kk][db]);
          }
        }
      }
    }
    __syncthreads();  // dS of every wave is in LDS; Q/dO tile no longer read

    // ---- dQ[:, this wave's 32 columns] = dS K over the workgroup's keys
    {
      f32x16 dqacc[MSUB];
#pragma unroll
      for (int m = 0; m < MSUB; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) dqacc[m][r] = 0.f;
#pragma unroll 4
      for (int kstep = 0; kstep < kBN / 16; ++kstep) {
        const uint8_t *kp = lds + L::kKs + kstep * 16 * kPitch + kt_rd;
        const bf16x8 ktf = cat4(lds_read_tr((const DISTCA_LDS void *)kp), lds_read_tr((const DISTCA_LDS void *)(kp + 4 * kPitch)));
#pragma unroll
        for (int m = 0; m < MSUB; ++m) {
          const bf16x8 dsa = *reinterpret_cast<const bf16x8 *>(lds + L::kDSs + m * 32 * L::kDsPitch + ds_rd + 32 * kstep);
          dqacc[m] = mfma32(dsa, ktf, dqacc[m]);
        }
      }
      float *dqp = a.dq_acc + qbase + dq_col;
#pragma unroll
      for (int m = 0; m < MSUB; ++m)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int ro = reinterpret_cast<const int *>(lds + L::kRowOff)[m * 32 + acc_row(r, g)];
          if (ro >= 0) unsafeAtomicAdd(dqp + (int64_t)ro * kHeadDim, dqacc[m][r]);
        }
    }
    if (has_next) store_tile();
    __syncthreads();
  }

  // ---- epilogue: dK, dV of this wave's keys (registers 4*cq..+3 of block db hold d0..d0+3)
#pragma unroll
  for (int kk = 0; kk < KSUB; ++kk) {
    const int key = kw0 + kk * 32 + l32;
    if (key < lk) {
      const int64_t off = (int64_t)(ks + key) * kv_stride + kvh * kHeadDim;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int cq = 0; cq < 4; ++cq) {
          const int d0 = 16 * db + 64 * (cq >> 1) + 8 * (cq & 1) + 4 * g;
          if (ALIAS) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
              unsafeAtomicAdd(a.dk_acc + off + d0 + rr, dkacc[kk][db][4 * cq + rr]);
              unsafeAtomicAdd(a.dv_acc + off + d0 + rr, dvacc[kk][db][4 * cq + rr]);
            }
          } else {
            *reinterpret_cast<bf16x4 *>(a.dk + off + d0) =
                cvt4(dkacc[kk][db][4 * cq], dkacc[kk][db][4 * cq + 1], dkacc[kk][db][4 * cq + 2], dkacc[kk][db][4 * cq + 3]);
            *reinterpret_cast<bf16x4 *>(a.dv + off + d0) =
                cvt4(dvacc[kk][db][4 * cq], dvacc[kk][db][4 * cq + 1], dvacc[kk][db][4 * cq + 2], dvacc[kk][db][4 * cq + 3]);
          }
        }
    }
  }
}

// delta[h][t] = sum_d dO[t][h][d] * O[t][h][d]; also clears the fp32 dQ accumulator row.
__global__ __launch_bounds__(256) void bwd_prepare_kernel(const __bf16 *__restrict__ dout, const __bf16 *__restrict__ out,
                                                         float *__restrict__ delta, float *__restrict__ dq_acc, int64_t rows,
                                                         int32_t hq, int32_t total_q) {
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int sub = threadIdx.x & 15;
  float s = 0.f;
  if (row < rows) {
    const bf16x8 a = *reinterpret_cast<const bf16x8 *>(dout + row * kHeadDim + sub * 8);
    const bf16x8 b = *reinterpret_cast<const bf16x8 *>(out + row * kHeadDim + sub * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) s += (float)a[i] * (float)b[i];
    f32x4 z = {0.f, 0.f, 0.f, 0.f};
    *reinterpret_cast<f32x4 *>(dq_acc + row * kHeadDim + sub * 8) = z;
    *reinterpret_cast<f32x4 *>(dq_acc + row * kHeadDim + sub * 8 + 4) = z;
  }
#pragma unroll
  for (int o = 8; o >= 1; o >>= 1) s += __shfl_xor(s, o, 64);
  if (row < rows && sub == 0) {
    const int64_t t = row / hq;
    const int h = (int)(row - t * hq);
    delta[(int64_t)h * total_q + t] = s;
  }
}

__global__ __launch_bounds__(256) void fill_zero_kernel(u32x4 *__restrict__ p, int64_t nvec) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < nvec; i += stride) p[i] = u32x4{0, 0, 0, 0};
}

// fp32 accumulator -> bf16, 8 elements per thread
__global__ __launch_bounds__(256) void cvt_bf16_kernel(const float *__restrict__ src, __bf16 *__restrict__ dst, int64_t n8) {
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i < n8; i += stride) {
    const f32x4 x = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + 2 * i);
    const f32x4 y = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src) + 2 * i + 1);
    reinterpret_cast<bf16x8 *>(dst)[i] = cvt8(x[0], x[1], x[2], x[3], y[0], y[1], y[2], y[3]);
  }
}

struct BwdWorkspace {
  int64_t sched, delta, dq_acc, dk_acc, dv_acc, total;
};
BwdWorkspace bwd_layout(const distca_ca_params *p, bool alias) {
  BwdWorkspace w;
  int64_t o = 0;
  w.sched = o; o += align_up(sched_bytes(p->num_tasks, bwd_max_items(p)), 256);
  w.delta = o; o += align_up((int64_t)p->num_heads_q * p->total_q * 4, 256);
  w.dq_acc = o; o += align_up((int64_t)p->total_q * p->num_heads_q * kHeadDim * 4, 256);
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
  int rc = validate_params(p);
  if (rc) return rc;
  if (p->deterministic)
    return fail(DISTCA_E_UNSUPPORTED, "ca_bwd: deterministic=1 is not available (dQ is accumulated with float atomics)");
  if (!dout || !q || !k || !v || !out || !lse || !dq || !dk || !dv || !cu_q || !cu_k) {
    if (p->num_tasks == 0 || p->total_q == 0) return DISTCA_OK;
    return fail(DISTCA_E_INVALID, "ca_bwd: null pointer");
  }
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(out) || !aligned16(dout) || !aligned16(dq) || !aligned16(dk) || !aligned16(dv))
    return fail(DISTCA_E_INVALID, "ca_bwd: tensors must be 16-byte aligned");
  const bool alias = kv_off != nullptr;
  const BwdWorkspace w = bwd_layout(p, alias);
  if (!workspace || workspace_bytes < w.total)
    return fail(DISTCA_E_WORKSPACE, "ca_bwd: workspace %lld B < required %lld B", (long long)workspace_bytes, (long long)w.total);
  if (!aligned16(workspace)) return fail(DISTCA_E_INVALID, "ca_bwd: workspace must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  uint8_t *ws = (uint8_t *)workspace;
  const int64_t kv_elems = (int64_t)p->total_k * p->num_heads_kv * kHeadDim;
  const int64_t q_elems = (int64_t)p->total_q * p->num_heads_q * kHeadDim;

  // dk/dv rows no task reads must come back as zero
  if (kv_elems > 0) {
    if (alias) {
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 2)), dim3(256), 0, s, (u32x4 *)(ws + w.dk_acc),
                         (w.total - w.dk_acc) / 16);
    } else {
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (u32x4 *)dk, kv_elems / 8);
      hipLaunchKernelGGL(fill_zero_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (u32x4 *)dv, kv_elems / 8);
    }
  }
  if (p->num_tasks == 0 || p->total_q == 0) return check_launch("ca_bwd(clear)");

  const SchedGeom geom = bwd_geom(p);
  const int64_t max_items = bwd_max_items(p);
  rc = launch_build_schedule(1, cu_q, cu_k, p->num_tasks, geom, (int32_t *)(ws + w.sched), max_items, s);
  if (rc) return rc;

  const int64_t rows = (int64_t)p->total_q * p->num_heads_q;
  hipLaunchKernelGGL(bwd_prepare_kernel, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, s, (const __bf16 *)dout,
                     (const __bf16 *)out, (float *)(ws + w.delta), (float *)(ws + w.dq_acc), rows, p->num_heads_q, p->total_q);

  BwdArgs a;
  a.q = (const __bf16 *)q; a.k = (const __bf16 *)k; a.v = (const __bf16 *)v; a.dout = (const __bf16 *)dout;
  a.lse = lse; a.delta = (const float *)(ws + w.delta); a.dq_acc = (float *)(ws + w.dq_acc);
  a.dk = (__bf16 *)dk; a.dv = (__bf16 *)dv;
  a.dk_acc = alias ? (float *)(ws + w.dk_acc) : nullptr;
  a.dv_acc = alias ? (float *)(ws + w.dv_acc) : nullptr;
  a.cu_q = cu_q; a.cu_k = cu_k; a.kv_off = kv_off;
  a.sched = (const int32_t *)(ws + w.sched);
  a.sched_items_off = (int32_t)sched_header_ints(p->num_tasks);
  a.hq = p->num_heads_q; a.hkv = p->num_heads_kv; a.group = p->num_heads_q / p->num_heads_kv;
  a.total_q = p->total_q; a.causal = p->causal != 0; a.scale = p->softmax_scale;
  const int64_t grid = max_items * p->num_heads_kv;
  if (grid > 0x7fffffff) return fail(DISTCA_E_INVALID, "ca_bwd: grid too large");
  using L = BwdLds<kBwdKsub, kBwdMsub>;
  static bool attr_set = false;
  if (!attr_set) {
    hipError_t e1 = hipFuncSetAttribute((const void *)ca_bwd_kernel<kBwdKsub, kBwdMsub, false>, hipFuncAttributeMaxDynamicSharedMemorySize, L::kTotal);
    hipError_t e2 = hipFuncSetAttribute((const void *)ca_bwd_kernel<kBwdKsub, kBwdMsub, true>, hipFuncAttributeMaxDynamicSharedMemorySize, L::kTotal);
    if (e1 != hipSuccess || e2 != hipSuccess) return fail(DISTCA_E_LAUNCH, "ca_bwd: cannot reserve %d B of LDS", L::kTotal);
    attr_set = true;
  }
  {
    ScopedTimer timer(DISTCA_TIMER_CA_BWD, s);
    if (alias)
      hipLaunchKernelGGL((ca_bwd_kernel<kBwdKsub, kBwdMsub, true>), dim3((unsigned)grid), dim3(256), L::kTotal, s, a);
    else
      hipLaunchKernelGGL((ca_bwd_kernel<kBwdKsub, kBwdMsub, false>), dim3((unsigned)grid), dim3(256), L::kTotal, s, a);
  }

  hipLaunchKernelGGL(cvt_bf16_kernel, dim3(grid_for(q_elems / 8)), dim3(256), 0, s, (const float *)(ws + w.dq_acc), (__bf16 *)dq, q_elems / 8);
  if (alias) {
    hipLaunchKernelGGL(cvt_bf16_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (const float *)(ws + w.dk_acc), (__bf16 *)dk, kv_elems / 8);
    hipLaunchKernelGGL(cvt_bf16_kernel, dim3(grid_for(kv_elems / 8)), dim3(256), 0, s, (const float *)(ws + w.dv_acc), (__bf16 *)dv, kv_elems / 8);
  }
  return check_launch("ca_bwd");
}
