// dK / dV of the varlen causal attention backward for gfx950, 64 keys per wave.
//
// One workgroup of 4 waves per (task, block of 256 keys, kv head), one wave per SIMD, so that a wave may use the
// SIMD's whole register file: the dK^T / dV^T accumulators of its 64 keys (2 key blocks x 4 blocks over d x 2
// matrices x 16 registers) fill the 256 accumulation registers, K of its keys stays in 64 vector registers as MFMA
// B operand, V of the workgroup's keys in LDS (and, as far as registers allow, in registers too: kVRegSlices*).  The query side (Q, dO and the row statistics of every head of the
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
// Of the eight 16-element slices over d of a wave's V rows, the first kVRegSlices* stay in registers as B operands
// beside K (as many as fit without spills inside the block loops: 12 fewer of a block's 72 LDS reads, -2 %); the
// rest is read from LDS every block.
#ifndef DISTCA_VREG_OWN
#define DISTCA_VREG_OWN 6
#endif
constexpr int kVRegSlicesOwn = DISTCA_VREG_OWN;  // the (task, key block) form
#ifndef DISTCA_VREG_SHARED
#define DISTCA_VREG_SHARED 4
#endif
constexpr int kVRegSlicesShared = DISTCA_VREG_SHARED;  // the form with a loop over a group's tasks, which has more values to hold
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
// so does not space its result from the vector instructions that read it (an eight-pass MFMA: 11 quad-cycles from
// its issue): the order of a block's instructions below, held in place by the scheduling fences, keeps between every
// such MFMA and the first read of its result either two later MFMAs, or one later MFMA (which cannot start before
// the pipe has finished the eight passes of the one in question) and at least four vector instructions.  Nowhere is
// a single MFMA the only separation; a change to the block body has to keep that.
__device__ __forceinline__ void mfma32_v(f32x16 &acc, elemx8 a, elemx8 b) {
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_v0(f32x16 &acc, elemx8 a, elemx8 b) {  // acc = A B
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma32_vc(f32x16 &acc, elemx8 a, elemx8 b, const f32x16 &c0) {  // acc = A B + c0
  asm volatile(DISTCA_MFMA32_ASM " %0, %1, %2, %3" : "=&v"(acc) : "v"(a), "v"(b), "v"(c0));
}

#define DKDV_SHARED 0
#define DKDV_SEG 0
#include "attn_bwd_dkdv64_kernel.inc"
#undef DKDV_SHARED
#define DKDV_SHARED 1
#include "attn_bwd_dkdv64_kernel.inc"
#undef DKDV_SEG
#define DKDV_SEG 1
#include "attn_bwd_dkdv64_kernel.inc"
#undef DKDV_SHARED
#undef DKDV_SEG

}  // namespace

#ifndef DISTCA_F16
int dkdv64_lds_bytes() { return kLds; }
#endif

int DISTCA_FN(launch_dkdv64)(const BwdArgs &a, int64_t grid, bool atomic_sums, bool shared, hipStream_t stream) {
  if (device_setup_pending(kSlotBwdLds64)) {
    hipError_t e1 = hipFuncSetAttribute((const void *)ca_bwd_dkdv64_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    hipError_t e2 = hipFuncSetAttribute((const void *)ca_bwd_dkdv64_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    hipError_t e3 = hipFuncSetAttribute((const void *)ca_bwd_dkdv64_shared_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e3 == hipSuccess) e3 = hipFuncSetAttribute((const void *)ca_bwd_dkdv64_shards_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
    if (e1 != hipSuccess || e2 != hipSuccess || e3 != hipSuccess) return fail(DISTCA_E_LAUNCH, "ca_bwd: cannot reserve %d B of LDS", kLds);
    device_setup_done(kSlotBwdLds64);
  }
  if (shared && atomic_sums) return fail(DISTCA_E_INVALID, "ca_bwd: items over groups of tasks are never cut into pieces");
  if (a.shards.num_shards > 0 && !shared) return fail(DISTCA_E_INVALID, "ca_bwd: K/V shards in place need tasks over shared stored rows");
  if (shared && a.shards.num_shards > 0)
    hipLaunchKernelGGL(ca_bwd_dkdv64_shards_kernel, dim3((unsigned)grid), dim3(kThreads), kLds, stream, a);
  else if (shared)
    hipLaunchKernelGGL(ca_bwd_dkdv64_shared_kernel, dim3((unsigned)grid), dim3(kThreads), kLds, stream, a);
  else if (atomic_sums)
    hipLaunchKernelGGL((ca_bwd_dkdv64_kernel<true>), dim3((unsigned)grid), dim3(kThreads), kLds, stream, a);
  else
    hipLaunchKernelGGL((ca_bwd_dkdv64_kernel<false>), dim3((unsigned)grid), dim3(kThreads), kLds, stream, a);
  return DISTCA_OK;
}

}  // namespace distca
