// Shared device helpers for the gfx950 core-attention kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace distca {

// The 16-bit element type of q, k, v, out and the gradients.  The attention sources are compiled twice: as they are
// for bf16, and with -DDISTCA_F16 for IEEE half precision; DISTCA_FN gives what they export a name per element type.
#ifdef DISTCA_F16
typedef _Float16 elem_t;
#define DISTCA_FN(name) name##_f16
#define DISTCA_MFMA32_ASM "v_mfma_f32_32x32x16_f16"
#else
typedef __bf16 elem_t;
#define DISTCA_FN(name) name
#define DISTCA_MFMA32_ASM "v_mfma_f32_32x32x16_bf16"
#endif
typedef elem_t elemx8 __attribute__((ext_vector_type(8)));
typedef elem_t elemx4 __attribute__((ext_vector_type(4)));
typedef elem_t elemx2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));

#define DISTCA_LDS __attribute__((address_space(3)))

// D = A(32x16) * B(16x32) + C on one wave64.
//   A operand: lane l holds row l%32, k = 8*(l/32) .. +7
//   B operand: lane l holds col l%32, k = 8*(l/32) .. +7
//   C/D:       lane l holds col l%32, register r holds row 8*(r/4) + 4*(l/32) + r%4
__device__ __forceinline__ f32x16 mfma32(elemx8 a, elemx8 b, f32x16 c) {
#ifdef DISTCA_F16
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
#else
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
#endif
}

// Row index (0..31) inside a 32x32 accumulator block for register r of lane-half g.
__device__ __forceinline__ constexpr int acc_row(int r, int g) { return 8 * (r >> 2) + 4 * g + (r & 3); }

// Transposing LDS read.  Within each group of 16 lanes, lane j supplies the address of
// 4 consecutive 16-bit elements; lane L of the group receives element (L%4) of the
// chunks supplied by lanes 4e + L/4, e = 0..3.  With lane j pointing at
// (row r0 + j/4, col c0 + 4*(j%4)) of a row-major tile, lane L ends up with
// column c0 + L of rows r0 .. r0+3.
// An LDS pointer from a 32-bit LDS address.
__device__ __forceinline__ const DISTCA_LDS void *lds_ptr(uint32_t addr) { return reinterpret_cast<const DISTCA_LDS void *>(static_cast<uintptr_t>(addr)); }
__device__ __forceinline__ elemx4 lds_read_tr(const DISTCA_LDS void *p) {
  s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((DISTCA_LDS s16x4 *)p);
  return __builtin_bit_cast(elemx4, v);
}

__device__ __forceinline__ elemx8 cat4(elemx4 lo, elemx4 hi) {
  return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
}

__device__ __forceinline__ elemx8 cvt8(float a0, float a1, float a2, float a3, float a4, float a5, float a6, float a7) {
  f32x8 v = {a0, a1, a2, a3, a4, a5, a6, a7};
  return __builtin_convertvector(v, elemx8);
}
__device__ __forceinline__ elemx4 cvt4(float a0, float a1, float a2, float a3) {
  f32x4 v = {a0, a1, a2, a3};
  return __builtin_convertvector(v, elemx4);
}

// max / sum of x over the lane pair (l, l^32).
__device__ __forceinline__ float pair_max(float x) { return __builtin_fmaxf(x, __shfl_xor(x, 32, 64)); }
__device__ __forceinline__ float pair_sum(float x) { return x + __shfl_xor(x, 32, 64); }

// LDS-direct global loads.  One piece per active lane goes from global memory straight into
// LDS at lds_base + piece_bytes * lane, with no staging registers.  The compiler is not told
// that these are memory operations: the caller orders them with wait_vm0() followed by a
// barrier before any wave reads the destination.  M0 is written here and used by nothing
// else in these kernels.
__device__ __forceinline__ uint32_t uniform32(uint32_t x) { return __builtin_amdgcn_readfirstlane(x); }
// Values that are the same in every lane, moved to scalar registers: what is loaded from memory counts as differing
// from lane to lane for the compiler, and so does everything computed from it (a task's bounds, its base pointers,
// loop limits), which then costs vector instructions and registers where scalar ones would do.
__device__ __forceinline__ int uniform_int(int x) { return (int)uniform32((uint32_t)x); }
__device__ __forceinline__ int64_t uniform_int64(int64_t x) {
  const uint64_t u = (uint64_t)x;
  const uint64_t hi = uniform32((uint32_t)(u >> 32)), lo = uniform32((uint32_t)u);  // (each half widened as unsigned)
  return (int64_t)((hi << 32) | lo);
}
// A pointer that is the same in every lane, moved to scalar registers.  Where the compiler cannot prove that (the value
// derives from a work item read through LDS), it keeps a vector copy, and under pressure parks that copy in scratch
// memory: the reload's wait then also waits for every LDS-direct load in flight, which it does not count as its own.
template <typename T>
__device__ __forceinline__ T *uniform_ptr(T *p) {
  const uint64_t u = reinterpret_cast<uint64_t>(p);
  const uint64_t hi = uniform32((uint32_t)(u >> 32)), lo = uniform32((uint32_t)u);
  return reinterpret_cast<T *>((hi << 32) | lo);
}
__device__ __forceinline__ void lds_direct_load16(const void *gbase, uint32_t voff, uint32_t lds_base) {
  const uint64_t gb = reinterpret_cast<uint64_t>(gbase);
  const uint64_t gbu = ((uint64_t)uniform32((uint32_t)(gb >> 32)) << 32) | uniform32((uint32_t)gb);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(voff), "s"(gbu), "s"(uniform32(lds_base)) : "memory");
}
// 16 bytes per lane from a per-lane pointer; lane L's data lands at lds_base + 16*L.
__device__ __forceinline__ void lds_direct_load16_ptr(const void *gptr_lane, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gptr_lane), "s"(uniform32(lds_base)) : "memory");
}
__device__ __forceinline__ void lds_direct_load4_base(const void *gbase, uint32_t voff, uint32_t lds_base) {
  const uint64_t gb = reinterpret_cast<uint64_t>(gbase);
  const uint64_t gbu = ((uint64_t)uniform32((uint32_t)(gb >> 32)) << 32) | uniform32((uint32_t)gb);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(voff), "s"(gbu), "s"(uniform32(lds_base)) : "memory");
}
__device__ __forceinline__ void lds_direct_load4(const void *gptr_lane, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gptr_lane), "s"(uniform32(lds_base)) : "memory");
}
__device__ __forceinline__ void wait_vm0() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// Swizzle of a row-major LDS tile with 256-byte rows (16 chunks of 16 bytes, no padding):
// chunk c of row r is stored at chunk position c ^ tile_swz(r).  With it both read shapes of
// the MFMA operands are free of bank conflicts (128-bit reads of one chunk column over 32 rows,
// and the transposing 64-bit reads over 4-row x 32-byte patches), and a row keeps its 256
// contiguous bytes, so LDS-direct loads can fill four rows per instruction.
__device__ __forceinline__ int tile_swz(int r) { return ((r & 3) << 1) | ((r & 4) << 1) | ((r >> 3) & 1); }

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

}  // namespace distca
