// fa2a shard pack / unpack and duplicate-gradient accumulation for gfx950.
//
// Behaviour follows the three kernels of the reference's csrc/core/memcpy.cu
// (memcpy_nvshmem_non_cp :22-74, memcpy_nvshmem_cp :77-155, inplace_grad_sum_kernel
// :158-236); the decomposition does not.  A shard is contiguous on both sides (rows
// start_s.. of the tensor, bytes offset_s.. of the buffer), so the job is a list of
// contiguous segment copies.  The logical token range is cut into one equal slice per
// workgroup; a workgroup locates the shard holding its first token with a block-wide
// prefix scan of the shard lengths, then walks shards, streaming 16-byte vectors with
// non-temporal loads and stores (the data is touched once, keeping it out of L2 leaves
// the cache to whoever runs next).
#include "api_util.h"
#include "common.h"

namespace distca {
namespace {

// What a plain 3 GiB device-to-device copy reaches on this part, by shape of the kernel (HBM peak 8 TB/s): 1024-thread
// workgroups over contiguous slices with 4 vectors per lane in flight 69.7 %, with 8 in flight 73 %; 512- and
// 256-thread workgroups 65-70 %; plain instead of non-temporal loads or stores 66-67 %; hipMemcpyDtoD 59 %.  Best is a
// workgroup that issues every load of its slice before its first store and then ends (one loop round per slice):
// 75-76 %; each further round of the same workgroup costs 2-4 %, and a slice that ends in a round of fewer vectors
// loses more (16 in flight over a slice of one and a half rounds: 68 %).  So a slice is one round where tokens
// allow, and the last, partial round of a run inside a shard is issued like a whole one with the lanes past the end
// switched off.  On the 262 144-token q/k/v workload, one launch for the three tensors: 10 vectors per lane
// (160 KiB slices) 75.4 / 75.3 % packing / unpacking, 16 (256 KiB) 75.0 / 75.5 %, 8 in three rounds 70.7 / 71.7 %,
// 20 or 24 in one round 73 %, 32 in one round 65 %.
constexpr int kPackThreads = 1024;
constexpr int kPackWaves = kPackThreads / 64;
#ifndef DISTCA_PACK_UNROLL
#define DISTCA_PACK_UNROLL 10
#endif
#ifndef DISTCA_PACK_SLICE_ROUNDS
#define DISTCA_PACK_SLICE_ROUNDS 1
#endif
constexpr int kUnroll = DISTCA_PACK_UNROLL;
constexpr int64_t kRoundBytes = (int64_t)kUnroll * kPackThreads * 16;  // bytes a workgroup moves per loop round

// Inclusive block scan of one int64 per thread.
__device__ __forceinline__ int64_t block_inclusive_scan(int64_t v, int64_t *lds_wave_sums) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    int64_t o = __shfl_up(v, off, 64);
    if (lane >= off) v += o;
  }
  __syncthreads();  // protect lds_wave_sums from the previous round's readers
  if (lane == 63) lds_wave_sums[wave] = v;
  __syncthreads();
  int64_t base = 0;
  for (int w = 0; w < wave; ++w) base += lds_wave_sums[w];
  return v + base;
}

struct Cursor {
  int64_t seg;        // shard index s in [0, num_seq)
  int64_t seg_start;  // first token of shard s inside one pass over the shard list
  int64_t total;      // sum of all shard lengths
};

// Finds the shard containing position `pos` (0 <= pos < total) of the concatenated
// shard list, and the total length.  All threads return the same values.
__device__ Cursor locate(const int64_t *__restrict__ seq_tokens, int64_t num_seq, int64_t pos, bool need_total,
                         int64_t *lds_scratch /* >= kPackWaves + 2 int64 */) {
  int64_t *wave_sums = lds_scratch;               // kPackWaves
  int64_t *found = lds_scratch + kPackWaves;      // [seg, seg_start]
  int64_t running = 0;
  if (threadIdx.x == 0) { found[0] = num_seq; found[1] = 0; }
  for (int64_t c0 = 0; c0 < num_seq; c0 += kPackThreads) {
    const int64_t i = c0 + threadIdx.x;
    const int64_t len = (i < num_seq) ? seq_tokens[i] : 0;
    const int64_t incl = running + block_inclusive_scan(len, wave_sums);
    if (len > 0 && incl - len <= pos && pos < incl) { found[0] = i; found[1] = incl - len; }
    __syncthreads();
    // the last thread holds the chunk total
    if (threadIdx.x == kPackThreads - 1) wave_sums[0] = incl;
    __syncthreads();
    running = wave_sums[0];
    __syncthreads();
    if (!need_total && found[0] < num_seq) break;  // uniform: found[] is in LDS
  }
  Cursor c;
  c.seg = found[0];
  c.seg_start = found[1];
  c.total = running;
  return c;
}

template <bool STORE_NT>
__device__ __forceinline__ void copy_bytes(uint8_t *__restrict__ dst, const uint8_t *__restrict__ src, int64_t bytes) {
  const int64_t nvec = bytes >> 4;
  const u32x4 *s = reinterpret_cast<const u32x4 *>(src);
  u32x4 *d = reinterpret_cast<u32x4 *>(dst);
  int64_t i = threadIdx.x;
  for (; i + (kUnroll - 1) * kPackThreads < nvec; i += kUnroll * kPackThreads) {
    u32x4 r[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) r[u] = __builtin_nontemporal_load(s + i + u * kPackThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      if (STORE_NT) __builtin_nontemporal_store(r[u], d + i + u * kPackThreads);
      else d[i + u * kPackThreads] = r[u];
    }
  }
  if (i < nvec) {
    // the last, partial round: every load is issued before the first store, as in a whole round
    u32x4 r[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (i + u * kPackThreads < nvec) r[u] = __builtin_nontemporal_load(s + i + u * kPackThreads);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u)
      if (i + u * kPackThreads < nvec) {
        if (STORE_NT) __builtin_nontemporal_store(r[u], d + i + u * kPackThreads);
        else d[i + u * kPackThreads] = r[u];
      }
  }
}

// One kernel for the plain and the replicating ("cp") form.
//   plain: logical token L in [0, num_tokens) is row L of the tensor; shard list walked once.
//   cp:    logical token L in [0, num_tokens*max_cp); the shard list is walked max_cp times,
//          pass c covering replica c.  Packing reads row L % num_tokens, unpacking writes row L.
template <bool TO_BUF, bool CP>
__device__ __forceinline__ void pack_slice(uint8_t *__restrict__ tensor, uint8_t *__restrict__ buffer,
                                           const int64_t *__restrict__ seq_offset, const int64_t *__restrict__ seq_tokens,
                                           const int8_t *__restrict__ mask, int64_t num_seq, int64_t token_bytes,
                                           int64_t num_tokens, int32_t max_cp, int64_t t0, int64_t t1, int64_t *lds_scratch) {
  int64_t cp = 0, pos = t0, total = 0;
  if (CP) {
    Cursor c = locate(seq_tokens, num_seq, 0, true, lds_scratch);
    total = c.total;
    if (total <= 0) return;
    cp = t0 / total;
    if (cp >= max_cp) return;  // a tensor with more rows than the shards add up to: the slices past the last replica own nothing
    pos = t0 - cp * total;
    __syncthreads();
  }
  Cursor cur = locate(seq_tokens, num_seq, pos, false, lds_scratch);
  if (cur.seg >= num_seq) return;  // t0 lies beyond the last shard
  int64_t seg = cur.seg;
  int64_t seg_start = cp * total + cur.seg_start;  // logical start of (cp, seg)

  while (seg_start < t1) {
    const int64_t len = seq_tokens[seg];
    const int64_t seg_end = seg_start + len;
    bool live;
    if (CP) live = mask[seg * max_cp + cp] != 0;
    else live = (!TO_BUF || mask == nullptr) ? true : (mask[seg] != 0);
    const int64_t a = seg_start > t0 ? seg_start : t0;
    const int64_t b = seg_end < t1 ? seg_end : t1;
    if (live && a < b) {
      const int64_t off = CP ? seq_offset[cp * num_seq + seg] : seq_offset[seg];
      uint8_t *buf = buffer + off + (a - seg_start) * token_bytes;
      if (CP && TO_BUF) {
        // source rows wrap modulo num_tokens
        int64_t n = b - a, lg = a;
        while (n > 0) {
          const int64_t row = lg % num_tokens;
          int64_t run = num_tokens - row;
          if (run > n) run = n;
          copy_bytes<true>(buf, tensor + row * token_bytes, run * token_bytes);
          buf += run * token_bytes;
          lg += run;
          n -= run;
        }
      } else {
        uint8_t *ten = tensor + a * token_bytes;
        if (TO_BUF) copy_bytes<true>(buf, ten, (b - a) * token_bytes);
        else copy_bytes<true>(ten, buf, (b - a) * token_bytes);
      }
    }
    seg_start = seg_end;
    if (++seg == num_seq) {
      if (!CP) break;
      seg = 0;
      if (++cp >= max_cp) break;
    }
  }
}

// One kernel for the plain and the replicating ("cp") form.
//   plain: logical token L in [0, num_tokens) is row L of the tensor; shard list walked once.
//   cp:    logical token L in [0, num_tokens*max_cp); the shard list is walked max_cp times,
//          pass c covering replica c.  Packing reads row L % num_tokens, unpacking writes row L.
template <bool TO_BUF, bool CP>
__global__ __launch_bounds__(kPackThreads) void pack_kernel(
    uint8_t *__restrict__ tensor, uint8_t *__restrict__ buffer, const int64_t *__restrict__ seq_offset,
    const int64_t *__restrict__ seq_tokens, const int8_t *__restrict__ mask, int64_t num_seq, int64_t token_bytes,
    int64_t num_tokens, int32_t max_cp, int64_t tokens_per_wg) {
  __shared__ int64_t lds_scratch[kPackWaves + 2];
  const int64_t logical_tokens = CP ? num_tokens * max_cp : num_tokens;
  int64_t t0 = (int64_t)blockIdx.x * tokens_per_wg;
  int64_t t1 = t0 + tokens_per_wg;
  if (t1 > logical_tokens) t1 = logical_tokens;
  if (t0 >= t1) return;
  pack_slice<TO_BUF, CP>(tensor, buffer, seq_offset, seq_tokens, mask, num_seq, token_bytes, num_tokens, max_cp, t0, t1, lds_scratch);
}

// Several tensors against one buffer in one launch (the q, k and v of a tick): workgroups [first_wg, first_wg of the
// next job) serve job j.  One launch has one tail instead of three, and the small tensors' slices fill the gaps
// the large one leaves.
constexpr int kMaxPackJobs = DISTCA_PACK_MAX_JOBS;
struct PackJob {
  uint8_t *tensor;
  const int64_t *seq_offset, *seq_tokens;
  const int8_t *mask;
  int64_t num_seq, token_bytes, num_tokens, tokens_per_wg;
  int32_t first_wg;
};
struct PackJobs {
  PackJob job[kMaxPackJobs];
  int32_t n;
};
template <bool TO_BUF>
__global__ __launch_bounds__(kPackThreads) void pack_multi_kernel(PackJobs jobs, uint8_t *__restrict__ buffer) {
  __shared__ int64_t lds_scratch[kPackWaves + 2];
  int j = 0;
#pragma unroll
  for (int i = 1; i < kMaxPackJobs; ++i)
    if (i < jobs.n && (int)blockIdx.x >= jobs.job[i].first_wg) j = i;
  const PackJob &jb = jobs.job[j];
  int64_t t0 = (int64_t)((int)blockIdx.x - jb.first_wg) * jb.tokens_per_wg;
  int64_t t1 = t0 + jb.tokens_per_wg;
  if (t1 > jb.num_tokens) t1 = jb.num_tokens;
  if (t0 >= t1) return;
  pack_slice<TO_BUF, false>(jb.tensor, buffer, jb.seq_offset, jb.seq_tokens, TO_BUF ? jb.mask : nullptr, jb.num_seq, jb.token_bytes,
                            jb.num_tokens, 1, t0, t1, lds_scratch);
}

template <typename T>
struct Add;
template <>
struct Add<float> {
  static __device__ __forceinline__ u32x4 apply(u32x4 a, u32x4 b) {
    f32x4 x = __builtin_bit_cast(f32x4, a), y = __builtin_bit_cast(f32x4, b);
    f32x4 r = {x[0] + y[0], x[1] + y[1], x[2] + y[2], x[3] + y[3]};
    return __builtin_bit_cast(u32x4, r);
  }
};
template <>
struct Add<_Float16> {
  typedef _Float16 h8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ u32x4 apply(u32x4 a, u32x4 b) {
    h8 x = __builtin_bit_cast(h8, a), y = __builtin_bit_cast(h8, b);
    h8 r;
#pragma unroll
    for (int i = 0; i < 8; ++i) r[i] = x[i] + y[i];
    return __builtin_bit_cast(u32x4, r);
  }
};
template <>
struct Add<__bf16> {
  // bf16 + bf16: exact in fp32 up to one rounding that never lands on a bf16 tie, so
  // fp32 add followed by round-to-nearest-even equals the correctly rounded bf16 sum.
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  static __device__ __forceinline__ u32x4 apply(u32x4 a, u32x4 b) {
    bf16x8 x = __builtin_bit_cast(bf16x8, a), y = __builtin_bit_cast(bf16x8, b);
    f32x8 fx = __builtin_convertvector(x, f32x8), fy = __builtin_convertvector(y, f32x8);
    f32x8 s;
#pragma unroll
    for (int i = 0; i < 8; ++i) s[i] = fx[i] + fy[i];
    return __builtin_bit_cast(u32x4, __builtin_convertvector(s, bf16x8));
  }
};

// data[start_s + t] += data[copy_start_id[s][c] + t] for c = 0..num_copies[s]-1 in order,
// one rounding per addition.  Rows are cut into per-workgroup slices like pack_kernel.
template <typename T>
__global__ __launch_bounds__(kPackThreads) void grad_sum_kernel(T *__restrict__ data, const int32_t *__restrict__ num_copies,
                                                              const int64_t *__restrict__ copy_start_id,
                                                              const int64_t *__restrict__ seq_lens, int64_t num_tokens,
                                                              int64_t hidden, int64_t num_seq, int64_t max_copies,
                                                              int64_t tokens_per_wg) {
  __shared__ int64_t lds_scratch[kPackWaves + 2];
  int64_t t0 = (int64_t)blockIdx.x * tokens_per_wg;
  int64_t t1 = t0 + tokens_per_wg;
  if (t1 > num_tokens) t1 = num_tokens;
  if (t0 >= t1) return;
  Cursor cur = locate(seq_lens, num_seq, t0, false, lds_scratch);
  if (cur.seg >= num_seq) return;
  int64_t seg = cur.seg, seg_start = cur.seg_start;
  constexpr int kPerVec = 16 / sizeof(T);
  const int64_t row_vecs = hidden / kPerVec;        // vector part of a row
  const int64_t row_tail = hidden - row_vecs * kPerVec;
  while (seg_start < t1 && seg < num_seq) {
    const int64_t len = seq_lens[seg];
    const int64_t seg_end = seg_start + len;
    const int32_t nc = num_copies[seg];
    const int64_t a = seg_start > t0 ? seg_start : t0;
    const int64_t b = seg_end < t1 ? seg_end : t1;
    if (nc > 0 && a < b) {
      const int64_t *starts = copy_start_id + seg * max_copies;
      if (row_tail == 0 && ((hidden * sizeof(T)) & 15) == 0) {
        // rows are whole 16-byte vectors and contiguous: treat [a,b) as one vector run
        const int64_t nvec = (b - a) * row_vecs;
        u32x4 *main_p = reinterpret_cast<u32x4 *>(data + a * hidden);
        for (int64_t i = threadIdx.x; i < nvec; i += kPackThreads) {
          u32x4 m = main_p[i];
          for (int32_t c = 0; c < nc; ++c) {
            const u32x4 *cp = reinterpret_cast<const u32x4 *>(data + (starts[c] + (a - seg_start)) * hidden);
            m = Add<T>::apply(m, __builtin_nontemporal_load(cp + i));
          }
          main_p[i] = m;
        }
      } else {
        const int64_t n = (b - a) * hidden;
        T *main_p = data + a * hidden;
        for (int64_t i = threadIdx.x; i < n; i += kPackThreads) {
          T m = main_p[i];
          for (int32_t c = 0; c < nc; ++c) m = (T)(m + data[(starts[c] + (a - seg_start)) * hidden + i]);
          main_p[i] = m;
        }
      }
    }
    seg_start = seg_end;
    ++seg;
  }
}

// Tokens per workgroup slice: kSliceRounds loop rounds (one: 160 KiB at 10 vectors per lane), rounded to whole
// tokens; never below one round.
constexpr int kSliceRounds = DISTCA_PACK_SLICE_ROUNDS;
int64_t slice_tokens(int64_t logical_tokens, int64_t token_bytes, int *grid) {
  int64_t bytes = kSliceRounds * kRoundBytes;
  const int64_t total = logical_tokens * token_bytes, want = (int64_t)num_compute_units() * 4;
  while (bytes > kRoundBytes && total / bytes < want) bytes -= kRoundBytes;
  int64_t per = (bytes + token_bytes / 2) / token_bytes;
  if (per < 1) per = 1;
  const int64_t g = (logical_tokens + per - 1) / per;
  *grid = (int)(g < 0x7fffffff ? g : 0x7fffffff);
  return per;
}

}  // namespace
}  // namespace distca

using namespace distca;

extern "C" int distca_memcpy_non_cp(void *tensor, void *buffer, const int64_t *seq_offset, const int64_t *seq_tokens,
                                    const int8_t *copy_seq_mask, int64_t num_seq, int64_t token_bytes, int64_t num_tokens,
                                    int to_buffer, void *stream) {
  if (num_seq < 0 || num_tokens < 0 || token_bytes < 0) return fail(DISTCA_E_INVALID, "memcpy_non_cp: negative size");
  if (num_tokens == 0 || num_seq == 0 || token_bytes == 0) return DISTCA_OK;
  if (!tensor || !buffer || !seq_offset || !seq_tokens) return fail(DISTCA_E_INVALID, "memcpy_non_cp: null pointer");
  if (token_bytes % 16) return fail(DISTCA_E_INVALID, "memcpy_non_cp: token_bytes=%lld is not a multiple of 16", (long long)token_bytes);
  if (!aligned16(tensor) || !aligned16(buffer)) return fail(DISTCA_E_INVALID, "memcpy_non_cp: tensor/buffer must be 16-byte aligned");
  if (num_tokens >= (1ll << 31)) return fail(DISTCA_E_INVALID, "memcpy_non_cp: num_tokens must be < 2^31");
  int grid;
  int64_t per = slice_tokens(num_tokens, token_bytes, &grid);
  hipStream_t s = (hipStream_t)stream;
  uint8_t *t = (uint8_t *)tensor, *b = (uint8_t *)buffer;
  ScopedTimer timer(DISTCA_TIMER_MEMCPY_NON_CP, s);
  if (to_buffer)
    hipLaunchKernelGGL((pack_kernel<true, false>), dim3(grid), dim3(kPackThreads), 0, s, t, b, seq_offset, seq_tokens,
                       copy_seq_mask, num_seq, token_bytes, num_tokens, 1, per);
  else
    hipLaunchKernelGGL((pack_kernel<false, false>), dim3(grid), dim3(kPackThreads), 0, s, t, b, seq_offset, seq_tokens,
                       (const int8_t *)nullptr, num_seq, token_bytes, num_tokens, 1, per);
  return check_launch("memcpy_non_cp");
}

extern "C" int distca_memcpy_non_cp_multi(const distca_pack_job *jobs, int32_t num_jobs, void *buffer, int to_buffer, void *stream) {
  if (num_jobs < 0 || num_jobs > kMaxPackJobs) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: %d jobs (0..%d)", num_jobs, kMaxPackJobs);
  if (num_jobs == 0) return DISTCA_OK;
  if (!jobs) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: null job list");
  PackJobs pj;
  pj.n = 0;
  int64_t wg = 0;
  for (int i = 0; i < num_jobs; ++i) {
    const distca_pack_job &in = jobs[i];
    if (in.num_seq < 0 || in.num_tokens < 0 || in.token_bytes < 0) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: job %d: negative size", i);
    if (in.num_tokens == 0 || in.num_seq == 0 || in.token_bytes == 0) continue;
    if (!in.tensor || !buffer || !in.seq_offset || !in.seq_tokens) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: job %d: null pointer", i);
    if (in.token_bytes % 16) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: job %d: token_bytes=%lld is not a multiple of 16", i, (long long)in.token_bytes);
    if (!aligned16(in.tensor) || !aligned16(buffer)) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: job %d: tensor/buffer must be 16-byte aligned", i);
    if (in.num_tokens >= (1ll << 31)) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: job %d: num_tokens must be < 2^31", i);
    PackJob &o = pj.job[pj.n++];
    int grid;
    o.tokens_per_wg = slice_tokens(in.num_tokens, in.token_bytes, &grid);
    o.tensor = (uint8_t *)in.tensor;
    o.seq_offset = in.seq_offset;
    o.seq_tokens = in.seq_tokens;
    o.mask = in.copy_seq_mask;
    o.num_seq = in.num_seq;
    o.token_bytes = in.token_bytes;
    o.num_tokens = in.num_tokens;
    o.first_wg = (int32_t)wg;
    wg += grid;
    if (wg > 0x7fffffff) return fail(DISTCA_E_INVALID, "memcpy_non_cp_multi: grid too large");
  }
  if (pj.n == 0) return DISTCA_OK;
  hipStream_t s = (hipStream_t)stream;
  ScopedTimer timer(DISTCA_TIMER_MEMCPY_NON_CP, s);
  if (to_buffer) hipLaunchKernelGGL((pack_multi_kernel<true>), dim3((unsigned)wg), dim3(kPackThreads), 0, s, pj, (uint8_t *)buffer);
  else hipLaunchKernelGGL((pack_multi_kernel<false>), dim3((unsigned)wg), dim3(kPackThreads), 0, s, pj, (uint8_t *)buffer);
  return check_launch("memcpy_non_cp_multi");
}

extern "C" int distca_memcpy_cp(void *tensor, void *buffer, const int8_t *do_shard, const int64_t *seq_offset,
                                const int64_t *seq_tokens, int64_t token_bytes, int64_t num_tokens, int32_t max_cp,
                                int64_t num_seq, int to_buffer, void *stream) {
  if (num_seq < 0 || num_tokens < 0 || token_bytes < 0 || max_cp < 0) return fail(DISTCA_E_INVALID, "memcpy_cp: negative size");
  if (num_tokens == 0 || num_seq == 0 || token_bytes == 0 || max_cp == 0) return DISTCA_OK;
  if (!tensor || !buffer || !seq_offset || !seq_tokens || !do_shard) return fail(DISTCA_E_INVALID, "memcpy_cp: null pointer");
  if (token_bytes % 16) return fail(DISTCA_E_INVALID, "memcpy_cp: token_bytes=%lld is not a multiple of 16", (long long)token_bytes);
  if (!aligned16(tensor) || !aligned16(buffer)) return fail(DISTCA_E_INVALID, "memcpy_cp: tensor/buffer must be 16-byte aligned");
  if (num_tokens * (int64_t)max_cp >= (1ll << 31)) return fail(DISTCA_E_INVALID, "memcpy_cp: num_tokens*max_cp must be < 2^31");
  int grid;
  int64_t per = slice_tokens(num_tokens * max_cp, token_bytes, &grid);
  hipStream_t s = (hipStream_t)stream;
  uint8_t *t = (uint8_t *)tensor, *b = (uint8_t *)buffer;
  ScopedTimer timer(DISTCA_TIMER_MEMCPY_CP, s);
  if (to_buffer)
    hipLaunchKernelGGL((pack_kernel<true, true>), dim3(grid), dim3(kPackThreads), 0, s, t, b, seq_offset, seq_tokens, do_shard,
                       num_seq, token_bytes, num_tokens, max_cp, per);
  else
    hipLaunchKernelGGL((pack_kernel<false, true>), dim3(grid), dim3(kPackThreads), 0, s, t, b, seq_offset, seq_tokens, do_shard,
                       num_seq, token_bytes, num_tokens, max_cp, per);
  return check_launch("memcpy_cp");
}

extern "C" int distca_grad_sum(void *data, int dtype, const int32_t *num_copies, const int64_t *copy_start_id,
                               const int64_t *seq_lens, int64_t num_tokens, int64_t hidden, int64_t num_seq,
                               int64_t max_copies, void *stream) {
  if (num_tokens < 0 || hidden < 0 || num_seq < 0 || max_copies < 0) return fail(DISTCA_E_INVALID, "grad_sum: negative size");
  if (num_tokens == 0 || hidden == 0 || num_seq == 0 || max_copies == 0) return DISTCA_OK;
  if (!data || !num_copies || !copy_start_id || !seq_lens) return fail(DISTCA_E_INVALID, "grad_sum: null pointer");
  if (!aligned16(data)) return fail(DISTCA_E_INVALID, "grad_sum: data must be 16-byte aligned");
  const int64_t esz = dtype == DISTCA_DTYPE_F32 ? 4 : 2;
  int grid;
  int64_t per = slice_tokens(num_tokens, hidden * esz, &grid);
  hipStream_t s = (hipStream_t)stream;
  ScopedTimer timer(DISTCA_TIMER_GRAD_SUM, s);
  switch (dtype) {
    case DISTCA_DTYPE_F32:
      hipLaunchKernelGGL((grad_sum_kernel<float>), dim3(grid), dim3(kPackThreads), 0, s, (float *)data, num_copies,
                         copy_start_id, seq_lens, num_tokens, hidden, num_seq, max_copies, per);
      break;
    case DISTCA_DTYPE_F16:
      hipLaunchKernelGGL((grad_sum_kernel<_Float16>), dim3(grid), dim3(kPackThreads), 0, s, (_Float16 *)data, num_copies,
                         copy_start_id, seq_lens, num_tokens, hidden, num_seq, max_copies, per);
      break;
    case DISTCA_DTYPE_BF16:
      hipLaunchKernelGGL((grad_sum_kernel<__bf16>), dim3(grid), dim3(kPackThreads), 0, s, (__bf16 *)data, num_copies,
                         copy_start_id, seq_lens, num_tokens, hidden, num_seq, max_copies, per);
      break;
    default:
      return fail(DISTCA_E_UNSUPPORTED, "grad_sum: dtype %d (only fp32, fp16, bf16)", dtype);
  }
  return check_launch("grad_sum");
}
