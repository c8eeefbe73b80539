/*
 * distca_ca.h — C ABI of the MI355X (gfx950) core-attention server library.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void* so the header needs no HIP include).  All work is enqueued
 * asynchronously on `stream`; nothing synchronises with the host and nothing
 * allocates device memory — scratch space is brought in by the caller as a
 * workspace whose size the matching *_workspace_bytes() call reports.
 *
 * Return value: 0 on success, a negative DISTCA_E_* code on a rejected call.
 * distca_last_error() returns a thread-local human readable message for the
 * last non-zero return.
 *
 * Reference interfaces replaced (paths relative to the DistCA tree):
 *   csrc/core/memcpy.h:5-47            launch_memcpy_non_cp / launch_memcpy_cp /
 *                                      launch_inplace_grad_sum<T>
 *   csrc/bindings/all_to_all.cpp:47-254 the torch-op wrappers around them
 *   distca/runtime/megatron/ops/fused_comm_attn.py:151-197,259-272
 *                                      the flash-attn varlen fwd / bwd invocation
 */
#ifndef DISTCA_CA_H_
#define DISTCA_CA_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DISTCA_OK 0
#define DISTCA_E_INVALID (-1)   /* bad argument (shape, alignment, null pointer)  */
#define DISTCA_E_UNSUPPORTED (-2) /* valid request this build has no kernel for    */
#define DISTCA_E_WORKSPACE (-3) /* workspace too small                             */
#define DISTCA_E_LAUNCH (-4)    /* HIP reported an error at launch                 */

/* element types of distca_grad_sum */
#define DISTCA_DTYPE_F32 0
#define DISTCA_DTYPE_F16 1
#define DISTCA_DTYPE_BF16 2

const char *distca_last_error(void);
/* ABI version of this header: bumped whenever a signature changes. */
int distca_abi_version(void);

/* ---------------------------------------------------------------------------
 * fa2a shard pack / unpack.
 *
 * Replaces launch_memcpy_non_cp (csrc/core/memcpy.cu:240-282; kernel :22-74) as
 * reached through fast_a2a_memcpy_non_cp[_debug] (csrc/bindings/all_to_all.cpp:
 * 47-113).  `tensor` is a contiguous [num_tokens, token_bytes] byte matrix.
 * Shard s owns rows [start_s, start_s + seq_tokens[s]) with start_s the
 * exclusive prefix sum of seq_tokens, and the byte range
 * [seq_offset[s], seq_offset[s] + seq_tokens[s]*token_bytes) of `buffer`.
 * to_buffer != 0 packs tensor -> buffer, 0 unpacks buffer -> tensor.
 * copy_seq_mask (int8 [num_seq], may be NULL) skips shards whose entry is 0;
 * like the reference it is honoured only when packing.
 * Rows at or beyond num_tokens are never touched.
 * token_bytes, seq_offset[] and both base pointers must be multiples of 16
 * (token_bytes and the pointers are checked on the host; seq_offset[] and
 * seq_tokens[] live on the device and are the caller's responsibility, as is
 * sum(seq_tokens) >= num_tokens: rows past the last shard are left alone).
 * ------------------------------------------------------------------------- */
int distca_memcpy_non_cp(void *tensor, void *buffer,
                         const int64_t *seq_offset, const int64_t *seq_tokens,
                         const int8_t *copy_seq_mask, int64_t num_seq,
                         int64_t token_bytes, int64_t num_tokens, int to_buffer,
                         void *stream);

/* Several tensors packed into / unpacked from one buffer by one launch: what the
 * reference does with consecutive launch_memcpy_non_cp calls for the q, k and v of a
 * tick (post_a2a_qkv, distca/runtime/attn_kernels/dispatch.py:60-94; pre_a2a_qkv in
 * backward, :39-56).  Each job has the meaning of one distca_memcpy_non_cp call with
 * the same fields; results are identical to making those calls one after another, the
 * jobs' byte ranges in the buffer being disjoint.  At most DISTCA_PACK_MAX_JOBS jobs;
 * jobs with no tokens are skipped. */
#define DISTCA_PACK_MAX_JOBS 4
typedef struct distca_pack_job {
  void *tensor;
  const int64_t *seq_offset;   /* device, int64 [num_seq] */
  const int64_t *seq_tokens;   /* device, int64 [num_seq] */
  const int8_t *copy_seq_mask; /* device, int8 [num_seq] or NULL; packing only */
  int64_t num_seq;
  int64_t token_bytes;
  int64_t num_tokens;
} distca_pack_job;
int distca_memcpy_non_cp_multi(const distca_pack_job *jobs, int32_t num_jobs,
                               void *buffer, int to_buffer, void *stream);

/* Replaces launch_memcpy_cp (csrc/core/memcpy.cu:285-343; kernel :77-155) as
 * reached through fast_a2a_memcpy_cp[_debug] (all_to_all.cpp:116-179,243-254).
 * Logical shard (c, s), c < max_cp, s < num_seq, is live iff
 * do_shard[s*max_cp + c] != 0 and owns buffer bytes starting at
 * seq_offset[c*num_seq + s].  Packing reads rows start_s.. of the
 * [num_tokens, token_bytes] tensor for every live replica c; unpacking writes
 * rows c*num_tokens + start_s.. of the [max_cp, num_tokens, token_bytes]
 * tensor (which the caller pre-zeroes, dispatch_fn.py:79-80).
 * seq_tokens must add up to num_tokens (the reference assumes the same,
 * memcpy.cu:96-110); slices of a larger tensor that lie past the last replica
 * are left alone.  seq_offset[] and seq_tokens[] are device arrays and are not
 * checked: 16-byte alignment of the offsets and the ranges they name are the
 * caller's responsibility, as in the reference. */
int distca_memcpy_cp(void *tensor, void *buffer, const int8_t *do_shard,
                     const int64_t *seq_offset, const int64_t *seq_tokens,
                     int64_t token_bytes, int64_t num_tokens, int32_t max_cp,
                     int64_t num_seq, int to_buffer, void *stream);

/* Replaces launch_inplace_grad_sum<T> (csrc/core/memcpy.cu:346-410; kernel
 * :158-236) as reached through fast_a2a_grad_acc (all_to_all.cpp:182-240).
 * For every shard s with num_copies[s] > 0 and every row t of it:
 *   data[start_s + t] += data[copy_start_id[s*max_copies + c] + t],
 * c = 0 .. num_copies[s]-1 in that order, each addition rounded to `dtype`. */
int distca_grad_sum(void *data, int dtype, const int32_t *num_copies,
                    const int64_t *copy_start_id, const int64_t *seq_lens,
                    int64_t num_tokens, int64_t hidden, int64_t num_seq,
                    int64_t max_copies, void *stream);

/* ---------------------------------------------------------------------------
 * Core attention over a batch of CA tasks.
 *
 * Task b: query rows q[cu_seqlens_q[b] .. cu_seqlens_q[b+1]) (Lq rows) attend
 * to key/value rows k[ks .. ks+Lk) with Lk = cu_seqlens_k[b+1]-cu_seqlens_k[b]
 * and ks = kv_task_offsets ? kv_task_offsets[b] : cu_seqlens_k[b].  With
 * kv_task_offsets, tasks that start at the same row read prefixes of one stored
 * document (the reference materialises one copy of the prefix per task,
 * compute_metadata.py:429-448); tasks that start at different rows must not
 * share rows, and ks + Lk <= total_k.  With
 * causal != 0 row i sees column j iff j <= i + (Lk - Lq) (bottom-right
 * aligned, the flash-attn 2.1+ convention the reference relies on at
 * per_doc_cp_attn.py:326,406-411).  q-head h reads kv-head h / (Hq/Hkv).
 *
 * The sizes in distca_ca_params must bound what the device arrays say, since the
 * host sizes work lists and grids from them without reading device memory:
 * cu_seqlens_q[B] <= total_q, every Lq <= max_seqlen_q, every Lk <= max_seqlen_k,
 * and, when kv_task_offsets is NULL, cu_seqlens_k[B] <= total_k.  Work beyond
 * those bounds is dropped (and counted, see distca_ca_schedule_capacity), never
 * executed out of range.
 *
 * Layouts: q,out,dout,dq [total_q, Hq, D] 16-bit elements (bf16 or fp16, by
 * distca_ca_params.dtype); k,v,dk,dv [total_k, Hkv, D] the same; lse [Hq, total_q] fp32 natural-log with the scale included;
 * cu_seqlens_* int32 [B+1]; kv_task_offsets int32 [B] or NULL.
 * D must be 128 in this build.
 *
 * These two calls stand where fused_comm_attn.py:151-197 calls
 * flash_attn's varlen forward and :259-272 its varlen backward.
 * ------------------------------------------------------------------------- */
typedef struct distca_ca_params {
  int32_t num_tasks;    /* B                                                  */
  int32_t total_q;      /* rows of q / out                                    */
  int32_t total_k;      /* rows of k / v                                      */
  int32_t num_heads_q;  /* Hq                                                 */
  int32_t num_heads_kv; /* Hkv, divides Hq                                    */
  int32_t head_dim;     /* D                                                  */
  int32_t max_seqlen_q; /* upper bound of any task's Lq                       */
  int32_t max_seqlen_k; /* upper bound of any task's Lk                       */
  float softmax_scale;  /* multiplies q.k before softmax                      */
  int32_t causal;       /* 0 / 1                                              */
  int32_t deterministic;/* backward only: 1 = use no float atomics, so that two
                           runs give the same bits (the reference's server
                           default, fused_comm_attn.py:95-104).  0 allows them
                           where they pay: a batch too small to occupy the
                           device has its key blocks cut into pieces whose
                           dK/dV are added up with atomics                    */
  int32_t dtype;        /* element type of q, k, v, out and the gradients:
                           DISTCA_DTYPE_BF16 or DISTCA_DTYPE_F16; 0 (callers
                           written before the field existed) means bf16      */
} distca_ca_params;

/* Size of the workspace an attention call needs (no reference counterpart: flash-attn
 * allocates its own).  The workspace holds the work list the call builds on the device
 * and the counters its workgroups draw their work from (and, in the backward, the row
 * statistics: 8 bytes per query row and head; fp32 dK/dV accumulators only for a small
 * batch with deterministic == 0, whose key blocks are cut into pieces); its contents are rewritten
 * by every call, so calls that may run at the same time on different streams each need
 * a workspace of their own, while calls ordered on one stream can share one.           */
int64_t distca_ca_fwd_workspace_bytes(const distca_ca_params *p);
int64_t distca_ca_bwd_workspace_bytes(const distca_ca_params *p);

int distca_ca_fwd(const void *q, const void *k, const void *v, void *out,
                  float *lse, const int32_t *cu_seqlens_q,
                  const int32_t *cu_seqlens_k, const int32_t *kv_task_offsets,
                  const distca_ca_params *p, void *workspace,
                  int64_t workspace_bytes, void *stream);

/* distca_ca_fwd for callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc) and so cannot bring a
 * workspace: the work list, zero row and ticket counters live in a static device array
 * of distca_ca_fwd_noalloc_max_bytes() (1 MiB) inside the library, one copy per GPU,
 * held until the process ends.  It has no counterpart in the reference (flash-attn
 * allocates what it needs).  Same arguments, results and error codes as distca_ca_fwd
 * without the workspace pair; a batch whose distca_ca_fwd_workspace_bytes exceeds the
 * array is rejected with DISTCA_E_WORKSPACE (1 MiB holds about 65 000 work items, i.e.
 * 16.7 million query rows x heads-per-kv-head: config 5 needs a quarter of it).  The call
 * makes no hipMalloc / hipFree and rewrites everything it reads from the array, so it
 * does not depend on what the previous call left there; every call on a GPU uses that
 * GPU's one array, so calls that overlap on one GPU (two streams, two host threads)
 * race and must be ordered by the caller. */
int64_t distca_ca_fwd_noalloc_max_bytes(void);
int distca_ca_fwd_noalloc(const void *q, const void *k, const void *v, void *out,
                          float *lse, const int32_t *cu_seqlens_q,
                          const int32_t *cu_seqlens_k,
                          const int32_t *kv_task_offsets,
                          const distca_ca_params *p, void *stream);

/* The same forward with the query and output tokens where the CA server has them
 * (distca/runtime/megatron/ops/fused_comm_attn.py:298-389 unpacks q from the
 * receive buffer, runs attention, and packs [out | lse] tokens into the send
 * buffer, attn_kernels/dispatch.py:209-221; here the kernel reads and writes
 * those tokens in place).  Token t of task b of the queries starts at
 * q_base + q_task_off[b] + t * q_tok_bytes and holds Hq*D elements; of the output at
 * out_base + out_task_off[b] + t * out_tok_bytes and receives Hq*D elements, then,
 * when lse is NULL, Hq fp32 lse values and zero padding up to the next multiple
 * of 16 bytes.  A NULL offset array means the packed tensor (offset of task b =
 * cu_seqlens_q[b] tokens, token size Hq*D*2); lse == NULL needs out_task_off.
 * Offsets are device int64 arrays of num_tasks entries, multiples of 16; token
 * sizes are multiples of 16.  Ranges are the caller's responsibility. */
int distca_ca_fwd_tokens(const void *q_base, const int64_t *q_task_off,
                         int64_t q_tok_bytes, const void *k, const void *v,
                         void *out_base, const int64_t *out_task_off,
                         int64_t out_tok_bytes, float *lse,
                         const int32_t *cu_seqlens_q,
                         const int32_t *cu_seqlens_k,
                         const int32_t *kv_task_offsets,
                         const distca_ca_params *p, void *workspace,
                         int64_t workspace_bytes, void *stream);

/* The same forward with K and V, too, read where the CA server has them: every stored
 * K/V shard lies once somewhere in the receive buffer, and instead of unpacking the
 * shards into contiguous tensors first (post_a2a_qkv,
 * distca/runtime/attn_kernels/dispatch.py:60-94) the kernel addresses a stored row
 * through the table of shards.  Stored rows [row_start[s], row_start[s+1]) are the rows
 * of shard s and lie token after token (Hkv*D elements each) from byte k_offset[s] of
 * `k` (v_offset[s] of `v`; both may be the same buffer).  kv_task_offsets (required)
 * names stored rows, p->total_k = row_start[num_shards], and task_shard[b] is the shard
 * that holds row kv_task_offsets[b].  Offsets are multiples of 16.  All arrays are
 * device arrays; the ranges they name are the caller's responsibility. */
typedef struct distca_kv_shards {
  int32_t num_shards;
  const int32_t *row_start;  /* int32 [num_shards + 1], ascending                  */
  const int64_t *k_offset;   /* int64 [num_shards]                                 */
  const int64_t *v_offset;   /* int64 [num_shards]                                 */
  const int32_t *task_shard; /* int32 [num_tasks]                                  */
  const int64_t *dk_offset;  /* backward only: where the shards' dK / dV rows go,  */
  const int64_t *dv_offset;  /* byte offsets from `dk` / `dv`                      */
} distca_kv_shards;
int distca_ca_fwd_buffers(const void *q_base, const int64_t *q_task_off,
                          int64_t q_tok_bytes, const void *k, const void *v,
                          const distca_kv_shards *kv_shards, void *out_base,
                          const int64_t *out_task_off, int64_t out_tok_bytes,
                          float *lse, const int32_t *cu_seqlens_q,
                          const int32_t *cu_seqlens_k,
                          const int32_t *kv_task_offsets,
                          const distca_ca_params *p, void *workspace,
                          int64_t workspace_bytes, void *stream);

/* dk/dv rows are written once per task when kv_task_offsets is NULL.  When it
 * is given, dk/dv of a stored row hold the sum over every task that read the
 * row (what the reference obtains with duplicated KV copies and
 * inplace_grad_sum_kernel, csrc/core/memcpy.cu:158-236): one work item per
 * (stored document, block of 256 keys) walks the query rows of every task whose
 * prefix holds the block, sums in registers and writes the rows once, so the
 * result is the same in every run whatever `deterministic` says; rows that no
 * task reads come back as zeros. */
int distca_ca_bwd(const void *dout, const void *q, const void *k, const void *v,
                  const void *out, const float *lse, void *dq, void *dk,
                  void *dv, const int32_t *cu_seqlens_q,
                  const int32_t *cu_seqlens_k, const int32_t *kv_task_offsets,
                  const distca_ca_params *p, void *workspace,
                  int64_t workspace_bytes, void *stream);

/* The same backward with the query side where the CA server has it
 * (fused_comm_attn.py:407-461 unpacks the request tokens [dO | O | lse | q | pad]
 * of attn_kernels/dispatch.py:138-206 into four tensors, runs the backward and
 * packs dq; here the kernels read the parts of each token in place and write dq
 * tokens into the send buffer).  Token t of task b of the request starts at
 * req_base + req_task_off[b] + t * req_tok_bytes and holds Hq*D elements of dO, Hq*D
 * of O, Hq fp32 lse, Hq*D elements of q; dq token t of task b starts at
 * dq_base + dq_task_off[b] + t * dq_tok_bytes.  Needs Hq % 4 == 0 (the q part must
 * stay 16-byte aligned; other head counts return DISTCA_E_UNSUPPORTED and are
 * served by distca_ca_bwd on unpacked tensors).  dk / dv as in distca_ca_bwd. */
int distca_ca_bwd_tokens(const void *req_base, const int64_t *req_task_off,
                         int64_t req_tok_bytes, const void *k, const void *v,
                         void *dq_base, const int64_t *dq_task_off,
                         int64_t dq_tok_bytes, void *dk, void *dv,
                         const int32_t *cu_seqlens_q,
                         const int32_t *cu_seqlens_k,
                         const int32_t *kv_task_offsets,
                         const distca_ca_params *p, void *workspace,
                         int64_t workspace_bytes, void *stream);

/* The backward with K and V read through the table of shards as in
 * distca_ca_fwd_buffers, and dK / dV written where the shards' gradients belong in the
 * send buffer (dk_offset[s] / dv_offset[s] from `dk` / `dv`) instead of into
 * contiguous tensors that a pack pass would copy there (pre_a2a_qkv in backward,
 * attn_kernels/dispatch.py:39-56).  Every stored row is written: rows no task reads
 * as zeros.  Key blocks are never cut into pieces in this form (no float atomics:
 * the result is the same in every run). */
int distca_ca_bwd_buffers(const void *req_base, const int64_t *req_task_off,
                          int64_t req_tok_bytes, const void *k, const void *v,
                          const distca_kv_shards *kv_shards, void *dq_base,
                          const int64_t *dq_task_off, int64_t dq_tok_bytes,
                          void *dk, void *dv, const int32_t *cu_seqlens_q,
                          const int32_t *cu_seqlens_k,
                          const int32_t *kv_task_offsets,
                          const distca_ca_params *p, void *workspace,
                          int64_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------------------
 * Tile scheduler, host mirror.  The device builds the same list inside
 * distca_ca_fwd / distca_ca_bwd; this entry point runs the identical code on
 * host arrays so the balance invariants can be tested without a GPU.
 * kind 0 = forward (one item per (task, block of query rows), cost = KV tiles
 * visible to the block), 1 = backward (one item per (task, KV block), cost =
 * query blocks that see it; when the batch has too few key blocks to occupy
 * the device and p->deterministic is 0, a key block is cut into pieces of
 * consecutive query blocks, whose dK/dV the kernel adds up in fp32).  Writes
 * up to max_items (task, block, cost, piece | pieces << 16) quadruples sorted
 * by descending cost and returns the item count, or a negative error.  In a
 * backward list bit 31 of the fourth word marks the items whose query blocks
 * the kernel walks upwards from the diagonal instead of downwards from the
 * end (alternate rounds of as many items as compute units serve a kv head, so
 * that items running side by side stream the same rows): piece = word &
 * 0xffff, pieces = (word >> 16) & 0x7fff.  The reference has no counterpart: flash-attn launches a static
 * (m-block, batch, head) grid sized by max_seqlen_q.
 * ------------------------------------------------------------------------- */
int64_t distca_ca_schedule_host(int kind, const int32_t *cu_seqlens_q,
                                const int32_t *cu_seqlens_k,
                                const distca_ca_params *p, int32_t *items,
                                int64_t max_items);
/* Number of work items the list of `kind` (0 forward, 1 backward dK/dV, 2 backward dQ)
 * has room for inside the workspace, computed from the sizes in p alone.  The device
 * builder never writes more; it counts what did not fit in word 2 of the list's header
 * (always 0 when p bounds the sequence lengths as required above).  No reference
 * counterpart. */
int64_t distca_ca_schedule_capacity(int kind, const distca_ca_params *p);
/* tile geometry used by the kernels of `kind` for the head layout in p:
 * out[0] = query rows (tokens) per block, out[1] = kv rows per block. */
int distca_ca_tile_shape(int kind, const distca_ca_params *p, int32_t out[2]);

/* ---------------------------------------------------------------------------
 * Per-kernel timing, for benchmarks.  No counterpart in the reference (which
 * wraps CUDA events around its flash-attn calls in Python,
 * tests/test_e2e_combined.py:1947-1999).  While enabled, every entry point
 * brackets its dominant kernel with HIP events recorded on the stream the
 * kernel is launched on; distca_timing_read waits for those events, returns
 * the summed duration and launch count of kernel `which` since the last read
 * and clears them.  Not thread safe; leave disabled outside benchmarks.
 * ------------------------------------------------------------------------- */
#define DISTCA_TIMER_CA_FWD 0      /* ca_fwd_kernel                          */
#define DISTCA_TIMER_CA_BWD 1      /* ca_bwd_dkdv64_kernel                   */
#define DISTCA_TIMER_MEMCPY_NON_CP 2
#define DISTCA_TIMER_MEMCPY_CP 3
#define DISTCA_TIMER_GRAD_SUM 4
#define DISTCA_TIMER_CA_BWD_DQ 5   /* ca_bwd_dq64_kernel                     */
#define DISTCA_TIMER_COUNT 6
void distca_timing_enable(int on);
int distca_timing_read(int which, double *total_ms, int64_t *launches);

/* ---------------------------------------------------------------------------
 * What the device delivers for the MFMA instruction the attention kernels are
 * made of, measured on the spot.  No counterpart in the reference: a
 * diagnostic for benchmarks, which print it beside the kernels' own rate.  One
 * wave on every SIMD issues 8 * iters v_mfma_f32_32x32x16_bf16 on pseudo-random
 * operands and, behind every MFMA, nothing (kind 0), one 1 KB LDS read (1),
 * four v_fma_f32 (2), two v_exp_f32 (3), or (4) what the attention backward has
 * beside an MFMA on average: half of a 1 KB LDS read, two v_fma_f32, half a
 * v_exp_f32 and half a v_cvt_pk_bf16_f32.  All of it fits into the MFMA's
 * shadow, so that the pipe stays fully occupied and the result shows what the
 * power limit leaves of the clock.  Returns the MFMA rate in TFLOP/s (by HIP
 * events on `stream`), the cycles per MFMA and the shader clock in GHz (by the
 * device's cycle and real-time counters).  scratch32: 32 bytes of device
 * memory.  Synchronises `stream`.
 * ------------------------------------------------------------------------- */
int distca_probe_mfma_rate(int kind, int iters, void *scratch32, double *tflops,
                           double *cycles_per_mfma, double *clock_ghz,
                           void *stream);

#ifdef __cplusplus
}
#endif
#endif /* DISTCA_CA_H_ */
