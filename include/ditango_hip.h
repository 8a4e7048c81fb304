/*
 * libditango_hip.so -- C ABI of the MI355X (gfx950) kernels behind DiTango's
 * cached block attention.
 *
 * The reference (chen-yy20/ditango) is pure Python; the GPU arithmetic of this
 * path lives in the third-party flash_attn wheel and in eager torch ops.  Each
 * entry point below replaces one of those call sites; the citation names the
 * reference interface it stands in for.  All pointers are device pointers
 * unless the comment says "host".  Every function enqueues work on `stream`
 * (a hipStream_t passed as void*), never synchronises, never allocates, and
 * returns DT_OK or a negative error code; dt_last_error() then holds a
 * message for the calling thread.
 *
 * Tensor layouts (element strides, innermost dimension contiguous):
 *   q / out state   bf16  [B, Sq, H, D]   (IEEE half instead where an entry point or a flag says so:
 *   k, v chunk      bf16  [B, Sk, H, D]    dt_attn_chunk_f16_fwd, DT_ATTN_FP16, DT_FP16, DT_IO_FP16)
 *   lse state       fp32  [B, H, Sq]     (DT_LSE_BHS, flash-attn's layout)
 *                   fp32  [B, Sq, H]     (DT_LSE_BSH, the running layout
 *                                         [B,S,H,1] of utils.py:49)
 * D is 64 or 128.  Base pointers and the q/k/v token, head and batch strides
 * must keep every row 16-byte aligned.
 */
#ifndef DITANGO_HIP_H
#define DITANGO_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DT_OK 0
#define DT_ERR_INVALID (-1)     /* bad argument (shape, alignment, null pointer, limit) */
#define DT_ERR_UNSUPPORTED (-2) /* valid request this build does not cover (e.g. head dim) */
#define DT_ERR_HIP (-3)         /* a HIP runtime call failed */

#define DT_BF16 0
#define DT_FP32 1
#define DT_FP16 2 /* IEEE binary16 */

#define DT_LSE_BHS 0
#define DT_LSE_BSH 1

#define DT_NORM_NONE 0
#define DT_NORM_RMS 1    /* x * rsqrt(mean(x^2) + eps) * weight */
#define DT_NORM_LAYER 2  /* (x - mean) * rsqrt(var + eps) * weight + bias */

#define DT_ROPE_NONE 0
#define DT_ROPE_INTERLEAVED 1 /* pairs (2i, 2i+1) rotate together */
#define DT_ROPE_HALVES 2      /* element d pairs with d +- half of its section ("rotate_half") */

#define DT_ROUND_NORM_BF16 1 /* round to bf16 where the callers' bf16 norm modules do */
#define DT_ROUND_ROPE_BF16 2 /* RoPE products and their sum each rounded to bf16 */
#define DT_IO_FP16 4         /* x and y are fp16; the two bits above then round to fp16 */

#define DT_MAX_CHUNKS 40       /* KV chunks one launch can address */
#define DT_MAX_JOBS 40         /* attention states one launch can produce */
#define DT_MAX_JOB_ENTRIES 64  /* total chunk references over all jobs of a launch */
#define DT_MAX_MERGE 64        /* states one merge launch can combine */
#define DT_MAX_SEGMENTS 8      /* segments of a packed batch in one device-scheduled launch */

int dt_version(void);
const char* dt_last_error(void);

/*
 * One KV chunk of non-causal attention: out = softmax(q k^T * scale) v and the
 * natural-log lse.  Replaces
 *   flash_attn_func(q, k, v, dropout_p=0.0, return_attn_probs=True)
 * as called at core/attention.py:137-143 and :185-191 (first two results).
 * out is bf16 [B,Sq,H,D] contiguous, lse fp32 [B,H,Sq] contiguous.
 * softmax_scale <= 0 selects D^-0.5 (flash_attn's default).
 */
int dt_attn_chunk_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                      int32_t B, int32_t Sq, int32_t Sk, int32_t H, int32_t D,
                      int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                      int64_t kv_stride_b, int64_t kv_stride_s, int64_t kv_stride_h,
                      float softmax_scale, void* stream);

/*
 * The same call for IEEE half tensors (flash_attn_func takes fp16 or bf16; the reference passes whatever
 * dtype the model runs in, core/attention.py:137-143, and executor/hunyuanvideo offers --precision fp16):
 * q, k, v and out are fp16, the products run on the fp16 MFMA, P is rounded to fp16 where the bf16 path
 * rounds it to bf16.  Everything else as above.  The launches that take `flags` do the same under
 * DT_ATTN_FP16.
 */
int dt_attn_chunk_f16_fwd(const void* q, const void* k, const void* v, void* out, float* lse,
                          int32_t B, int32_t Sq, int32_t Sk, int32_t H, int32_t D,
                          int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                          int64_t kv_stride_b, int64_t kv_stride_s, int64_t kv_stride_h,
                          float softmax_scale, void* stream);

/*
 * The same call site (core/attention.py:185-191) for fp32 tensors, computed in fp32 throughout (vector
 * ALU, expf / logf): the attention of the fp32 numbers themselves, not of their bf16 roundings.
 * flash_attn_func takes no fp32; the
 * reference runs its CPU-runnable configuration (fp32, B=1, H=4, d=64, 512 queries x 4 chunks of
 * 512 keys) on its torch math path, and this entry point is that path's counterpart here.  q / k / v
 * fp32 with element strides and a contiguous last dimension; out fp32 [B,Sq,H,D] contiguous, lse
 * fp32 [B,H,Sq].  Sk = 0 yields out = 0, lse = -inf.  Not tuned (about 1 TFLOP/s): model-sized
 * bf16 work belongs on dt_attn_chunk_fwd.
 */
int dt_attn_chunk_f32_fwd(const float* q, const float* k, const float* v, float* out, float* lse,
                          int32_t B, int32_t Sq, int32_t Sk, int32_t H, int32_t D,
                          int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                          int64_t kv_stride_b, int64_t kv_stride_s, int64_t kv_stride_h,
                          float softmax_scale, void* stream);

/*
 * Several attention states in one launch.  Job j attends q to the
 * concatenation of the chunks job_chunks[job_begin[j] .. job_begin[j+1]) and
 * writes ONE state (out_ptrs[j], lse_ptrs[j]).  A job of one chunk is the call
 * above; a job of several chunks equals computing each chunk separately and
 * folding the results with update_out_and_lse (core/attention.py:185-196,
 * utils.py:42-84), i.e. the "fresh" state of a target block.
 * k_ptrs/v_ptrs/kv_lens/kv_stride_b, job_begin, job_chunks, out_ptrs,
 * lse_ptrs are HOST arrays; they are copied into the kernel arguments.
 * All chunks share kv_stride_s / kv_stride_h.
 */
int dt_attn_jobs_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                     int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                     int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                     const int32_t* kv_lens, const int64_t* kv_stride_b,
                     int64_t kv_stride_s, int64_t kv_stride_h,
                     int32_t n_jobs, const int32_t* job_begin, const int32_t* job_chunks,
                     void* const* out_ptrs, float* const* lse_ptrs,
                     float softmax_scale, void* stream);

/*
 * The same launch with sub-ranges: job j covers the query rows
 * [job_q_begin[j], job_q_begin[j] + job_q_len[j]) only (other rows of its
 * destination are left untouched) and chunk reference e covers the keys
 * [entry_kv_begin[e], entry_kv_begin[e] + entry_kv_len[e]) of its chunk.  One
 * segment of a packed variable-length batch is one such job, so this replaces
 *   flash_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_kv, max_seqlen_q,
 *                          max_seqlen_kv, dropout_p=0.0, return_attn_probs=True)
 * as called at core/attention.py:314-324 and :366-376, where q/k/v are packed
 * [total, H, D] (pass B = 1, Sq = total) and the lse is [H, total].  A job
 * without keys writes out = 0, lse = -inf.  Either pair of range arrays may be
 * NULL (whole rows / whole chunks).  All range arrays are HOST arrays.
 */
int dt_attn_seg_jobs_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                         int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                         int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                         const int32_t* kv_lens, const int64_t* kv_stride_b,
                         int64_t kv_stride_s, int64_t kv_stride_h,
                         int32_t n_jobs, const int32_t* job_begin, const int32_t* job_chunks,
                         const int32_t* entry_kv_begin, const int32_t* entry_kv_len,
                         const int32_t* job_q_begin, const int32_t* job_q_len,
                         void* const* out_ptrs, float* const* lse_ptrs,
                         float softmax_scale, void* stream);

/*
 * Same, driven by a schedule that lives in device memory (dt_build_schedule*):
 * job j (0 <= j < max_jobs) is active iff j < *dev_count and computes the
 * single chunk id dev_compute_ids[j], writing its state into cache slot
 * `id` of the state arena (slot_out + id*slot_out_stride elements,
 * slot_lse + id*slot_lse_stride elements), or into (diag_out, diag_lse) when
 * id == diag -- the local chunk is recomputed on every call and never cached
 * (core/attention.py:137-144,193-194).  max_jobs sizes the grid; the host
 * never reads the schedule.
 */
int dt_attn_sched_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                      int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                      int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                      const int32_t* kv_lens, const int64_t* kv_stride_b,
                      int64_t kv_stride_s, int64_t kv_stride_h,
                      const int32_t* dev_compute_ids, const int32_t* dev_count, int32_t max_jobs,
                      void* slot_out, int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride,
                      int32_t diag, void* diag_out, float* diag_lse,
                      float softmax_scale, void* stream);

/*
 * The device-scheduled launch on a packed variable-length batch (q [1, total, H, D], the layout of
 * flash_attn_varlen_func as called at core/attention.py:314-324): segment s covers the query
 * rows [seg_q_begin[s], + seg_q_len[s]) and, inside chunk c, the keys
 * [seg_kv_begin[c * n_seg + s], + seg_kv_len[c * n_seg + s]).  Every scheduled chunk runs once
 * per segment and writes that segment's rows of its slot; rows outside every segment are left
 * untouched.  n_seg <= DT_MAX_SEGMENTS, n_chunks * n_seg <= DT_MAX_JOB_ENTRIES; the four
 * range arrays are HOST arrays.  With n_seg = 1 covering all rows and keys it is
 * dt_attn_sched_fwd.  No counterpart in the reference (its varlen path has no mask mode).
 */
int dt_attn_sched_seg_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                          int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                          int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                          const int32_t* kv_lens, const int64_t* kv_stride_b,
                          int64_t kv_stride_s, int64_t kv_stride_h,
                          const int32_t* dev_compute_ids, const int32_t* dev_count, int32_t max_jobs,
                          void* slot_out, int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride,
                          int32_t diag, void* diag_out, float* diag_lse,
                          int32_t n_seg, const int32_t* seg_q_begin, const int32_t* seg_q_len,
                          const int32_t* seg_kv_begin, const int32_t* seg_kv_len,
                          float softmax_scale, void* stream);

/*
 * The two variable-length launches with the segment boundaries in DEVICE memory -- the calling
 * convention of
 *   flash_attn_varlen_func(q, k, v, cu_seqlens_q, cu_seqlens_kv, max_seqlen_q, max_seqlen_kv, ...)
 * at core/attention.py:314-324 and :366-376, whose cu_seqlens are int32 device tensors
 * (executor/hunyuanvideo/hunyuan_transformer.py:789-792) and, for the other chunks, arrive with K/V
 * over the ring (core/attention.py:307-311).  The host never reads them: no copy, no synchronisation,
 * and the launch can be captured in a HIP graph while the boundaries change between replays.
 *   cu_seqlens_q   device int32 [n_seg + 1]: segment s covers query rows [cu_q[s], cu_q[s+1])
 *   cu_seqlens_kv  HOST array of n_chunks device pointers, each int32 [n_seg + 1]: the keys of segment
 *                  s inside chunk c are [cu_kv[c][s], cu_kv[c][s+1]) (NULL allowed for an empty chunk)
 *   max_seqlen_q   host upper bound of the segment lengths; it sizes the grid, so rows of a longer
 *                  segment would be left uncomputed (flash-attn's contract for the same argument)
 * The kernel clamps every boundary it reads to the rows / keys that exist, so a malformed list gives
 * wrong rows but no stray access.  n_seg is not limited by DT_MAX_SEGMENTS (n_seg * max_jobs <= 65535).
 * dt_attn_varlen_jobs_fwd: job j is segment job_segment[j] (HOST array) of the state (out_ptrs[j],
 * lse_ptrs[j]) over its chunk list; the segments of one state are separate jobs with one destination.
 * dt_attn_sched_varlen_fwd: every scheduled chunk runs once per segment, as in dt_attn_sched_seg_fwd.
 * No tail balancing (the jobs cover row sub-ranges), hence no workspace.
 */
int dt_attn_varlen_jobs_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                            int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                            int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                            const int32_t* kv_lens, const int64_t* kv_stride_b,
                            int64_t kv_stride_s, int64_t kv_stride_h,
                            int32_t n_jobs, const int32_t* job_begin, const int32_t* job_chunks,
                            const int32_t* job_segment, int32_t n_seg,
                            const int32_t* cu_seqlens_q, const int32_t* const* cu_seqlens_kv, int32_t max_seqlen_q,
                            void* const* out_ptrs, float* const* lse_ptrs,
                            float softmax_scale, int32_t flags, void* stream);
int dt_attn_sched_varlen_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                             int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                             int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                             const int32_t* kv_lens, const int64_t* kv_stride_b,
                             int64_t kv_stride_s, int64_t kv_stride_h,
                             const int32_t* dev_compute_ids, const int32_t* dev_count, int32_t max_jobs,
                             void* slot_out, int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride,
                             int32_t diag, void* diag_out, float* diag_lse,
                             int32_t n_seg, const int32_t* cu_seqlens_q, const int32_t* const* cu_seqlens_kv,
                             int32_t max_seqlen_q, float softmax_scale, int32_t flags, void* stream);

/*
 * Zeroes the rows [*first_row, n_rows) of a dense [n_rows, row_bytes] tensor, first_row read from
 * DEVICE memory (clamped to 0..n_rows): rows of a packed batch that belong to no segment
 * (cu_seqlens_q[n_seg] < total) come out of flash_attn_varlen_func as zeros, and with the boundaries
 * on the device the host cannot slice them off.  row_bytes a multiple of 16, dst 16-byte aligned.
 * Stands in for that part of the call at core/attention.py:314-324.
 */
int dt_zero_rows_from(void* dst, int64_t n_rows, int64_t row_bytes, const int32_t* first_row, void* stream);

/*
 * dt_attn_seg_jobs_fwd and dt_attn_sched_seg_fwd with a workspace (device memory, 16-byte aligned, at most
 * dt_attn_workspace_bytes() are used; NULL or too small: plain launch).  All workgroups of an
 * attention launch are equal pieces of work, so its last round usually fills only part of the
 * chip; with a workspace the work items of that round are each cut into several ranges of key
 * tiles that run side by side and write partial states into the workspace, and a small kernel
 * folds them into the destination -- 2 to 8 % off a launch.  Used only when every job covers all
 * query rows.  Calls that share a workspace must not overlap (same stream, or disjoint
 * workspaces).  No counterpart in the reference.
 *
 * flags: DT_ATTN_Q_PRESCALED says that the caller has folded softmax_scale * log2(e) into q before
 * rounding it to bf16 (in the QK-norm weight, or through dt_qk_norm_rope's out_scale): the scores
 * q k^T are then exponents of 2 as they stand, softmax_scale is ignored, and the softmax needs a
 * quarter fewer vector instructions (4 % faster at D = 128, 10 % at D = 64).  out and lse are those
 * of softmax(q k^T * ln 2).  The reference has no such mode (flash_attn_func scales inside).
 * DT_ATTN_FP16 says that q, k, v, the output states (and the partial states in the workspace) are IEEE
 * half instead of bfloat16, as in dt_attn_chunk_f16_fwd; it does not combine with DT_ATTN_Q_PRESCALED
 * (DT_ERR_UNSUPPORTED).
 */
#define DT_ATTN_Q_PRESCALED 1
#define DT_ATTN_FP16 2
int64_t dt_attn_workspace_bytes(void);
int dt_attn_seg_jobs_ws_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                            int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                            int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                            const int32_t* kv_lens, const int64_t* kv_stride_b,
                            int64_t kv_stride_s, int64_t kv_stride_h,
                            int32_t n_jobs, const int32_t* job_begin, const int32_t* job_chunks,
                            const int32_t* entry_kv_begin, const int32_t* entry_kv_len,
                            const int32_t* job_q_begin, const int32_t* job_q_len,
                            void* const* out_ptrs, float* const* lse_ptrs,
                            float softmax_scale, int32_t flags, void* workspace, int64_t workspace_bytes,
                            void* stream);
int dt_attn_sched_seg_ws_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                             int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                             int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                             const int32_t* kv_lens, const int64_t* kv_stride_b,
                             int64_t kv_stride_s, int64_t kv_stride_h,
                             const int32_t* dev_compute_ids, const int32_t* dev_count, int32_t max_jobs,
                             void* slot_out, int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride,
                             int32_t diag, void* diag_out, float* diag_lse,
                             int32_t n_seg, const int32_t* seg_q_begin, const int32_t* seg_q_len,
                             const int32_t* seg_kv_begin, const int32_t* seg_kv_len,
                             float softmax_scale, int32_t flags, void* workspace, int64_t workspace_bytes,
                             void* stream);

/*
 * dt_attn_seg_jobs_ws_fwd for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops, harnesses that forbid hipMalloc): no workspace argument, the tail of the
 * launch is split inside a device array that is part of the library (DT_NOALLOC_TAIL_SLOTS partial
 * states of 256 queries x 128 bf16 + 256 lse values = 34 078 720 bytes, held by every GPU the
 * library runs on until the process ends).  No counterpart in the reference.  Arguments, limits,
 * errors and results are those of dt_attn_seg_jobs_ws_fwd called with a workspace of exactly that
 * size: the split is planned to fit the array (a tail that would need more parts gets fewer), so the
 * scratch need does not grow with the input and no shape is turned away on its account.  The call
 * makes no hipMalloc / hipFree; the array's device address is looked up once per device on the first
 * call there (hipGetSymbolAddress: make that first call outside a graph capture).  Every GPU holds
 * its own copy of the array and the lookup answers for the CURRENT device, so the device that owns
 * q / out (and the stream) must be current when the call is made; a q that lives on another device
 * is refused with DT_ERR_INVALID.  All calls on one GPU share the array: calls that overlap in time
 * on one GPU (different streams or threads) race on it; order them on one stream.  Nothing in the
 * array has to start at zero (every partial state that is read was written by the same call).
 */
#define DT_NOALLOC_TAIL_SLOTS 512
int dt_attn_seg_jobs_noalloc_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D,
                                 int64_t q_stride_b, int64_t q_stride_s, int64_t q_stride_h,
                                 int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                                 const int32_t* kv_lens, const int64_t* kv_stride_b,
                                 int64_t kv_stride_s, int64_t kv_stride_h,
                                 int32_t n_jobs, const int32_t* job_begin, const int32_t* job_chunks,
                                 const int32_t* entry_kv_begin, const int32_t* entry_kv_len,
                                 const int32_t* job_q_begin, const int32_t* job_q_len,
                                 void* const* out_ptrs, float* const* lse_ptrs,
                                 float softmax_scale, int32_t flags, void* stream);

/*
 * N-way LSE merge: lse = logsumexp_i lse_i, out = sum_i exp(lse_i - lse) out_i.
 * Replaces the chain of update_out_and_lse / _update_out_and_lse calls
 * (utils.py:24-84; called at core/attention.py:116,144,194,196,213 and
 * core/cache.py:42) with one pass over HBM.  outs[i] is [B,Sq,H,D] contiguous
 * in src_dtype[i] (DT_BF16, DT_FP16 or DT_FP32, in any mix); lses[i] is fp32 in src_lse_layout[i].  A state whose lse is
 * -inf contributes nothing.  dst may alias one of the inputs of the same dtype
 * and layout (in-place cache coarsening, core/cache.py:28-46).  A pointer may
 * appear more than once (the reference can merge the local chunk twice,
 * core/attention.py:120-145 followed by :193-194).
 * outs, lses, src_dtype, src_lse_layout are HOST arrays of length n.
 */
int dt_merge_states(int32_t n, const void* const* outs, const float* const* lses,
                    const int32_t* src_dtype, const int32_t* src_lse_layout,
                    void* dst_out, int32_t dst_dtype, float* dst_lse, int32_t dst_lse_layout,
                    int32_t B, int32_t Sq, int32_t H, int32_t D, void* stream);

/*
 * State cache store / load: one streaming copy of (out, lse) between a caller
 * tensor and a cache slot (out bf16 [B,Sq,H,D], lse fp32 [B,H,Sq]).  Replaces
 * proCache.store_block / get_block (core/cache.py:75-84), which in the
 * reference keep Python references to fp32 tensors.  dt_state_copy is the same
 * copy between any two state formats (out in DT_BF16 / DT_FP16 / DT_FP32, lse in
 * either layout), e.g. for the fp16 slots of a model that runs in fp16.
 */
int dt_cache_store(const void* src_out, int32_t src_dtype, const float* src_lse, int32_t src_lse_layout,
                   void* slot_out, float* slot_lse,
                   int32_t B, int32_t Sq, int32_t H, int32_t D, void* stream);
int dt_cache_load(const void* slot_out, const float* slot_lse,
                  void* dst_out, int32_t dst_dtype, float* dst_lse, int32_t dst_lse_layout,
                  int32_t B, int32_t Sq, int32_t H, int32_t D, void* stream);
int dt_state_copy(const void* src_out, int32_t src_dtype, const float* src_lse, int32_t src_lse_layout,
                  void* dst_out, int32_t dst_dtype, float* dst_lse, int32_t dst_lse_layout,
                  int32_t B, int32_t Sq, int32_t H, int32_t D, void* stream);

/*
 * Device-side schedule builder.  mask is uint8 [T,L,C] (1 = reuse the cached
 * state of chunk c at step t, layer l; 0 = recompute).  For row (t,l):
 *   compute_ids = [diag (if 0 <= diag < C)] + ascending {c != diag : mask == 0}
 *   reuse_ids   = ascending {c != diag : mask != 0}
 *   counts      = {len(compute_ids), len(reuse_ids)}
 * Unused tail entries are set to -1.  The reference derives the equivalent
 * decision on the host from the stride table (core/attention.py:90-116,
 * core/redundancy_map.py:49-87); this kernel is the per-chunk generalisation.
 * dt_build_schedule handles one row (outputs int32 [C], [C], [2]);
 * dt_build_schedule_table all rows (outputs int32 [T,L,C], [T,L,C], [T,L,2]).
 * C <= 1024.
 */
int dt_build_schedule(const uint8_t* mask, int32_t T, int32_t L, int32_t C, int32_t t, int32_t l,
                      int32_t diag, int32_t* compute_ids, int32_t* reuse_ids, int32_t* counts,
                      void* stream);
int dt_build_schedule_table(const uint8_t* mask, int32_t T, int32_t L, int32_t C, int32_t diag,
                            int32_t* compute_ids, int32_t* reuse_ids, int32_t* counts, void* stream);

/*
 * Relative-L1 partial sums for the profiling mode: accumulates, over entries
 * where neither input is NaN, sums[0] += |a-b|, sums[1] += |a|, sums[2] += |b|,
 * sums[3] += count (all fp64, device memory, caller zeroes them).  Replaces the
 * mask-select / abs / mean chain with its three host syncs in rel_l1
 * (utils.py:214-241), used by record_out_redundancy
 * (core/redundancy_map.py:174-197).  a, b are fp32, n elements.
 */
int dt_rel_l1_sums(const float* a, const float* b, int64_t n, double* sums, void* stream);

/*
 * Producer side of an attention call: normalise every head row of x over D, apply the
 * rotary position embedding to the token rows [rope_begin, rope_end) and write the result
 * as bf16 [B,S,H,D] contiguous, the layout the attention entry points read -- one pass over
 * HBM.  Replaces the eager chains in front of proAttention.attn / varlen_attn at
 *   executor/cogvideox/attention_processor.py:55-71 (attn.norm_q / norm_k = LayerNorm over D;
 *     apply_rotary_emb on query[:, :, text_seqlen:] only; transpose + contiguous),
 *   executor/hunyuanvideo/hunyuan_transformer.py:177-191 (RMSNorm over D; apply_rotary_emb with
 *     interleaved pairs),
 *   executor/step/blocks.py:66-75 with executor/step/rope.py:13-90 (RMSNorm; rotate_half RoPE
 *     applied separately to the sections [64,32,32] of D).
 * x is bf16 with element strides (x_stride_b, x_stride_s, x_stride_h) and a contiguous last
 * dimension, so q, k or v can be read in place out of a fused QKV projection; with
 * norm = rope = 0 the call is the strided-to-contiguous copy of v.  y may alias x when x is
 * already contiguous [B,S,H,D].
 * weight / bias: fp32 [D] or NULL (1 / 0).  cos / sin: fp32 [rope_end - rope_begin, D], row
 * s - rope_begin belongs to token s; batch b reads its tables at + b * table_stride_b
 * elements (0 = shared).  out[d] = x[d] * cos[d] + rot(x)[d] * sin[d] with
 *   DT_ROPE_INTERLEAVED: rot(x)[2i] = -x[2i+1], rot(x)[2i+1] = x[2i];
 *   DT_ROPE_HALVES: inside each section [lo, hi): rot(x)[d] = -x[d + (hi-lo)/2] in the first
 *     half, x[d - (hi-lo)/2] in the second.  sections (HOST array, n_sections <= 3, each a
 *     multiple of 16, summing to D; n_sections = 0 means one section of D).
 * rounding = 0 computes in fp32 and rounds once on the way out; the DT_ROUND_* bits reproduce
 * the intermediate bf16 roundings of the callers' eager modules.  With DT_IO_FP16 in `rounding`, x and y
 * are IEEE half (a model run in fp16) and those intermediate roundings are to fp16.
 * out_scale (> 0; 1 for none) multiplies the result before that last rounding: with
 * softmax_scale * log2(e) here for q, the attention may run with DT_ATTN_Q_PRESCALED.
 */
int dt_qk_norm_rope(const void* x, int64_t x_stride_b, int64_t x_stride_s, int64_t x_stride_h, void* y,
                    int32_t B, int32_t S, int32_t H, int32_t D,
                    int32_t norm, const float* weight, const float* bias, float eps,
                    int32_t rope, const float* cos, const float* sin, int64_t table_stride_b,
                    int32_t rope_begin, int32_t rope_end, const int32_t* sections, int32_t n_sections,
                    int32_t rounding, float out_scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* DITANGO_HIP_H */
