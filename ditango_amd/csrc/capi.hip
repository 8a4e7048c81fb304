// C ABI entry points of the chunk-attention kernel plus the error plumbing.
// Argument checks happen here, on the host, before any launch: the kernels
// assume the shapes, strides and alignments validated below.
#include <cstdarg>
#include <cstdio>
#include <cmath>

#include "dt_common.h"

namespace dt {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

int hip_fail(hipError_t e, const char* what) {
  if (e == hipSuccess) return DT_OK;
  set_error("%s: %s", what, hipGetErrorString(e));
  return DT_ERR_HIP;
}

}  // namespace dt

using namespace dt;

extern "C" int dt_version(void) { return 100; }
extern "C" const char* dt_last_error(void) { return g_error; }

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

static int fill_common(AttnArgs& a, const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                       int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                       const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb, int64_t kv_ss,
                       int64_t kv_sh, float softmax_scale) {
  if (B <= 0 || Sq <= 0 || H <= 0) {
    set_error("B, Sq, H must be positive (got %d, %d, %d)", B, Sq, H);
    return DT_ERR_INVALID;
  }
  if (D != 64 && D != 128) {
    set_error("head dim %d not built (64 and 128 are)", D);
    return DT_ERR_UNSUPPORTED;
  }
  if (!q || !aligned16(q) || (q_sb % 8) || (q_ss % 8) || (q_sh % 8)) {
    set_error("q must be non-null, 16-byte aligned, with strides that are multiples of 8 elements");
    return DT_ERR_INVALID;
  }
  if (n_chunks <= 0 || n_chunks > DT_MAX_CHUNKS) {
    set_error("%d KV chunks: need 1..%d", n_chunks, DT_MAX_CHUNKS);
    return DT_ERR_INVALID;
  }
  if (!k_ptrs || !v_ptrs || !kv_lens || !kv_sb) {
    set_error("null chunk table");
    return DT_ERR_INVALID;
  }
  if ((kv_ss % 8) || (kv_sh % 8) || kv_ss <= 0) {
    set_error("k/v token and head strides must be multiples of 8 elements");
    return DT_ERR_INVALID;
  }
  a.q = static_cast<const uint16_t*>(q);
  a.q_sb = q_sb; a.q_ss = q_ss; a.q_sh = q_sh;
  a.B = B; a.H = H; a.Sq = Sq;
  a.nqt = (Sq + 255) / 256;  // 256 queries per workgroup
  const int64_t total = (int64_t)B * H * a.nqt;
  if (total > (1 << 28)) {
    set_error("too many query tiles (%lld)", (long long)total);
    return DT_ERR_INVALID;
  }
  a.total = (int32_t)total;
  a.per_xcd = (a.total + 7) / 8;
  const float scale = softmax_scale > 0.f ? softmax_scale : 1.0f / std::sqrt((float)D);
  a.scale_log2 = scale * 1.4426950408889634f;
  for (int i = 0; i < n_chunks; ++i) {
    if (kv_lens[i] < 0) {
      set_error("chunk %d has negative length", i);
      return DT_ERR_INVALID;
    }
    if (kv_lens[i] > 0 && (!k_ptrs[i] || !v_ptrs[i] || !aligned16(k_ptrs[i]) || !aligned16(v_ptrs[i]) || (kv_sb[i] % 8))) {
      set_error("chunk %d: null or misaligned k/v", i);
      return DT_ERR_INVALID;
    }
    if ((int64_t)kv_lens[i] * kv_ss * 2 >= (1ll << 31)) {
      set_error("chunk %d: one (batch, head) plane spans 2 GiB or more; split the chunk", i);
      return DT_ERR_INVALID;
    }
    a.k[i] = static_cast<const uint16_t*>(k_ptrs[i]);
    a.v[i] = static_cast<const uint16_t*>(v_ptrs[i]);
    a.kv_len[i] = kv_lens[i];
    a.kv_sb[i] = kv_sb[i];
  }
  a.n_chunks = n_chunks;
  a.kv_ss = kv_ss;
  a.kv_sh = kv_sh;
  return DT_OK;
}

extern "C" int64_t dt_attn_workspace_bytes(void) { return kMaxTailSlots * (256 * 128 * 2 + 256 * 4); }

static int check_workspace(const void* workspace, int64_t workspace_bytes) {
  if (workspace && (!aligned16(workspace) || workspace_bytes < 0)) {
    set_error("workspace must be 16-byte aligned with a non-negative size");
    return DT_ERR_INVALID;
  }
  return DT_OK;
}

static int apply_flags(AttnArgs& a, int32_t flags) {
  if (flags & ~(DT_ATTN_Q_PRESCALED | DT_ATTN_FP16)) {
    set_error("unknown attention flags 0x%x", (unsigned)flags);
    return DT_ERR_INVALID;
  }
  if ((flags & DT_ATTN_Q_PRESCALED) && (flags & DT_ATTN_FP16)) {
    set_error("DT_ATTN_Q_PRESCALED and DT_ATTN_FP16 do not combine (the prescaled softmax keeps probabilities beyond fp16's range)");
    return DT_ERR_UNSUPPORTED;
  }
  a.q_prescaled = (flags & DT_ATTN_Q_PRESCALED) ? 1 : 0;
  a.elem_f16 = (flags & DT_ATTN_FP16) ? 1 : 0;
  return DT_OK;
}

extern "C" int dt_attn_seg_jobs_ws_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                                       int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                                       const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb,
                                       int64_t kv_ss, int64_t kv_sh, int32_t n_jobs, const int32_t* job_begin,
                                       const int32_t* job_chunks, const int32_t* entry_kv_begin,
                                       const int32_t* entry_kv_len, const int32_t* job_q_begin,
                                       const int32_t* job_q_len, void* const* out_ptrs, float* const* lse_ptrs,
                                       float softmax_scale, int32_t flags, void* workspace,
                                       int64_t workspace_bytes, void* stream) {
  if (int rc = check_workspace(workspace, workspace_bytes)) return rc;
  AttnArgs a{};
  if (int rc = fill_common(a, q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                           softmax_scale))
    return rc;
  if (int rc = apply_flags(a, flags)) return rc;
  if (n_jobs == 0) return DT_OK;
  if (n_jobs < 0 || n_jobs > DT_MAX_JOBS || !job_begin || !job_chunks || !out_ptrs || !lse_ptrs) {
    set_error("%d jobs: need 0..%d and non-null job tables", n_jobs, DT_MAX_JOBS);
    return DT_ERR_INVALID;
  }
  if (job_begin[0] != 0 || job_begin[n_jobs] > DT_MAX_JOB_ENTRIES) {
    set_error("job_begin must start at 0 and end at most at %d", DT_MAX_JOB_ENTRIES);
    return DT_ERR_INVALID;
  }
  if ((entry_kv_begin == nullptr) != (entry_kv_len == nullptr) || (job_q_begin == nullptr) != (job_q_len == nullptr)) {
    set_error("range arrays come in (begin, len) pairs");
    return DT_ERR_INVALID;
  }
  int32_t longest = 0;
  for (int j = 0; j < n_jobs; ++j) {
    if (job_begin[j + 1] < job_begin[j]) {
      set_error("job_begin is not monotone at job %d", j);
      return DT_ERR_INVALID;
    }
    if (!out_ptrs[j] || !lse_ptrs[j] || !aligned16(out_ptrs[j])) {
      set_error("job %d: null or misaligned destination", j);
      return DT_ERR_INVALID;
    }
    a.job_out[j] = static_cast<uint16_t*>(out_ptrs[j]);
    a.job_lse[j] = lse_ptrs[j];
    a.job_begin[j] = job_begin[j];
    const int32_t qb = job_q_begin ? job_q_begin[j] : 0;
    const int32_t ql = job_q_len ? job_q_len[j] : Sq;
    if (qb < 0 || ql < 0 || (int64_t)qb + ql > Sq) {
      set_error("job %d: query rows [%d, %d) outside [0, %d)", j, qb, qb + ql, Sq);
      return DT_ERR_INVALID;
    }
    a.job_q_begin[j] = qb;
    a.job_q_len[j] = ql;
    longest = ql > longest ? ql : longest;
  }
  a.job_begin[n_jobs] = job_begin[n_jobs];
  for (int e = 0; e < job_begin[n_jobs]; ++e) {
    const int32_t c = job_chunks[e];
    if (c < 0 || c >= n_chunks) {
      set_error("job chunk reference %d is outside the chunk table", c);
      return DT_ERR_INVALID;
    }
    const int32_t kb = entry_kv_begin ? entry_kv_begin[e] : 0;
    const int32_t kl = entry_kv_len ? entry_kv_len[e] : kv_lens[c];
    if (kb < 0 || kl < 0 || (int64_t)kb + kl > kv_lens[c]) {
      set_error("chunk reference %d: keys [%d, %d) outside chunk %d of length %d", e, kb, kb + kl, c, kv_lens[c]);
      return DT_ERR_INVALID;
    }
    a.job_chunks[e] = c;
    a.entry_kv_begin[e] = kb;
    a.entry_kv_len[e] = kl;
  }
  // size the grid for the longest job; shorter jobs leave their surplus workgroups at once
  a.nqt = (longest + 255) / 256;
  a.total = B * H * a.nqt;
  a.per_xcd = (a.total + 7) / 8;
  // the tail of the launch is only split when every job covers all query rows
  return launch_attn(a, D, n_jobs, (hipStream_t)stream, workspace, workspace_bytes, job_q_begin == nullptr);
}

// Device-resident segment boundaries: shared checks of the two varlen entry points.
static int fill_device_segments(AttnArgs& a, int32_t n_chunks, const int32_t* kv_lens, int32_t n_seg,
                                const int32_t* cu_seqlens_q, const int32_t* const* cu_seqlens_kv, int32_t max_seqlen_q,
                                int32_t B, int32_t Sq, int32_t H) {
  if (n_seg <= 0 || !cu_seqlens_q || !cu_seqlens_kv) {
    set_error("device segment boundaries: need n_seg > 0, cu_seqlens_q and the per-chunk cu_seqlens_kv table");
    return DT_ERR_INVALID;
  }
  if (max_seqlen_q <= 0) {
    set_error("max_seqlen_q must be positive (got %d): it sizes the grid, the boundaries themselves are never read on the host", max_seqlen_q);
    return DT_ERR_INVALID;
  }
  if ((reinterpret_cast<uintptr_t>(cu_seqlens_q) & 3) != 0) {
    set_error("cu_seqlens_q must be 4-byte aligned");
    return DT_ERR_INVALID;
  }
  for (int c = 0; c < n_chunks; ++c) {
    if (kv_lens[c] > 0 && (!cu_seqlens_kv[c] || (reinterpret_cast<uintptr_t>(cu_seqlens_kv[c]) & 3) != 0)) {
      set_error("chunk %d: null or misaligned cu_seqlens_kv", c);
      return DT_ERR_INVALID;
    }
    // an empty chunk is never dereferenced for keys, but the kernel still reads its boundaries: point it at the queries'
    a.cu_kv[c] = cu_seqlens_kv[c] ? cu_seqlens_kv[c] : cu_seqlens_q;
  }
  a.cu_q = cu_seqlens_q;
  // size the grid for the longest segment the caller promises; shorter ones leave their surplus workgroups at once
  a.nqt = ((max_seqlen_q < Sq ? max_seqlen_q : Sq) + 255) / 256;
  a.total = B * H * a.nqt;
  a.per_xcd = (a.total + 7) / 8;
  return DT_OK;
}

extern "C" int dt_attn_varlen_jobs_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                                       int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                                       const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb,
                                       int64_t kv_ss, int64_t kv_sh, int32_t n_jobs, const int32_t* job_begin,
                                       const int32_t* job_chunks, const int32_t* job_segment, int32_t n_seg,
                                       const int32_t* cu_seqlens_q, const int32_t* const* cu_seqlens_kv,
                                       int32_t max_seqlen_q, void* const* out_ptrs, float* const* lse_ptrs,
                                       float softmax_scale, int32_t flags, void* stream) {
  AttnArgs a{};
  if (int rc = fill_common(a, q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                           softmax_scale))
    return rc;
  if (int rc = apply_flags(a, flags)) return rc;
  if (n_jobs == 0) return DT_OK;
  if (n_jobs < 0 || n_jobs > DT_MAX_JOBS || !job_begin || !job_chunks || !job_segment || !out_ptrs || !lse_ptrs) {
    set_error("%d jobs: need 0..%d and non-null job tables", n_jobs, DT_MAX_JOBS);
    return DT_ERR_INVALID;
  }
  if (job_begin[0] != 0 || job_begin[n_jobs] > DT_MAX_JOB_ENTRIES) {
    set_error("job_begin must start at 0 and end at most at %d", DT_MAX_JOB_ENTRIES);
    return DT_ERR_INVALID;
  }
  if (int rc = fill_device_segments(a, n_chunks, kv_lens, n_seg, cu_seqlens_q, cu_seqlens_kv, max_seqlen_q, B, Sq, H))
    return rc;
  for (int j = 0; j < n_jobs; ++j) {
    if (job_begin[j + 1] < job_begin[j]) {
      set_error("job_begin is not monotone at job %d", j);
      return DT_ERR_INVALID;
    }
    if (!out_ptrs[j] || !lse_ptrs[j] || !aligned16(out_ptrs[j])) {
      set_error("job %d: null or misaligned destination", j);
      return DT_ERR_INVALID;
    }
    if (job_segment[j] < 0 || job_segment[j] >= n_seg) {
      set_error("job %d: segment %d outside 0..%d", j, job_segment[j], n_seg - 1);
      return DT_ERR_INVALID;
    }
    a.job_out[j] = static_cast<uint16_t*>(out_ptrs[j]);
    a.job_lse[j] = lse_ptrs[j];
    a.job_begin[j] = job_begin[j];
    a.job_q_begin[j] = job_segment[j];   // with device boundaries this field names the segment
    a.job_q_len[j] = 0;
  }
  a.job_begin[n_jobs] = job_begin[n_jobs];
  for (int e = 0; e < job_begin[n_jobs]; ++e) {
    const int32_t c = job_chunks[e];
    if (c < 0 || c >= n_chunks) {
      set_error("job chunk reference %d is outside the chunk table", c);
      return DT_ERR_INVALID;
    }
    a.job_chunks[e] = c;
  }
  return launch_attn(a, D, n_jobs, (hipStream_t)stream, nullptr, 0, false);
}

// The same launch for callers that cannot allocate: the tail is split inside the library's own
// device array instead of a caller's workspace.
extern "C" int dt_attn_seg_jobs_noalloc_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                                            int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                                            const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb,
                                            int64_t kv_ss, int64_t kv_sh, int32_t n_jobs, const int32_t* job_begin,
                                            const int32_t* job_chunks, const int32_t* entry_kv_begin,
                                            const int32_t* entry_kv_len, const int32_t* job_q_begin,
                                            const int32_t* job_q_len, void* const* out_ptrs, float* const* lse_ptrs,
                                            float softmax_scale, int32_t flags, void* stream) {
  // The scratch array has one copy per GPU, at that GPU's own address, and the lookup below answers for the
  // CURRENT device: it must be the one that owns the tensors (and the stream), or the kernel would be handed
  // another GPU's array.
  if (q) {
    hipPointerAttribute_t attr{};
    int dev = -1;
    if (hipPointerGetAttributes(&attr, q) == hipSuccess && hipGetDevice(&dev) == hipSuccess &&
        attr.type == hipMemoryTypeDevice && attr.device != dev) {
      set_error("q lives on device %d but device %d is current: make the tensors' device current for this call", attr.device, dev);
      return DT_ERR_INVALID;
    }
    (void)hipGetLastError();  // a pointer the runtime does not know leaves an error behind; the checks below report it properly
  }
  void* scratch = nullptr;
  int64_t scratch_bytes = 0;
  if (int rc = static_tail_scratch(&scratch, &scratch_bytes)) return rc;
  return dt_attn_seg_jobs_ws_fwd(q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                                 n_jobs, job_begin, job_chunks, entry_kv_begin, entry_kv_len, job_q_begin, job_q_len,
                                 out_ptrs, lse_ptrs, softmax_scale, flags, scratch, scratch_bytes, stream);
}

extern "C" int dt_attn_seg_jobs_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                                    int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                                    const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb,
                                    int64_t kv_ss, int64_t kv_sh, int32_t n_jobs, const int32_t* job_begin,
                                    const int32_t* job_chunks, const int32_t* entry_kv_begin,
                                    const int32_t* entry_kv_len, const int32_t* job_q_begin,
                                    const int32_t* job_q_len, void* const* out_ptrs, float* const* lse_ptrs,
                                    float softmax_scale, void* stream) {
  return dt_attn_seg_jobs_ws_fwd(q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                                 n_jobs, job_begin, job_chunks, entry_kv_begin, entry_kv_len, job_q_begin, job_q_len,
                                 out_ptrs, lse_ptrs, softmax_scale, 0, nullptr, 0, stream);
}

extern "C" int dt_attn_jobs_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb, int64_t q_ss,
                                int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                                const int32_t* kv_lens, const int64_t* kv_sb, int64_t kv_ss, int64_t kv_sh,
                                int32_t n_jobs, const int32_t* job_begin, const int32_t* job_chunks,
                                void* const* out_ptrs, float* const* lse_ptrs, float softmax_scale, void* stream) {
  return dt_attn_seg_jobs_fwd(q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                              n_jobs, job_begin, job_chunks, nullptr, nullptr, nullptr, nullptr, out_ptrs, lse_ptrs,
                              softmax_scale, stream);
}

static int chunk_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int32_t B, int32_t Sq, int32_t Sk,
                     int32_t H, int32_t D, int64_t q_sb, int64_t q_ss, int64_t q_sh, int64_t kv_sb, int64_t kv_ss,
                     int64_t kv_sh, float softmax_scale, int32_t flags, void* stream) {
  const void* kp[1] = {k};
  const void* vp[1] = {v};
  const int32_t lens[1] = {Sk};
  const int64_t sbs[1] = {kv_sb};
  const int32_t begin[2] = {0, 1};
  const int32_t chunks[1] = {0};
  void* outs[1] = {out};
  float* lses[1] = {lse};
  return dt_attn_seg_jobs_ws_fwd(q, B, Sq, H, D, q_sb, q_ss, q_sh, 1, kp, vp, lens, sbs, kv_ss, kv_sh, 1, begin, chunks,
                                 nullptr, nullptr, nullptr, nullptr, outs, lses, softmax_scale, flags, nullptr, 0, stream);
}

extern "C" int dt_attn_chunk_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int32_t B,
                                 int32_t Sq, int32_t Sk, int32_t H, int32_t D, int64_t q_sb, int64_t q_ss, int64_t q_sh,
                                 int64_t kv_sb, int64_t kv_ss, int64_t kv_sh, float softmax_scale, void* stream) {
  return chunk_fwd(q, k, v, out, lse, B, Sq, Sk, H, D, q_sb, q_ss, q_sh, kv_sb, kv_ss, kv_sh, softmax_scale, 0, stream);
}

extern "C" int dt_attn_chunk_f16_fwd(const void* q, const void* k, const void* v, void* out, float* lse, int32_t B,
                                     int32_t Sq, int32_t Sk, int32_t H, int32_t D, int64_t q_sb, int64_t q_ss,
                                     int64_t q_sh, int64_t kv_sb, int64_t kv_ss, int64_t kv_sh, float softmax_scale,
                                     void* stream) {
  return chunk_fwd(q, k, v, out, lse, B, Sq, Sk, H, D, q_sb, q_ss, q_sh, kv_sb, kv_ss, kv_sh, softmax_scale, DT_ATTN_FP16,
                   stream);
}

// Checks and fields every device-scheduled launch shares.
static int fill_sched(AttnArgs& a, int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                      const int32_t* kv_lens, const int32_t* dev_compute_ids, const int32_t* dev_count, int32_t max_jobs,
                      void* slot_out, int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride, int32_t diag,
                      void* diag_out, float* diag_lse) {
  if (max_jobs < 0 || max_jobs > n_chunks) {
    set_error("max_jobs %d must be in 0..n_chunks (%d)", max_jobs, n_chunks);
    return DT_ERR_INVALID;
  }
  if (!dev_compute_ids || !dev_count || !slot_out || !slot_lse || !aligned16(slot_out) || (slot_out_stride % 8)) {
    set_error("null or misaligned schedule/arena pointer");
    return DT_ERR_INVALID;
  }
  for (int i = 0; i < n_chunks; ++i) {
    if (kv_lens[i] > 0 && (!k_ptrs[i] || !v_ptrs[i])) {
      set_error("chunk %d: null k/v", i);
      return DT_ERR_INVALID;
    }
  }
  if (diag >= 0 && diag < n_chunks && (!diag_out || !diag_lse || !aligned16(diag_out))) {
    set_error("diag chunk %d needs a destination outside the cache", diag);
    return DT_ERR_INVALID;
  }
  a.dev_ids = dev_compute_ids;
  a.dev_count = dev_count;
  a.slot_out = static_cast<uint16_t*>(slot_out);
  a.slot_lse = slot_lse;
  a.slot_out_stride = slot_out_stride;
  a.slot_lse_stride = slot_lse_stride;
  a.diag = diag;
  a.diag_out = static_cast<uint16_t*>(diag_out);
  a.diag_lse = diag_lse;
  return DT_OK;
}

extern "C" int dt_attn_sched_seg_ws_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                                        int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                                        const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb,
                                        int64_t kv_ss, int64_t kv_sh, const int32_t* dev_compute_ids,
                                        const int32_t* dev_count, int32_t max_jobs, void* slot_out,
                                        int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride,
                                        int32_t diag, void* diag_out, float* diag_lse, int32_t n_seg,
                                        const int32_t* seg_q_begin, const int32_t* seg_q_len,
                                        const int32_t* seg_kv_begin, const int32_t* seg_kv_len, float softmax_scale,
                                        int32_t flags, void* workspace, int64_t workspace_bytes, void* stream) {
  if (int rc = check_workspace(workspace, workspace_bytes)) return rc;
  AttnArgs a{};
  if (int rc = fill_common(a, q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                           softmax_scale))
    return rc;
  if (int rc = apply_flags(a, flags)) return rc;
  if (max_jobs == 0) return DT_OK;
  if (int rc = fill_sched(a, n_chunks, k_ptrs, v_ptrs, kv_lens, dev_compute_ids, dev_count, max_jobs, slot_out,
                          slot_out_stride, slot_lse, slot_lse_stride, diag, diag_out, diag_lse))
    return rc;
  int32_t jobs = max_jobs;
  if (n_seg != 0) {
    if (n_seg < 0 || n_seg > DT_MAX_SEGMENTS || (int64_t)n_seg * n_chunks > DT_MAX_JOB_ENTRIES) {
      set_error("%d segments x %d chunks: need 1..%d segments and at most %d (chunk, segment) pairs", n_seg, n_chunks,
                DT_MAX_SEGMENTS, DT_MAX_JOB_ENTRIES);
      return DT_ERR_INVALID;
    }
    if (!seg_q_begin || !seg_q_len || !seg_kv_begin || !seg_kv_len) {
      set_error("null segment range array");
      return DT_ERR_INVALID;
    }
    int32_t longest = 0;
    for (int s = 0; s < n_seg; ++s) {
      const int32_t qb = seg_q_begin[s], ql = seg_q_len[s];
      if (qb < 0 || ql < 0 || (int64_t)qb + ql > Sq) {
        set_error("segment %d: query rows [%d, %d) outside [0, %d)", s, qb, qb + ql, Sq);
        return DT_ERR_INVALID;
      }
      a.seg_q_begin[s] = qb;
      a.seg_q_len[s] = ql;
      longest = ql > longest ? ql : longest;
    }
    for (int c = 0; c < n_chunks; ++c)
      for (int s = 0; s < n_seg; ++s) {
        const int e = c * n_seg + s;
        const int32_t kb = seg_kv_begin[e], kl = seg_kv_len[e];
        if (kb < 0 || kl < 0 || (int64_t)kb + kl > kv_lens[c]) {
          set_error("segment %d: keys [%d, %d) outside chunk %d of length %d", s, kb, kb + kl, c, kv_lens[c]);
          return DT_ERR_INVALID;
        }
        a.entry_kv_begin[e] = kb;
        a.entry_kv_len[e] = kl;
      }
    a.n_seg = n_seg;
    // size the grid for the longest segment; shorter ones leave their surplus workgroups at once
    a.nqt = (longest + 255) / 256;
    a.total = B * H * a.nqt;
    a.per_xcd = (a.total + 7) / 8;
    jobs = max_jobs * n_seg;
  }
  return launch_attn(a, D, jobs, (hipStream_t)stream, workspace, workspace_bytes, n_seg == 0);
}

extern "C" int dt_attn_sched_varlen_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                                        int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                                        const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb,
                                        int64_t kv_ss, int64_t kv_sh, const int32_t* dev_compute_ids,
                                        const int32_t* dev_count, int32_t max_jobs, void* slot_out,
                                        int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride,
                                        int32_t diag, void* diag_out, float* diag_lse, int32_t n_seg,
                                        const int32_t* cu_seqlens_q, const int32_t* const* cu_seqlens_kv,
                                        int32_t max_seqlen_q, float softmax_scale, int32_t flags, void* stream) {
  AttnArgs a{};
  if (int rc = fill_common(a, q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                           softmax_scale))
    return rc;
  if (int rc = apply_flags(a, flags)) return rc;
  if (max_jobs == 0) return DT_OK;
  if (int rc = fill_sched(a, n_chunks, k_ptrs, v_ptrs, kv_lens, dev_compute_ids, dev_count, max_jobs, slot_out,
                          slot_out_stride, slot_lse, slot_lse_stride, diag, diag_out, diag_lse))
    return rc;
  if (n_seg <= 0 || (int64_t)n_seg * max_jobs > 65535) {
    set_error("%d segments x %d scheduled chunks: need at least one segment and at most 65535 launch planes", n_seg, max_jobs);
    return DT_ERR_INVALID;
  }
  if (int rc = fill_device_segments(a, n_chunks, kv_lens, n_seg, cu_seqlens_q, cu_seqlens_kv, max_seqlen_q, B, Sq, H))
    return rc;
  a.n_seg = n_seg;
  return launch_attn(a, D, max_jobs * n_seg, (hipStream_t)stream, nullptr, 0, false);
}

extern "C" int dt_attn_sched_seg_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb,
                                     int64_t q_ss, int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs,
                                     const void* const* v_ptrs, const int32_t* kv_lens, const int64_t* kv_sb,
                                     int64_t kv_ss, int64_t kv_sh, const int32_t* dev_compute_ids,
                                     const int32_t* dev_count, int32_t max_jobs, void* slot_out,
                                     int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride, int32_t diag,
                                     void* diag_out, float* diag_lse, int32_t n_seg, const int32_t* seg_q_begin,
                                     const int32_t* seg_q_len, const int32_t* seg_kv_begin,
                                     const int32_t* seg_kv_len, float softmax_scale, void* stream) {
  return dt_attn_sched_seg_ws_fwd(q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss,
                                  kv_sh, dev_compute_ids, dev_count, max_jobs, slot_out, slot_out_stride, slot_lse,
                                  slot_lse_stride, diag, diag_out, diag_lse, n_seg, seg_q_begin, seg_q_len,
                                  seg_kv_begin, seg_kv_len, softmax_scale, 0, nullptr, 0, stream);
}

extern "C" int dt_attn_sched_fwd(const void* q, int32_t B, int32_t Sq, int32_t H, int32_t D, int64_t q_sb, int64_t q_ss,
                                 int64_t q_sh, int32_t n_chunks, const void* const* k_ptrs, const void* const* v_ptrs,
                                 const int32_t* kv_lens, const int64_t* kv_sb, int64_t kv_ss, int64_t kv_sh,
                                 const int32_t* dev_compute_ids, const int32_t* dev_count, int32_t max_jobs,
                                 void* slot_out, int64_t slot_out_stride, float* slot_lse, int64_t slot_lse_stride,
                                 int32_t diag, void* diag_out, float* diag_lse, float softmax_scale, void* stream) {
  return dt_attn_sched_seg_fwd(q, B, Sq, H, D, q_sb, q_ss, q_sh, n_chunks, k_ptrs, v_ptrs, kv_lens, kv_sb, kv_ss, kv_sh,
                               dev_compute_ids, dev_count, max_jobs, slot_out, slot_out_stride, slot_lse,
                               slot_lse_stride, diag, diag_out, diag_lse, 0, nullptr, nullptr, nullptr, nullptr,
                               softmax_scale, stream);
}
