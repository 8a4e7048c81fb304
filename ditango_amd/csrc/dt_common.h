// Shared declarations of the kernel translation units (not part of the public ABI).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "ditango_hip.h"

namespace dt {

void set_error(const char* fmt, ...);
int hip_fail(hipError_t e, const char* what);

// Kernel arguments of the chunk-attention kernel.  Passed by value, so the
// chunk and job tables travel in the kernarg segment: no device-side table,
// no host-to-device copy per call.
struct AttnArgs {
  const __bf16* q;
  int64_t q_sb, q_ss, q_sh;
  int32_t B, H, Sq;
  int32_t nqt;        // query tiles per (batch, head)
  int32_t total;      // B*H*nqt work items per job
  int32_t per_xcd;    // work items handed to each of the 8 XCDs
  float scale_log2;   // softmax scale * log2(e)
  // chunk table
  int32_t n_chunks;
  const __bf16* k[DT_MAX_CHUNKS];
  const __bf16* v[DT_MAX_CHUNKS];
  int64_t kv_sb[DT_MAX_CHUNKS];
  int32_t kv_len[DT_MAX_CHUNKS];
  int64_t kv_ss, kv_sh;
  // host-listed jobs
  __bf16* job_out[DT_MAX_JOBS];
  float* job_lse[DT_MAX_JOBS];
  int32_t job_begin[DT_MAX_JOBS + 1];
  int32_t job_chunks[DT_MAX_JOB_ENTRIES];
  // query rows [job_q_begin, job_q_begin + job_q_len) of each job; keys [kv_begin, kv_begin + kv_len)
  // of each chunk reference (a segment of a packed variable-length batch is a job on sub-ranges)
  int32_t job_q_begin[DT_MAX_JOBS];
  int32_t job_q_len[DT_MAX_JOBS];
  int32_t entry_kv_begin[DT_MAX_JOB_ENTRIES];
  int32_t entry_kv_len[DT_MAX_JOB_ENTRIES];
  // device-listed jobs (dev_ids != nullptr): job j computes chunk dev_ids[j] if j < *dev_count
  const int32_t* dev_ids;
  const int32_t* dev_count;
  __bf16* slot_out;
  float* slot_lse;
  int64_t slot_out_stride, slot_lse_stride;
  int32_t diag;
  __bf16* diag_out;
  float* diag_lse;
  // device-listed jobs on a packed variable-length batch (n_seg > 0): launch job j is segment
  // j % n_seg of the chunk listed at j / n_seg; the keys of segment s inside chunk c are
  // entry_kv_begin/len[c * n_seg + s]
  int32_t n_seg;
  int32_t seg_q_begin[DT_MAX_SEGMENTS];
  int32_t seg_q_len[DT_MAX_SEGMENTS];
};

int launch_attn(const AttnArgs& a, int D, int n_jobs, hipStream_t stream);

}  // namespace dt
