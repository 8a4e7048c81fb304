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
  // q, K, V and the output states are 16-bit elements: bfloat16, or IEEE half when elem_f16 is set
  const uint16_t* q;
  int64_t q_sb, q_ss, q_sh;
  int32_t B, H, Sq;
  int32_t nqt;        // query tiles per (batch, head)
  int32_t total;      // B*H*nqt work items per job
  int32_t per_xcd;    // work items handed to each of the 8 XCDs
  float scale_log2;   // softmax scale * log2(e)
  int32_t q_prescaled;  // the caller folded scale_log2 into q: scores are already in log2 units
  int32_t elem_f16;     // the 16-bit tensors are IEEE half instead of bfloat16
  // chunk table
  int32_t n_chunks;
  const uint16_t* k[DT_MAX_CHUNKS];
  const uint16_t* v[DT_MAX_CHUNKS];
  int64_t kv_sb[DT_MAX_CHUNKS];
  int32_t kv_len[DT_MAX_CHUNKS];
  int64_t kv_ss, kv_sh;
  // host-listed jobs
  uint16_t* job_out[DT_MAX_JOBS];
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
  uint16_t* slot_out;
  float* slot_lse;
  int64_t slot_out_stride, slot_lse_stride;
  int32_t diag;
  uint16_t* diag_out;
  float* diag_lse;
  // device-listed jobs on a packed variable-length batch (n_seg > 0): launch job j is segment
  // j % n_seg of the chunk listed at j / n_seg; the keys of segment s inside chunk c are
  // entry_kv_begin/len[c * n_seg + s]
  int32_t n_seg;
  int32_t seg_q_begin[DT_MAX_SEGMENTS];
  int32_t seg_q_len[DT_MAX_SEGMENTS];
  // Segment boundaries that live in DEVICE memory (cu_q != nullptr), the calling convention of
  // flash_attn_varlen_func: cu_q[s], cu_q[s + 1] bound the query rows of segment s and cu_kv[c][s],
  // cu_kv[c][s + 1] its keys inside chunk c (every chunk brings its own boundaries).  The host never
  // reads them; the kernel clamps them to the tensors' extents.  A host-listed job then names its
  // segment in job_q_begin[job]; a device-listed job is segment job % n_seg as above.
  const int32_t* cu_q;
  const int32_t* cu_kv[DT_MAX_CHUNKS];
  // Tail balancing (workspace launches only).  The workgroups of a launch are equal pieces of
  // work, so its last round usually fills only part of the chip.  The main launch then leaves
  // the work items with index >= tail_idx0 of job tail_job alone (tail_job < 0: nothing is left);
  // extra grid planes behind the jobs run each of them as part_ways workgroups over disjoint
  // ranges of key tiles that write partial states into the workspace (same launch, so a part
  // starts as soon as a CU is free), and a small second kernel folds the parts into the
  // destination.
  int32_t n_jobs;      // grid planes (blockIdx.y) that are jobs; planes behind them hold tail parts
  int32_t tail_job;
  int32_t tail_idx0;
  int32_t tail_items;  // tail items per XCD lane of the grid (= tail workgroup slots / 8)
  int32_t part_ways;
  uint16_t* ws_out;   // [slot][256 queries][D]
  float* ws_lse;    // [slot][256]
};

// Dynamic LDS of one attention workgroup by head dimension (four 64-key buffers per operand).  The
// occupancy of a CU follows from it: one workgroup at 128, two at 64.
constexpr int kAttnLdsBytes128 = 131072;
constexpr int kAttnLdsBytes64 = 65536;

// Workspace bytes the tail balancing can use at most (what dt_attn_workspace_bytes reports).
constexpr int64_t kMaxTailSlots = 1536;

// The allocation-free entry point splits tails inside a device array of this many partial-state
// slots (sized for D = 128: 256 queries x 128 bf16 + 256 lse values each).
constexpr int64_t kStaticTailSlots = DT_NOALLOC_TAIL_SLOTS;
constexpr int64_t kStaticTailBytes = kStaticTailSlots * (256 * 128 * 2 + 256 * 4);
// Device address and size of that array on the current device (looked up once per device).
int static_tail_scratch(void** ptr, int64_t* bytes);

static_assert(sizeof(AttnArgs) <= 4096, "the kernel arguments travel in the 4 KB kernarg segment");

int launch_attn(const AttnArgs& a, int D, int n_jobs, hipStream_t stream, void* workspace = nullptr,
                int64_t workspace_bytes = 0, bool balance = false);

}  // namespace dt
