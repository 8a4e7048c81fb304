// Measurement aids of the benchmark (libditango_probes.so; declared in include/ditango_probes.h).  They
// replace nothing in the reference and are not part of the drop-in library: three micro-benchmarks that
// put a number next to the nominal peaks -- what this part sustains for back-to-back MFMAs, for MFMAs
// beside the online softmax's vector instructions, and for streaming reads in the merge kernel's pattern.
#include <cstdarg>
#include <cstdio>

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ditango_probes.h"
#include "dt_common.h"

static thread_local char g_probe_error[256] = "";

static void probe_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_probe_error, sizeof(g_probe_error), fmt, ap);
  va_end(ap);
}

static int probe_fail(hipError_t e, const char* what) {
  if (e == hipSuccess) return DTP_OK;
  probe_error("%s: %s", what, hipGetErrorString(e));
  return DTP_ERR_HIP;
}

extern "C" const char* dtp_last_error(void) { return g_probe_error; }

namespace dt {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeThreads = 512;  // the attention kernel's workgroup: 8 wavefronts, two per SIMD
constexpr int kReadThreads = 256;   // the merge kernel's workgroup
constexpr int kBatch = 8;           // streams whose loads are in flight together, as in the merge kernel

// Measurement aid: back-to-back bf16 MFMAs on registers, nothing else -- the rate (and the shader
// clock) this part sustains when only the matrix pipes work, i.e. what the power limit leaves of the
// nominal peak.  Same launch shape as the attention kernel (512 threads, two wavefronts per SIMD).
// Four accumulators keep four independent MFMAs in flight; the operands rotate through four register
// sets of pseudo-random values so that the operand buses toggle as they do on real data.
__global__ __launch_bounds__(kProbeThreads, 2) void mfma_probe_kernel(float* sink, int iters) {
  const uint32_t lane = threadIdx.x;
  bf16x8 av[4], bv[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      uint32_t ha = (lane * 8u + e + 1u) * 2654435761u + j * 40503u;
      uint32_t hb = (lane * 8u + e + 7u) * 2246822519u + j * 9973u;
      ha ^= ha >> 15;
      hb ^= hb >> 13;
      av[j][e] = (__bf16)((float)(int)(ha & 255u) * (1.f / 128.f) - 1.f);
      bv[j][e] = (__bf16)((float)(int)(hb & 255u) * (1.f / 128.f) - 1.f);
    }
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  for (int i = 0; i < iters; i += 4) {   // iters is rounded up to a multiple of 4; register indices stay static
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[j], bv[(j + u) & 3], acc[j], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) total += acc[j][r];
  if (total == 12345.678f) sink[0] = total;   // keeps the MFMAs alive; (almost) never true
}

// Measurement aid: what two wavefronts of a SIMD can issue side by side.  Wavefronts 0-3 of a workgroup (one
// per SIMD) issue 4 * iters back-to-back MFMAs as above; wavefronts 4-7 (the other wavefront of each SIMD)
// issue, per MFMA of their neighbour, the vector instructions the online softmax spends per MFMA of the
// attention kernel: kMix = 1 (head dimension 128: 32 MFMAs per 64-key tile against 32 fma, 32 exp, 32 add
// and 16 cvt) one v_fma_f32, one v_exp_f32, one v_add_f32 and half a v_cvt_pk_bf16_f32; kMix = 2 (head
// dimension 64, half the MFMAs per softmax element) twice that; kMix = 0 nothing (the MFMA wavefronts alone).
// The launch reserves the attention kernel's LDS for that head dimension, so one (128) or two (64) workgroups share a CU as there.
// The instructions are written out so that the mix is exactly this; their values do not matter.
template <int kMix>
__global__ __launch_bounds__(kProbeThreads, 2) void coissue_probe_kernel(float* sink, int iters) {
  extern __shared__ __attribute__((aligned(16))) uint8_t probe_lds[];   // unused: sized by the launch to set the occupancy
  const uint32_t lane = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  float total = 0.f;
  if (wave < 4) {
    bf16x8 av[4], bv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        uint32_t ha = (lane * 8u + e + 1u) * 2654435761u + j * 40503u;
        uint32_t hb = (lane * 8u + e + 7u) * 2246822519u + j * 9973u;
        ha ^= ha >> 15;
        hb ^= hb >> 13;
        av[j][e] = (__bf16)((float)(int)(ha & 255u) * (1.f / 128.f) - 1.f);
        bv[j][e] = (__bf16)((float)(int)(hb & 255u) * (1.f / 128.f) - 1.f);
      }
    f32x16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
    for (int i = 0; i < iters; i += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[j], bv[(j + u) & 3], acc[j], 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) total += acc[j][r];
  } else if (kMix > 0) {
    float s[8], t[8], rs0 = 0.f, rs1 = 0.f;
    const float c = 0.18f, m = -0.25f;
#pragma unroll
    for (int e = 0; e < 8; ++e) s[e] = (float)(int)((lane * 8u + e) & 63u) * 0.05f - 1.6f;
    uint32_t pk = 0;
    for (int i = 0; i < iters; ++i) {   // one trip = the vector work beside 4 MFMAs
#pragma unroll
      for (int e = 0; e < 4 * kMix; ++e) {
        asm volatile("v_fma_f32 %0, %1, %2, %3" : "=v"(t[e]) : "v"(s[e]), "v"(c), "v"(m));
        asm volatile("v_exp_f32 %0, %0" : "+v"(t[e]));
      }
#pragma unroll
      for (int e = 0; e < 4 * kMix; e += 2) {
        asm volatile("v_add_f32 %0, %1, %0" : "+v"(rs0) : "v"(t[e]));
        asm volatile("v_add_f32 %0, %1, %0" : "+v"(rs1) : "v"(t[e + 1]));
        asm volatile("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(pk) : "v"(t[e]), "v"(t[e + 1]));
      }
    }
    total = rs0 + rs1 + (float)pk;
  }
  if (total == 12345.678f) sink[0] = total;   // keeps the work alive; (almost) never true
}

// Yardstick for the kernels above: reads n streams the way the merge kernel reads its states
// (a workgroup takes 32 consecutive 256-byte rows of every stream, 16 bytes per lane, all streams of
// a batch of 8 in flight before the first use) and discards the data.
struct ProbeArgs {
  const uint8_t* stream[DTP_MAX_STREAMS];
  int32_t n;
  int64_t rows;  // 256-byte rows per stream
  uint32_t* sink;
};

__global__ __launch_bounds__(kReadThreads) void hbm_read_probe_kernel(const ProbeArgs a) {
  const int64_t row = (int64_t)blockIdx.x * 32 + threadIdx.x / 16;
  const int c = threadIdx.x % 16;
  uint32_t acc = 0;
  for (int s0 = 0; s0 < a.n; s0 += kBatch) {
    u32x4 v[kBatch][2];
#pragma unroll
    for (int s = 0; s < kBatch; ++s)
#pragma unroll
      for (int p = 0; p < 2; ++p) {
        const int64_t r = row + 16 * p;
        v[s][p] = u32x4{0u, 0u, 0u, 0u};
        if (s0 + s < a.n && r < a.rows) v[s][p] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(a.stream[s0 + s] + r * 256 + 16 * c));
      }
#pragma unroll
    for (int s = 0; s < kBatch; ++s)
#pragma unroll
      for (int p = 0; p < 2; ++p) acc ^= v[s][p].x ^ v[s][p].y ^ v[s][p].z ^ v[s][p].w;
  }
  // keeps the loads alive; a real store happens only for one bit pattern in 2^32 per lane
  if (acc == 0x9e3779b9u) a.sink[0] = acc;
}

// A kernel that does nothing: what a launch of a given grid costs before it moves a byte.
__global__ void empty_kernel() {}

}  // namespace dt

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

template <int kMix>
static int launch_coissue(int workgroups, int iters, size_t lds_bytes, float* sink, hipStream_t stream) {
  // more than 64 KB of dynamic LDS has to be allowed once per kernel and device
  static thread_local int allowed_dev = -1;
  int dev = 0;
  if (int rc = probe_fail(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (allowed_dev != dev) {
    if (int rc = probe_fail(hipFuncSetAttribute(reinterpret_cast<const void*>(&dt::coissue_probe_kernel<kMix>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, dt::kAttnLdsBytes128),
                              "hipFuncSetAttribute"))
      return rc;
    allowed_dev = dev;
  }
  hipLaunchKernelGGL(dt::coissue_probe_kernel<kMix>, dim3((unsigned)workgroups), dim3(dt::kProbeThreads), lds_bytes, stream, sink, iters);
  return probe_fail(hipGetLastError(), "coissue_probe launch");
}

extern "C" int dtp_coissue_probe(int32_t workgroups, int32_t iters, int32_t head_dim, int32_t with_softmax, float* sink,
                                void* stream) {
  if (workgroups <= 0 || iters <= 0 || iters % 4 != 0 || !sink || (head_dim != 64 && head_dim != 128)) {
    probe_error("co-issue probe: workgroups and iters must be positive, iters a multiple of 4, head_dim 64 or 128, and sink non-null");
    return DTP_ERR_INVALID;
  }
  // the attention kernel's LDS footprint decides how many workgroups share a CU, as it does there
  const size_t lds = head_dim == 128 ? dt::kAttnLdsBytes128 : dt::kAttnLdsBytes64;
  if (!with_softmax) return launch_coissue<0>(workgroups, iters, lds, sink, (hipStream_t)stream);
  if (head_dim == 128) return launch_coissue<1>(workgroups, iters, lds, sink, (hipStream_t)stream);
  return launch_coissue<2>(workgroups, iters, lds, sink, (hipStream_t)stream);
}

extern "C" int dtp_mfma_probe(int32_t workgroups, int32_t iters, float* sink, void* stream) {
  if (workgroups <= 0 || iters <= 0 || iters % 4 != 0 || !sink) {
    probe_error("mfma probe: workgroups and iters must be positive, iters a multiple of 4, and sink non-null");
    return DTP_ERR_INVALID;
  }
  hipLaunchKernelGGL(dt::mfma_probe_kernel, dim3((unsigned)workgroups), dim3(dt::kProbeThreads), 0, (hipStream_t)stream, sink, iters);
  return probe_fail(hipGetLastError(), "mfma_probe launch");
}

extern "C" int dtp_hbm_read_probe(const void* const* streams, int32_t n_streams, int64_t bytes, uint32_t* sink,
                                 void* stream) {
  if (!streams || !sink || n_streams <= 0 || n_streams > DTP_MAX_STREAMS || bytes <= 0 || (bytes % 256)) {
    probe_error("read probe: need 1..%d streams of a positive multiple of 256 bytes and a sink", DTP_MAX_STREAMS);
    return DTP_ERR_INVALID;
  }
  dt::ProbeArgs a{};
  for (int i = 0; i < n_streams; ++i) {
    if (!streams[i] || !aligned16(streams[i])) {
      probe_error("read probe: stream %d is null or misaligned", i);
      return DTP_ERR_INVALID;
    }
    a.stream[i] = static_cast<const uint8_t*>(streams[i]);
  }
  a.n = n_streams;
  a.rows = bytes / 256;
  a.sink = sink;
  const int64_t wgs = (a.rows + 31) / 32;
  if (wgs > 0x7fffffffLL) {
    probe_error("read probe grid too large");
    return DTP_ERR_INVALID;
  }
  hipLaunchKernelGGL(dt::hbm_read_probe_kernel, dim3((unsigned)wgs), dim3(dt::kReadThreads), 0, (hipStream_t)stream, a);
  return probe_fail(hipGetLastError(), "hbm_read_probe launch");
}

extern "C" int dtp_empty_launch(int32_t workgroups, int32_t threads, void* stream) {
  if (workgroups <= 0 || threads <= 0 || threads > 1024 || threads % 64 != 0) {
    probe_error("empty launch: need a positive grid and 64..1024 threads in multiples of 64");
    return DTP_ERR_INVALID;
  }
  hipLaunchKernelGGL(dt::empty_kernel, dim3((unsigned)workgroups), dim3((unsigned)threads), 0, (hipStream_t)stream);
  return probe_fail(hipGetLastError(), "empty launch");
}
