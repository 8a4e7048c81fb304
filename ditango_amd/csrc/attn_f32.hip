// Chunk attention in fp32 from fp32 inputs: out = softmax(q k^T * scale) v and the natural-log lse.
//
// The bf16 MFMA kernel (attn_fwd.hip) is the path of the model-sized configurations; this one exists
// for callers that hold fp32 tensors and want the attention of THOSE numbers, not of their bf16
// roundings -- the reference's CPU-runnable configuration (fp32, 512 queries x 4 chunks of 512 keys,
// 4 heads, d = 64, which the reference runs on its torch math path because flash_attn_func takes no
// fp32).  Everything is fp32 on the vector ALU with expf / logf, so results agree with an fp32 or fp64
// closed form to rounding error.  It is not tuned: about 1 TFLOP/s.
//
// One workgroup of 256 threads = 64 queries of one (batch, head).  Key tiles of 64 go through the
// LDS.  Thread (query, g), g = 0..3: scores of the 16 keys {g, g + 4, ...} of the tile for its query,
// online softmax shared by the 4 threads of a query through lane exchanges, then the accumulation of
// the query's output elements [g * D/4, (g + 1) * D/4) over all 64 keys (probabilities pass through
// the LDS).
#include <cmath>

#include "dt_common.h"

namespace dt {
namespace {

constexpr int kThreadsF32 = 256;
constexpr int kBQF = 64;   // queries per workgroup
constexpr int kBKF = 64;   // keys per tile

struct AttnF32Args {
  const float* q;
  const float* k;
  const float* v;
  float* out;
  float* lse;
  int64_t q_sb, q_ss, q_sh, kv_sb, kv_ss, kv_sh;
  int32_t B, H, Sq, Sk;
  float scale;
};

template <int D>
struct F32Lds {
  static constexpr int kPitch = D + 1;             // rows of Q / K / V: odd pitch, no bank conflicts across rows
  static constexpr int kPitchP = kBKF + 1;
  static constexpr int kFloats = 3 * kBQF * kPitch + kBQF * kPitchP;
  static constexpr int kBytes = kFloats * 4;
};

template <int D>
__global__ __launch_bounds__(kThreadsF32) void attn_f32_kernel(const AttnF32Args a) {
  using L = F32Lds<D>;
  extern __shared__ __attribute__((aligned(16))) float lds_f32[];
  float* qs = lds_f32;                       // [64][D+1]
  float* ks = qs + kBQF * L::kPitch;         // [64][D+1]
  float* vs = ks + kBKF * L::kPitch;         // [64][D+1]
  float* ps = vs + kBKF * L::kPitch;         // [64][65]
  const int tid = threadIdx.x;
  const int qi = tid >> 2, g = tid & 3;
  const int bh = blockIdx.y;
  const int b = bh / a.H, h = bh - b * a.H;
  const int q0 = blockIdx.x * kBQF;
  constexpr int kDG = D / 4;                 // output elements of a query per thread

  // Q tile -> LDS (rows past Sq repeat the last row; their results are not stored)
  for (int i = tid; i < kBQF * D; i += kThreadsF32) {
    const int r = i / D, d = i - r * D;
    int row = q0 + r;
    if (row > a.Sq - 1) row = a.Sq - 1;
    qs[r * L::kPitch + d] = a.q[(int64_t)b * a.q_sb + (int64_t)row * a.q_ss + (int64_t)h * a.q_sh + d];
  }
  float m = -INFINITY, l = 0.f;
  float o[kDG];
#pragma unroll
  for (int d = 0; d < kDG; ++d) o[d] = 0.f;

  for (int k0 = 0; k0 < a.Sk; k0 += kBKF) {
    __syncthreads();   // the previous tile's K / V / P are no longer read (and Q is in place)
    for (int i = tid; i < kBKF * D; i += kThreadsF32) {
      const int r = i / D, d = i - r * D;
      const int key = k0 + r;
      const bool in = key < a.Sk;
      const int64_t off = (int64_t)b * a.kv_sb + (int64_t)(in ? key : 0) * a.kv_ss + (int64_t)h * a.kv_sh + d;
      ks[r * L::kPitch + d] = in ? a.k[off] : 0.f;
      vs[r * L::kPitch + d] = in ? a.v[off] : 0.f;
    }
    __syncthreads();
    // scores of this thread's 16 keys
    float s[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) s[j] = 0.f;
    const float* qrow = qs + qi * L::kPitch;
    for (int d = 0; d < D; ++d) {
      const float qd = qrow[d];
#pragma unroll
      for (int j = 0; j < 16; ++j) s[j] = fmaf(qd, ks[(4 * j + g) * L::kPitch + d], s[j]);
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      s[j] = (k0 + 4 * j + g < a.Sk) ? s[j] * a.scale : -INFINITY;
      tmax = fmaxf(tmax, s[j]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 1));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 2));
    const float m_new = fmaxf(m, tmax);        // finite: every tile has at least one key
    const float alpha = expf(m - m_new);       // exp(-inf) = 0 on the first tile
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float p = expf(s[j] - m_new);
      psum += p;
      ps[qi * L::kPitchP + 4 * j + g] = p;
    }
    psum += __shfl_xor(psum, 1);
    psum += __shfl_xor(psum, 2);
    l = l * alpha + psum;
    m = m_new;
#pragma unroll
    for (int d = 0; d < kDG; ++d) o[d] *= alpha;
    __syncthreads();   // the probabilities of all 4 threads of a query are in the LDS
    const float* prow = ps + qi * L::kPitchP;
    for (int key = 0; key < kBKF; ++key) {
      const float p = prow[key];
      const float* vrow = vs + key * L::kPitch + g * kDG;
#pragma unroll
      for (int d = 0; d < kDG; ++d) o[d] = fmaf(p, vrow[d], o[d]);
    }
  }
  const int row = q0 + qi;
  if (row < a.Sq) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    float* dst = a.out + (((int64_t)b * a.Sq + row) * a.H + h) * D + g * kDG;
#pragma unroll
    for (int d = 0; d < kDG; ++d) dst[d] = o[d] * inv;
    if (g == 0) a.lse[((int64_t)b * a.H + h) * a.Sq + row] = l > 0.f ? m + logf(l) : -INFINITY;
  }
}

template <int D>
int launch_f32(const AttnF32Args& a, hipStream_t stream) {
  static thread_local int allowed_dev = -1;
  int dev = 0;
  if (int rc = hip_fail(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (allowed_dev != dev) {
    if (int rc = hip_fail(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_f32_kernel<D>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, F32Lds<D>::kBytes),
                          "hipFuncSetAttribute"))
      return rc;
    allowed_dev = dev;
  }
  const dim3 grid((unsigned)((a.Sq + kBQF - 1) / kBQF), (unsigned)(a.B * a.H), 1);
  hipLaunchKernelGGL(attn_f32_kernel<D>, grid, dim3(kThreadsF32), F32Lds<D>::kBytes, stream, a);
  return hip_fail(hipGetLastError(), "attn_f32 launch");
}

}  // namespace
}  // namespace dt

using namespace dt;

extern "C" int dt_attn_chunk_f32_fwd(const float* q, const float* k, const float* v, float* out, float* lse, int32_t B,
                                     int32_t Sq, int32_t Sk, int32_t H, int32_t D, int64_t q_sb, int64_t q_ss,
                                     int64_t q_sh, int64_t kv_sb, int64_t kv_ss, int64_t kv_sh, float softmax_scale,
                                     void* stream) {
  if (B <= 0 || Sq <= 0 || H <= 0 || Sk < 0) {
    set_error("B, Sq, H must be positive and Sk non-negative (got %d, %d, %d, %d)", B, Sq, H, Sk);
    return DT_ERR_INVALID;
  }
  if (D != 64 && D != 128) {
    set_error("head dim %d not built (64 and 128 are)", D);
    return DT_ERR_UNSUPPORTED;
  }
  if (!q || !out || !lse || (Sk > 0 && (!k || !v))) {
    set_error("null pointer argument");
    return DT_ERR_INVALID;
  }
  if ((int64_t)B * H > 65535) {
    set_error("B * H = %lld exceeds the grid's second dimension", (long long)B * H);
    return DT_ERR_INVALID;
  }
  AttnF32Args a{};
  a.q = q; a.k = k; a.v = v; a.out = out; a.lse = lse;
  a.q_sb = q_sb; a.q_ss = q_ss; a.q_sh = q_sh;
  a.kv_sb = kv_sb; a.kv_ss = kv_ss; a.kv_sh = kv_sh;
  a.B = B; a.H = H; a.Sq = Sq; a.Sk = Sk;
  a.scale = softmax_scale > 0.f ? softmax_scale : 1.0f / std::sqrt((float)D);
  if (D == 128) return launch_f32<128>(a, (hipStream_t)stream);
  return launch_f32<64>(a, (hipStream_t)stream);
}
