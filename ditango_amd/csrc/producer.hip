// Producer side of an attention call: per-head QK normalisation and rotary position
// embedding in one pass over HBM, written as the bf16 (or fp16) [B,S,H,D] tensor the attention
// kernel reads.  Replaces the chains of eager ops in front of the attention call at
// executor/cogvideox/attention_processor.py:55-71 (LayerNorm over D, interleaved RoPE on the
// video tokens only), executor/hunyuanvideo/hunyuan_transformer.py:177-191 (RMSNorm over D,
// interleaved RoPE) and executor/step/blocks.py:66-75 with executor/step/rope.py:13-90
// (RMSNorm, rotate-half RoPE on three sections of D).
//
// HBM-bound: rows*D*2 bytes in, rows*D*2 bytes out; the cos/sin tables are shared by all
// heads of a token and stay in cache.
#include "dt_common.h"

namespace dt {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kHeads = 8;  // heads of one token handled by a lane group with one set of table loads

struct PrepArgs {
  const uint16_t* x;   // bfloat16, or IEEE half (DT_IO_FP16)
  uint16_t* y;
  int64_t xs_b, xs_s, xs_h;
  int32_t B, S, H;
  int32_t norm, rope, rounding;
  const float* w;
  const float* bias;
  float eps;
  float out_scale;  // multiplies the result before its rounding to the output type
  const float* cos;
  const float* sin;
  int64_t tab_sb;
  int32_t rope_begin, rope_end;
  int32_t sec_end[3];  // rotate-half sections [0,e0) [e0,e1) [e1,D); unused ones end at D
};

// kHalf: the 16-bit type is IEEE half, else bfloat16
template <bool kHalf>
__device__ __forceinline__ float round16(float v) {
  if constexpr (kHalf) return (float)(_Float16)v;
  else return (float)(__bf16)v;
}

template <bool kHalf>
__device__ __forceinline__ uint32_t pack2(float lo, float hi) {
  f32x2 f;
  f.x = lo;
  f.y = hi;
  // round to nearest even
  if constexpr (kHalf) return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));
  else return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}

template <bool kHalf>
__device__ __forceinline__ void unpack8(const u32x4 r, float (&v)[8]) {
  const uint32_t u[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (kHalf) {
      const f32x2 f = __builtin_convertvector(__builtin_bit_cast(f16x2, u[i]), f32x2);
      v[2 * i] = f.x;
      v[2 * i + 1] = f.y;
    } else {
      v[2 * i] = __builtin_bit_cast(float, u[i] << 16);
      v[2 * i + 1] = __builtin_bit_cast(float, u[i] & 0xffff0000u);
    }
  }
}

template <int G>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int m = 1; m < G; m <<= 1) v += __shfl_xor(v, m);
  return v;
}

// One lane group of D/8 lanes handles up to kHeads heads of one token; a lane owns the
// 8 consecutive elements [8c, 8c+8) of each of those rows.
template <int D, bool kHalf>
__global__ __launch_bounds__(kThreads) void qk_norm_rope_kernel(const PrepArgs a) {
  constexpr int G = D / 8;
  const int c = threadIdx.x % G;
  const int hgroups = (a.H + kHeads - 1) / kHeads;
  const int64_t n_items = (int64_t)a.B * a.S * hgroups;
  const int64_t item = (int64_t)blockIdx.x * (kThreads / G) + threadIdx.x / G;
  if (item >= n_items) return;  // a lane group leaves as a whole; the exchanges below stay inside a group
  const int hg = (int)(item % hgroups);
  const int64_t bs = item / hgroups;
  const int s = (int)(bs % a.S);
  const int b = (int)(bs / a.S);
  const int h0 = hg * kHeads;
  const int nh = (a.H - h0 < kHeads) ? a.H - h0 : kHeads;
  const int d0 = 8 * c;

  const uint16_t* xp = a.x + (int64_t)b * a.xs_b + (int64_t)s * a.xs_s + (int64_t)h0 * a.xs_h + d0;
  u32x4 raw[kHeads];
#pragma unroll
  for (int r = 0; r < kHeads; ++r)
    if (r < nh) raw[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xp + (int64_t)r * a.xs_h));

  const bool do_rope = a.rope != DT_ROPE_NONE && s >= a.rope_begin && s < a.rope_end;
  float cs[8], sn[8];
  if (do_rope) {
    const int64_t t = (int64_t)b * a.tab_sb + (int64_t)(s - a.rope_begin) * D + d0;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(a.cos + t);
    const f32x4 c1 = *reinterpret_cast<const f32x4*>(a.cos + t + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(a.sin + t);
    const f32x4 s1 = *reinterpret_cast<const f32x4*>(a.sin + t + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      cs[i] = c0[i]; cs[4 + i] = c1[i];
      sn[i] = s0[i]; sn[4 + i] = s1[i];
    }
  }
  float w[8], bias[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    w[i] = 1.0f;
    bias[i] = 0.0f;
  }
  if (a.norm != DT_NORM_NONE && a.w) {
    const f32x4 w0 = *reinterpret_cast<const f32x4*>(a.w + d0);
    const f32x4 w1 = *reinterpret_cast<const f32x4*>(a.w + d0 + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { w[i] = w0[i]; w[4 + i] = w1[i]; }
  }
  if (a.norm == DT_NORM_LAYER && a.bias) {
    const f32x4 b0 = *reinterpret_cast<const f32x4*>(a.bias + d0);
    const f32x4 b1 = *reinterpret_cast<const f32x4*>(a.bias + d0 + 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) { bias[i] = b0[i]; bias[4 + i] = b1[i]; }
  }

  // rotate-half partner of this lane inside its section
  int partner = 0;
  float rot_sign = 0.0f;
  if (a.rope == DT_ROPE_HALVES) {
    int lo = 0, hi = a.sec_end[0];
    if (d0 >= a.sec_end[0]) { lo = a.sec_end[0]; hi = a.sec_end[1]; }
    if (d0 >= a.sec_end[1]) { lo = a.sec_end[1]; hi = a.sec_end[2]; }
    const int half8 = (hi - lo) / 16;  // half a section, in lanes
    const bool first = d0 < lo + (hi - lo) / 2;
    partner = (int)(threadIdx.x & 63) + (first ? half8 : -half8);
    rot_sign = first ? -1.0f : 1.0f;
  }
  const bool round_norm = (a.rounding & DT_ROUND_NORM_BF16) != 0;
  const bool round_rope = (a.rounding & DT_ROUND_ROPE_BF16) != 0;

  uint16_t* yp = a.y + (((int64_t)b * a.S + s) * a.H + h0) * D + d0;
#pragma unroll
  for (int r = 0; r < kHeads; ++r) {
    if (r >= nh) break;
    float v[8];
    unpack8<kHalf>(raw[r], v);
    if (a.norm == DT_NORM_RMS) {
      float ss = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += v[i] * v[i];
      ss = group_sum<G>(ss);
      const float rs = 1.0f / sqrtf(ss * (1.0f / D) + a.eps);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = v[i] * rs;
        if (round_norm) t = round16<kHalf>(t);
        t *= w[i];
        if (round_norm) t = round16<kHalf>(t);
        v[i] = t;
      }
    } else if (a.norm == DT_NORM_LAYER) {
      float sum = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) sum += v[i];
      const float mean = group_sum<G>(sum) * (1.0f / D);
      float ss = 0.0f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        v[i] -= mean;
        ss += v[i] * v[i];
      }
      ss = group_sum<G>(ss);
      const float rs = 1.0f / sqrtf(ss * (1.0f / D) + a.eps);
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        float t = v[i] * rs * w[i] + bias[i];
        if (round_norm) t = round16<kHalf>(t);
        v[i] = t;
      }
    }
    if (a.rope != DT_ROPE_NONE) {  // uniform; the exchange runs for all lanes of the wavefront
      float rot[8];
      if (a.rope == DT_ROPE_INTERLEAVED) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          rot[2 * i] = -v[2 * i + 1];
          rot[2 * i + 1] = v[2 * i];
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) rot[i] = rot_sign * __shfl(v[i], partner);
      }
      if (do_rope) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (round_rope)
            v[i] = round16<kHalf>(v[i] * cs[i]) + round16<kHalf>(rot[i] * sn[i]);
          else
            v[i] = v[i] * cs[i] + rot[i] * sn[i];
        }
      }
    }
    if (a.out_scale != 1.0f) {  // uniform
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] *= a.out_scale;
    }
    u32x4 o;
    o.x = pack2<kHalf>(v[0], v[1]);
    o.y = pack2<kHalf>(v[2], v[3]);
    o.z = pack2<kHalf>(v[4], v[5]);
    o.w = pack2<kHalf>(v[6], v[7]);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(yp + (int64_t)r * D));
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace
}  // namespace dt

using namespace dt;

extern "C" int dt_qk_norm_rope(const void* x, int64_t x_stride_b, int64_t x_stride_s, int64_t x_stride_h, void* y,
                               int32_t B, int32_t S, int32_t H, int32_t D, int32_t norm, const float* weight,
                               const float* bias, float eps, int32_t rope, const float* cos, const float* sin,
                               int64_t table_stride_b, int32_t rope_begin, int32_t rope_end,
                               const int32_t* sections, int32_t n_sections, int32_t rounding, float out_scale,
                               void* stream) {
  if (B <= 0 || S <= 0 || H <= 0) {
    set_error("B, S, H must be positive (got %d, %d, %d)", B, S, H);
    return DT_ERR_INVALID;
  }
  if (D != 64 && D != 128) {
    set_error("head dim %d not built (64 and 128 are)", D);
    return DT_ERR_UNSUPPORTED;
  }
  if (!x || !y || !aligned16(x) || !aligned16(y) || (x_stride_b & 7) || (x_stride_s & 7) || (x_stride_h & 7)) {
    set_error("x and y must be non-null, 16-byte aligned, with strides that are multiples of 8 elements");
    return DT_ERR_INVALID;
  }
  if (norm < DT_NORM_NONE || norm > DT_NORM_LAYER || rope < DT_ROPE_NONE || rope > DT_ROPE_HALVES ||
      (rounding & ~(DT_ROUND_NORM_BF16 | DT_ROUND_ROPE_BF16 | DT_IO_FP16))) {
    set_error("bad norm / rope / rounding code (%d, %d, %d)", norm, rope, rounding);
    return DT_ERR_INVALID;
  }
  if (!(out_scale > 0.0f) || !(out_scale < INFINITY)) {
    set_error("out_scale must be positive and finite (1 for none)");
    return DT_ERR_INVALID;
  }
  if ((weight && !aligned16(weight)) || (bias && !aligned16(bias))) {
    set_error("weight and bias must be 16-byte aligned");
    return DT_ERR_INVALID;
  }
  PrepArgs a{};
  a.x = static_cast<const uint16_t*>(x);
  a.y = static_cast<uint16_t*>(y);
  a.xs_b = x_stride_b; a.xs_s = x_stride_s; a.xs_h = x_stride_h;
  a.B = B; a.S = S; a.H = H;
  a.norm = norm; a.rope = rope; a.rounding = rounding & (DT_ROUND_NORM_BF16 | DT_ROUND_ROPE_BF16);
  const bool half = (rounding & DT_IO_FP16) != 0;
  a.w = weight; a.bias = bias; a.eps = eps;
  a.out_scale = out_scale;
  a.sec_end[0] = a.sec_end[1] = a.sec_end[2] = D;
  if (rope != DT_ROPE_NONE) {
    if (rope_begin < 0 || rope_end > S || rope_begin > rope_end) {
      set_error("rope rows [%d, %d) outside [0, %d)", rope_begin, rope_end, S);
      return DT_ERR_INVALID;
    }
    if (rope_begin < rope_end && (!cos || !sin || !aligned16(cos) || !aligned16(sin) || (table_stride_b & 3))) {
      set_error("cos/sin tables must be non-null and 16-byte aligned");
      return DT_ERR_INVALID;
    }
    a.cos = cos; a.sin = sin; a.tab_sb = table_stride_b;
    a.rope_begin = rope_begin; a.rope_end = rope_end;
    if (rope == DT_ROPE_HALVES) {
      if (n_sections < 0 || n_sections > 3 || (n_sections > 0 && !sections)) {
        set_error("rotate-half RoPE takes 0..3 sections");
        return DT_ERR_INVALID;
      }
      int end = 0;
      for (int i = 0; i < n_sections; ++i) {
        if (sections[i] <= 0 || (sections[i] & 15)) {
          set_error("section %d has %d elements: need a positive multiple of 16", i, sections[i]);
          return DT_ERR_INVALID;
        }
        end += sections[i];
        a.sec_end[i] = end;
      }
      if (n_sections > 0 && end != D) {
        set_error("sections sum to %d, head dim is %d", end, D);
        return DT_ERR_INVALID;
      }
      for (int i = n_sections > 0 ? n_sections : 1; i < 3; ++i) a.sec_end[i] = D;
    }
  }
  const int groups_per_wg = kThreads / (D / 8);
  const int64_t items = (int64_t)B * S * ((H + kHeads - 1) / kHeads);
  const int64_t wgs = (items + groups_per_wg - 1) / groups_per_wg;
  if (wgs > 0x7fffffffLL) {
    set_error("too many rows (%lld workgroups)", (long long)wgs);
    return DT_ERR_INVALID;
  }
  const dim3 grid((unsigned)wgs), block(kThreads);
  if (D == 128) {
    if (half) hipLaunchKernelGGL((qk_norm_rope_kernel<128, true>), grid, block, 0, (hipStream_t)stream, a);
    else hipLaunchKernelGGL((qk_norm_rope_kernel<128, false>), grid, block, 0, (hipStream_t)stream, a);
  } else {
    if (half) hipLaunchKernelGGL((qk_norm_rope_kernel<64, true>), grid, block, 0, (hipStream_t)stream, a);
    else hipLaunchKernelGGL((qk_norm_rope_kernel<64, false>), grid, block, 0, (hipStream_t)stream, a);
  }
  return hip_fail(hipGetLastError(), "qk_norm_rope launch");
}
