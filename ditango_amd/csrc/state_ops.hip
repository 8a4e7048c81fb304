// HBM-bound kernels around the attention-state cache (gfx950):
//   * N-way LSE merge       (utils.py:24-84 of the reference, fused to one pass)
//   * state copy / convert  (cache store and load, core/cache.py:75-84)
//   * schedule builder      (per-chunk generalisation of core/attention.py:90-116)
//   * relative-L1 sums      (utils.py:214-241)
//
// Work decomposition of the row-mapped copy kernel: one workgroup handles a run of
// consecutive queries of ONE (batch, head), a group of D/8 lanes owns one row
// (query, head), and the lse values of consecutive rows are consecutive floats in
// the [B,H,Sq] layout.  The merge works on 256-byte units instead (see there).
#include <algorithm>

#include "dt_common.h"

namespace dt {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kBatch = 8;       // states whose loads are in flight together (all states in one 16-bit type, 8 states and more)
constexpr int kBatchMixed = 4;  // ... when the launch mixes fp32 with 16-bit states, or merges fewer than 8 states

struct MergeArgs {
  int32_t n;
  int32_t B, Sq, H;
  const void* out[DT_MAX_MERGE];
  const float* lse[DT_MAX_MERGE];
  uint64_t fp32_mask;   // bit i: out[i] is fp32 (else a 16-bit type)
  uint64_t f16_mask;    // bit i: out[i] is IEEE half (neither bit: bfloat16)
  uint64_t bsh_mask;    // bit i: lse[i] is [B,Sq,H] (else [B,H,Sq])
  void* dst_out;
  float* dst_lse;
  int32_t dst_dtype;    // DT_BF16 / DT_FP32 / DT_FP16
  int32_t dst_bsh;
};

// The two 16-bit elements of a word, widened (f16: IEEE half, else bfloat16), and back (round to nearest even).
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void widen16x2(uint32_t w, bool f16, float& lo, float& hi) {
  if (f16) {
    const f32x2 f = __builtin_convertvector(__builtin_bit_cast(f16x2, w), f32x2);
    lo = f.x;
    hi = f.y;
  } else {
    lo = __uint_as_float(w << 16);
    hi = __uint_as_float(w & 0xffff0000u);
  }
}

__device__ __forceinline__ int64_t lse_index(bool bsh, int b, int h, int s, int H, int Sq) {
  return bsh ? ((int64_t)b * Sq + s) * H + h : ((int64_t)b * H + h) * Sq + s;
}

// A lane owns 8 elements of its row: [4c, 4c+4) and [D/2 + 4c, D/2 + 4c + 4), c = lane index
// within the row's lane group.  Every load/store instruction is then contiguous across the
// group (8 bytes per lane for the 16-bit types, 16 bytes per lane for fp32), for any dtype on either
// side; a lane owning 8 consecutive elements would write fp32 as two interleaved half-sector
// streams.
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
struct Row8 {
  u32x4 lo, hi;  // 16-bit types: lo.xy = first group, lo.zw = second group; fp32: lo / hi = the two groups
};

template <int D>
__device__ __forceinline__ Row8 load_row8(const void* base, bool fp32, int64_t row_elem, int c) {
  Row8 r;
  if (fp32) {
    const float* p = reinterpret_cast<const float*>(base) + row_elem + 4 * c;
    r.lo = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    r.hi = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p + D / 2));
  } else {
    const uint16_t* p = reinterpret_cast<const uint16_t*>(base) + row_elem + 4 * c;
    const u32x2 g0 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    const u32x2 g1 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p + D / 2));
    r.lo.x = g0.x; r.lo.y = g0.y; r.lo.z = g1.x; r.lo.w = g1.y;
    r.hi = r.lo;
  }
  return r;
}

__device__ __forceinline__ void unpack_row8(const Row8& r, int dtype, float (&x)[8]) {
  if (dtype == DT_FP32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = __uint_as_float(r.lo[i]);
      x[4 + i] = __uint_as_float(r.hi[i]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) widen16x2(r.lo[i], dtype == DT_FP16, x[2 * i], x[2 * i + 1]);
  }
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  f32x2 f;
  f.x = lo;
  f.y = hi;
  const bf16x2 b = __builtin_convertvector(f, bf16x2);  // round to nearest even
  return __builtin_bit_cast(uint32_t, b);
}
__device__ __forceinline__ uint32_t pack16x2(float lo, float hi, bool f16) {
  if (!f16) return pack_bf16x2(lo, hi);
  f32x2 f;
  f.x = lo;
  f.y = hi;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, f16x2));  // round to nearest even
}

template <int D>
__device__ __forceinline__ void store_row8(void* base, int dtype, int64_t row_elem, int c, const float (&x)[8]) {
  if (dtype == DT_FP32) {
    float* p = reinterpret_cast<float*>(base) + row_elem + 4 * c;
    u32x4 a, b;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[i] = __float_as_uint(x[i]);
      b[i] = __float_as_uint(x[4 + i]);
    }
    __builtin_nontemporal_store(a, reinterpret_cast<u32x4*>(p));
    __builtin_nontemporal_store(b, reinterpret_cast<u32x4*>(p + D / 2));
  } else {
    uint16_t* p = reinterpret_cast<uint16_t*>(base) + row_elem + 4 * c;
    const bool f16 = dtype == DT_FP16;
    u32x2 g0, g1;
    g0.x = pack16x2(x[0], x[1], f16);
    g0.y = pack16x2(x[2], x[3], f16);
    g1.x = pack16x2(x[4], x[5], f16);
    g1.y = pack16x2(x[6], x[7], f16);
    __builtin_nontemporal_store(g0, reinterpret_cast<u32x2*>(p));
    __builtin_nontemporal_store(g1, reinterpret_cast<u32x2*>(p + D / 2));
  }
}

// Workgroup -> (query run, batch*head) with the head index fastest: workgroups that run at
// the same time then cover whole [query][head][d] rows, i.e. contiguous memory, in every
// stream, instead of one 2*D-byte slice out of every H*2*D bytes.
__device__ __forceinline__ void decode_wg(int wg, int B, int H, int& st, int& b, int& h) {
  const int bh_count = B * H;
  st = wg / bh_count;
  const int bh = wg - st * bh_count;
  b = bh / H;
  h = bh - b * H;
}

// ---- N-way merge ------------------------------------------------------------------------------
// A group of 16 lanes owns one UNIT = 128 consecutive elements of the [B,Sq,H,D] tensors: one row
// at D = 128, two rows that are neighbours in memory at D = 64.  A lane owns elements [4c, 4c+4) and
// [64+4c, 64+4c+4) of its unit, so every load and store instruction of the group covers 128 (bf16) or
// 256 (fp32) contiguous bytes for either head dimension (a lane owning 8 consecutive elements would
// write fp32 as two interleaved half-sector streams); at D = 64 the two halves of a lane belong to
// two different rows and carry their own lse, maximum and denominator (with a lane group per 128-byte
// row instead, every load instruction touched half of each cache line: -10 to -30 % at D = 64).
// Units go to workgroups (16 per pass, P passes) in one of two ways:
//   MAP_LINEAR  consecutive units in memory order: every stream a workgroup reads is one contiguous
//               block, but its lse values in the [B,H,Sq] layout are one 32-byte sector apiece;
//   MAP_TILED   a tile of 4*P consecutive queries x 4 consecutive head units, tiles ordered head-fastest:
//               every row read is still part of a contiguous kilobyte that the neighbouring workgroup
//               continues, and the lse values of a head are a run of 4*P consecutive floats, i.e. whole
//               sectors at P = 2; two tiles that follow each other along the queries go to the same XCD
//               (fetched bytes 1.108 -> 1.029 x the state bytes at 8 states of 93 MB; what is left are
//               runs that straddle a 64-byte line because a head's lse row starts at any multiple of 4).
// States are consumed in branch-free, fully unrolled batches of kBatch (all loads of a batch are in
// flight before the first use; the pointers come from the kernel arguments with a uniform index, so
// they are scalar loads issued together) and folded with the running-maximum rescale; the remainder
// goes through a fully unrolled smaller batch.
constexpr int kUnitLanes = 16;
constexpr int kUnitsPerPass = kThreads / kUnitLanes;
constexpr int kTileHeadUnits = 4;
enum { MAP_LINEAR = 1, MAP_TILED = 2 };

template <int R>
struct UnitPos {           // where the R rows of a unit sit
  int b[R], h[R], s[R];
  bool live[R];
  int64_t elem;            // element offset of the unit in [B,Sq,H,D]
};

template <int R>
struct UnitAcc {
  float acc[8];
  float m[R], den[R];
};

template <int R, int NB, int P>
struct UnitRegs {
  float l[P][R][NB];
  u32x4 rb[P][NB];   // all states of one 16-bit type
  Row8 r[P][NB];     // mixed dtypes
};

template <int R, int NB, int FAST, int P>
__device__ __forceinline__ void unit_load(const MergeArgs& a, int i0, const UnitPos<R> (&u)[P], int cc,
                                          UnitRegs<R, NB, P>& g) {
#pragma unroll
  for (int j = 0; j < NB; ++j) {
    const int i = i0 + j;
    const float* lp = a.lse[i];
    const void* op = a.out[i];
    const bool bsh = (a.bsh_mask >> i) & 1;
    const bool f32 = (a.fp32_mask >> i) & 1;
#pragma unroll
    for (int p = 0; p < P; ++p) {
#pragma unroll
      for (int r = 0; r < R; ++r)
        g.l[p][r][j] = u[p].live[r] ? lp[lse_index(bsh, u[p].b[r], u[p].h[r], u[p].s[r], a.H, a.Sq)] : -INFINITY;
      const bool live_lo = u[p].live[0], live_hi = u[p].live[R - 1];
      if (FAST == 1 || FAST == 2) {
        const uint16_t* q = reinterpret_cast<const uint16_t*>(op) + u[p].elem + 4 * cc;
        u32x2 g0 = u32x2{0u, 0u}, g1 = u32x2{0u, 0u};
        if (live_lo) g0 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q));
        if (live_hi) g1 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q + 64));
        g.rb[p][j].x = g0.x; g.rb[p][j].y = g0.y; g.rb[p][j].z = g1.x; g.rb[p][j].w = g1.y;
      } else {
        Row8 v;
        v.lo = u32x4{0u, 0u, 0u, 0u};
        v.hi = v.lo;
        if (f32) {
          const float* q = reinterpret_cast<const float*>(op) + u[p].elem + 4 * cc;
          if (live_lo) v.lo = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q));
          if (live_hi) v.hi = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q + 64));
        } else {
          const uint16_t* q = reinterpret_cast<const uint16_t*>(op) + u[p].elem + 4 * cc;
          u32x2 g0 = u32x2{0u, 0u}, g1 = u32x2{0u, 0u};
          if (live_lo) g0 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q));
          if (live_hi) g1 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q + 64));
          v.lo.x = g0.x; v.lo.y = g0.y; v.lo.z = g1.x; v.lo.w = g1.y;
        }
        g.r[p][j] = v;
      }
    }
  }
}

template <int R, int NB, int FAST, int P>
__device__ __forceinline__ void unit_fold(const MergeArgs& a, int i0, const UnitRegs<R, NB, P>& g,
                                          UnitAcc<R> (&ua)[P]) {
  constexpr int kPer = 8 / R;   // elements of a lane that belong to one row
#pragma unroll
  for (int p = 0; p < P; ++p) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      float m_new = ua[p].m[r];
#pragma unroll
      for (int j = 0; j < NB; ++j) m_new = fmaxf(m_new, g.l[p][r][j]);
      if (m_new > -INFINITY) {
        const float rescale = __expf(ua[p].m[r] - m_new);  // exp(-inf) = 0 on the first non-empty batch
        ua[p].den[r] *= rescale;
#pragma unroll
        for (int k = 0; k < kPer; ++k) ua[p].acc[r * kPer + k] *= rescale;
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          const float w = __expf(g.l[p][r][j] - m_new);
          float x[8];
          if (FAST == 1 || FAST == 2) {
#pragma unroll
            for (int q = 0; q < 4; ++q) widen16x2(g.rb[p][j][q], FAST == 2, x[2 * q], x[2 * q + 1]);
          } else {
            const int i = i0 + j;
            const int other = (FAST == 0 && ((a.f16_mask >> i) & 1)) ? DT_FP16 : DT_BF16;
            unpack_row8(g.r[p][j], ((a.fp32_mask >> i) & 1) ? DT_FP32 : other, x);
          }
          ua[p].den[r] += w;
#pragma unroll
          for (int k = 0; k < kPer; ++k)
            ua[p].acc[r * kPer + k] = __builtin_fmaf(w, x[r * kPer + k], ua[p].acc[r * kPer + k]);
        }
        ua[p].m[r] = m_new;
      }
    }
  }
}

template <int R, int NB, int FAST, int P>
__device__ __forceinline__ void unit_batch(const MergeArgs& a, int i0, const UnitPos<R> (&u)[P], int cc,
                                           UnitAcc<R> (&ua)[P]) {
  UnitRegs<R, NB, P> g;
  unit_load<R, NB, FAST, P>(a, i0, u, cc, g);
  unit_fold<R, NB, FAST, P>(a, i0, g, ua);
}

template <int R, int FAST, int NB, int P>
__device__ __forceinline__ void unit_rest(const MergeArgs& a, int i0, int rest, const UnitPos<R> (&u)[P],
                                          int cc, UnitAcc<R> (&ua)[P]) {
  if constexpr (NB >= 1) {
    if (rest == NB) unit_batch<R, NB, FAST, P>(a, i0, u, cc, ua);
    else unit_rest<R, FAST, NB - 1, P>(a, i0, rest, u, cc, ua);
  }
}

// Where the P units of this lane group sit (see the two mappings above); false when the workgroup is one
// of those that pad the tiled grid.
template <int D, int MAP, int P>
__device__ __forceinline__ bool unit_positions(int B, int Sq, int H, UnitPos<128 / D> (&u)[P]) {
  constexpr int R = 128 / D;
  constexpr int kUnitsPerWg = kUnitsPerPass * P;
  constexpr int kTileQueries = kUnitsPerWg / kTileHeadUnits;
  constexpr int kTileQueriesPerPass = kUnitsPerPass / kTileHeadUnits;
  const int rr = threadIdx.x / kUnitLanes;
  const int64_t rows_total = (int64_t)B * Sq * H;
  int tb = 0, ts0 = 0, thu0 = 0;
  if constexpr (MAP == MAP_TILED) {
    const int n_hg = H / (R * kTileHeadUnits);
    const int n_qt = (Sq + kTileQueries - 1) / kTileQueries;
    // Two tiles that follow each other along the queries share the 64-byte lines of their lse runs.
    // Workgroups go to the 8 XCDs in turn; the pair is handed to ONE XCD as two consecutive workgroups
    // of it, so that the line is fetched into one L2 once instead of into two.
    const int n_qt2 = (n_qt + 1) >> 1;
    const uint32_t xcd = blockIdx.x & 7u, j = blockIdx.x >> 3;
    const uint32_t sup = (j >> 1) * 8u + xcd;
    if (sup >= (uint32_t)B * n_qt2 * n_hg) return false;
    const int hg = sup % n_hg;
    const int t = sup / n_hg;
    const int qt = 2 * (t % n_qt2) + (int)(j & 1u);
    if (qt >= n_qt) return false;
    tb = t / n_qt2;
    ts0 = qt * kTileQueries;
    thu0 = hg * kTileHeadUnits;
  }
#pragma unroll
  for (int p = 0; p < P; ++p) {
    if constexpr (MAP == MAP_TILED) {
      const int s = ts0 + p * kTileQueriesPerPass + rr / kTileHeadUnits;
      const int h0 = (thu0 + rr % kTileHeadUnits) * R;
      const bool ok = s < Sq;
      const int sc = ok ? s : 0;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        u[p].b[r] = tb;
        u[p].h[r] = h0 + r;
        u[p].s[r] = sc;
        u[p].live[r] = ok;
      }
      u[p].elem = (((int64_t)tb * Sq + sc) * H + h0) * D;
    } else {
      const int64_t unit = (int64_t)blockIdx.x * kUnitsPerWg + p * kUnitsPerPass + rr;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int64_t row = unit * R + r;
        u[p].live[r] = row < rows_total;
        const int64_t rc = u[p].live[r] ? row : 0;
        if (rows_total <= 0x7fffffffLL) {   // uniform: the common case divides in 32 bits
          const uint32_t bs = (uint32_t)rc / (uint32_t)H;
          u[p].h[r] = (int)((uint32_t)rc - bs * (uint32_t)H);
          u[p].b[r] = (int)(bs / (uint32_t)Sq);
          u[p].s[r] = (int)(bs - (uint32_t)u[p].b[r] * (uint32_t)Sq);
        } else {
          const int64_t bs = rc / H;
          u[p].h[r] = (int)(rc - bs * H);
          u[p].b[r] = (int)(bs / Sq);
          u[p].s[r] = (int)(bs - (int64_t)u[p].b[r] * Sq);
        }
      }
      u[p].elem = u[p].live[0] ? unit * 128 : 0;
    }
  }
  return true;
}

// Workgroups a launch over these units needs.
static int64_t unit_grid(int B, int Sq, int H, int D, bool tiled, int passes) {
  const int R = 128 / D;
  const int units_per_wg = kUnitsPerPass * passes;
  if (tiled) {
    // pairs of query tiles, 8 pairs (one per XCD) x 2 workgroups at a time
    const int tile_q = units_per_wg / kTileHeadUnits;
    const int64_t n_qt2 = ((Sq + tile_q - 1) / tile_q + 1) / 2;
    return 16 * (((int64_t)B * n_qt2 * (H / (R * kTileHeadUnits)) + 7) / 8);
  }
  const int64_t units = ((int64_t)B * Sq * H + R - 1) / R;
  return (units + units_per_wg - 1) / units_per_wg;
}
static bool unit_tiles_fit(int H, int D) { return H % ((128 / D) * kTileHeadUnits) == 0; }

// FAST: 1 = every state bfloat16, 2 = every state IEEE half (one decode, no per-state dtype); mixed dtypes:
// 3 = bfloat16 and fp32 only, 0 = any of the three.
// KB: states per batch.  A mixed-dtype batch holds twice the bytes per state and pass of a 16-bit one; in batches of
// 8 that is 106 registers and 4 resident wavefronts per SIMD (against 70 and 7), in batches of 4 again 70 and 7 --
// and 5.8 instead of 4.3 TB/s on an fp32 running state merged with four bf16 blocks at the HunyuanVideo share (the
// running-state update of utils.py:24-40 as the reference calls it, two states: 5.7 instead of 4.9 TB/s).
template <int D, int FAST, int MAP, int P, int KB>
__global__ __launch_bounds__(kThreads) void merge_states_kernel(const MergeArgs a) {
  constexpr int R = 128 / D;
  const int cc = threadIdx.x % kUnitLanes;
  UnitPos<R> u[P];
  UnitAcc<R> ua[P];
  if (!unit_positions<D, MAP, P>(a.B, a.Sq, a.H, u)) return;
#pragma unroll
  for (int p = 0; p < P; ++p) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      ua[p].m[r] = -INFINITY;
      ua[p].den[r] = 0.f;
    }
#pragma unroll
    for (int k = 0; k < 8; ++k) ua[p].acc[k] = 0.f;
  }
  int i0 = 0;
  for (; i0 + KB <= a.n; i0 += KB) unit_batch<R, KB, FAST, P>(a, i0, u, cc, ua);
  unit_rest<R, FAST, KB - 1, P>(a, i0, a.n - i0, u, cc, ua);
  constexpr int kPer = 8 / R;
#pragma unroll
  for (int p = 0; p < P; ++p) {
    float o[8];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float inv = ua[p].den[r] > 0.f ? 1.f / ua[p].den[r] : 0.f;
#pragma unroll
      for (int k = 0; k < kPer; ++k) o[r * kPer + k] = ua[p].acc[r * kPer + k] * inv;
    }
    const bool live_lo = u[p].live[0], live_hi = u[p].live[R - 1];
    if (a.dst_dtype == DT_FP32) {
      float* q = reinterpret_cast<float*>(a.dst_out) + u[p].elem + 4 * cc;
      u32x4 v0, v1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v0[i] = __float_as_uint(o[i]);
        v1[i] = __float_as_uint(o[4 + i]);
      }
      if (live_lo) __builtin_nontemporal_store(v0, reinterpret_cast<u32x4*>(q));
      if (live_hi) __builtin_nontemporal_store(v1, reinterpret_cast<u32x4*>(q + 64));
    } else {
      uint16_t* q = reinterpret_cast<uint16_t*>(a.dst_out) + u[p].elem + 4 * cc;
      const bool f16 = a.dst_dtype == DT_FP16;
      u32x2 g0, g1;
      g0.x = pack16x2(o[0], o[1], f16);
      g0.y = pack16x2(o[2], o[3], f16);
      g1.x = pack16x2(o[4], o[5], f16);
      g1.y = pack16x2(o[6], o[7], f16);
      if (live_lo) __builtin_nontemporal_store(g0, reinterpret_cast<u32x2*>(q));
      if (live_hi) __builtin_nontemporal_store(g1, reinterpret_cast<u32x2*>(q + 64));
    }
    if (a.dst_lse != nullptr) {
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (cc == r && u[p].live[r])
          a.dst_lse[lse_index(a.dst_bsh != 0, u[p].b[r], u[p].h[r], u[p].s[r], a.H, a.Sq)] =
              ua[p].den[r] > 0.f ? ua[p].m[r] + __logf(ua[p].den[r]) : -INFINITY;
    }
  }
}

struct CopyArgs {
  const void* src_out;
  const float* src_lse;
  void* dst_out;
  float* dst_lse;
  int32_t B, Sq, H;
  int32_t src_dtype, src_bsh, dst_dtype, dst_bsh;   // DT_BF16 / DT_FP32 / DT_FP16
};


constexpr int kCopyRows = 1;  // rows per lane group (2 and 4 measured: -6 % and -12 %)

// SRC / DST: the DT_* codes of the two sides, fixed at compile time (the launcher picks the instantiation).
template <int D, int SRC, int DST>
__global__ __launch_bounds__(kThreads) void state_copy_kernel(const CopyArgs a) {
  constexpr int kLanesPerRow = D / 8;
  constexpr int kRowsPerPass = kThreads / kLanesPerRow;
  constexpr int kRowsPerWg = kRowsPerPass * kCopyRows;
  int st, b, h;
  decode_wg(blockIdx.x, a.B, a.H, st, b, h);
  const int rr = threadIdx.x / kLanesPerRow;
  const int cc = threadIdx.x % kLanesPerRow;
  Row8 r[kCopyRows];
  float l[kCopyRows];
  const bool copy_lse = (cc == 0 && a.dst_lse != nullptr && a.src_lse != nullptr);
#pragma unroll
  for (int p = 0; p < kCopyRows; ++p) {
    const int s = st * kRowsPerWg + p * kRowsPerPass + rr;
    if (s < a.Sq) {
      const int64_t elem = (((int64_t)b * a.Sq + s) * a.H + h) * D;
      r[p] = load_row8<D>(a.src_out, SRC == DT_FP32, elem, cc);
      if (copy_lse) l[p] = a.src_lse[lse_index(a.src_bsh != 0, b, h, s, a.H, a.Sq)];
    }
  }
#pragma unroll
  for (int p = 0; p < kCopyRows; ++p) {
    const int s = st * kRowsPerWg + p * kRowsPerPass + rr;
    if (s < a.Sq) {
      const int64_t elem = (((int64_t)b * a.Sq + s) * a.H + h) * D;
      float x[8];
      unpack_row8(r[p], SRC, x);
      store_row8<D>(a.dst_out, DST, elem, cc, x);
      if (copy_lse) a.dst_lse[lse_index(a.dst_bsh != 0, b, h, s, a.H, a.Sq)] = l[p];
    }
  }
}

// The same copy on 256-byte units (see the merge): at D = 64 a lane group then moves two neighbouring
// rows and every load / store instruction covers whole 128-byte lines, where the row-mapped kernel above
// touches half of each line per instruction.
template <int D, int MAP, int SRC, int DST>
__global__ __launch_bounds__(kThreads) void state_copy_units_kernel(const CopyArgs a) {
  constexpr int R = 128 / D;
  const int cc = threadIdx.x % kUnitLanes;
  UnitPos<R> u[1];
  if (!unit_positions<D, MAP, 1>(a.B, a.Sq, a.H, u)) return;
  const bool live_lo = u[0].live[0], live_hi = u[0].live[R - 1];
  const bool with_lse = a.dst_lse != nullptr && a.src_lse != nullptr;
  float l = 0.f;
  bool my_lse = false;
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (with_lse && cc == r && u[0].live[r]) {
      my_lse = true;
      l = a.src_lse[lse_index(a.src_bsh != 0, u[0].b[r], u[0].h[r], u[0].s[r], a.H, a.Sq)];
    }
  float x[8];
  if (SRC == DT_FP32) {
    const float* q = reinterpret_cast<const float*>(a.src_out) + u[0].elem + 4 * cc;
    u32x4 v0 = u32x4{0u, 0u, 0u, 0u}, v1 = v0;
    if (live_lo) v0 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q));
    if (live_hi) v1 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q + 64));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[i] = __uint_as_float(v0[i]);
      x[4 + i] = __uint_as_float(v1[i]);
    }
  } else {
    const uint16_t* q = reinterpret_cast<const uint16_t*>(a.src_out) + u[0].elem + 4 * cc;
    u32x2 g0 = u32x2{0u, 0u}, g1 = g0;
    if (live_lo) g0 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q));
    if (live_hi) g1 = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(q + 64));
    const bool f16 = SRC == DT_FP16;
    widen16x2(g0.x, f16, x[0], x[1]);
    widen16x2(g0.y, f16, x[2], x[3]);
    widen16x2(g1.x, f16, x[4], x[5]);
    widen16x2(g1.y, f16, x[6], x[7]);
  }
  if (DST == DT_FP32) {
    float* q = reinterpret_cast<float*>(a.dst_out) + u[0].elem + 4 * cc;
    u32x4 v0, v1;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v0[i] = __float_as_uint(x[i]);
      v1[i] = __float_as_uint(x[4 + i]);
    }
    if (live_lo) __builtin_nontemporal_store(v0, reinterpret_cast<u32x4*>(q));
    if (live_hi) __builtin_nontemporal_store(v1, reinterpret_cast<u32x4*>(q + 64));
  } else {
    uint16_t* q = reinterpret_cast<uint16_t*>(a.dst_out) + u[0].elem + 4 * cc;
    const bool f16 = DST == DT_FP16;
    u32x2 g0, g1;
    g0.x = pack16x2(x[0], x[1], f16);
    g0.y = pack16x2(x[2], x[3], f16);
    g1.x = pack16x2(x[4], x[5], f16);
    g1.y = pack16x2(x[6], x[7], f16);
    if (live_lo) __builtin_nontemporal_store(g0, reinterpret_cast<u32x2*>(q));
    if (live_hi) __builtin_nontemporal_store(g1, reinterpret_cast<u32x2*>(q + 64));
  }
#pragma unroll
  for (int r = 0; r < R; ++r)
    if (my_lse && cc == r)
      a.dst_lse[lse_index(a.dst_bsh != 0, u[0].b[r], u[0].h[r], u[0].s[r], a.H, a.Sq)] = l;
}

// bf16 or fp16 state -> fp32 state (a cache load): `out` is an elementwise widening in the same element order,
// so it runs as a flat pass -- a lane takes 4 consecutive elements (8 bytes in, 16 bytes out), one
// load and one store, both non-temporal (+5 % over the row-mapped kernel above in this direction; in
// the narrowing direction the row-mapped kernel is the faster one by 5-13 %, so it keeps that).  The
// workgroups in front of those of `out` (dispatched first, so that they run beside the streaming ones
// instead of as a tail) move the lse: one run of `lse_run` query positions x all heads per workgroup,
// read in the source's order, written in the destination's, through the LDS in between, so that
// both sides are coalesced whichever way the [H][S] / [S][H] layouts differ.
constexpr int kConvThreads = 256;

__global__ __launch_bounds__(kConvThreads) void state_widen_kernel(const CopyArgs a, int64_t groups, uint32_t wgs_lse,
                                                                   int lse_run) {
  extern __shared__ float conv_lds[];   // [H][lse_run]
  if (blockIdx.x >= wgs_lse) {
    const int64_t g = (int64_t)(blockIdx.x - wgs_lse) * kConvThreads + threadIdx.x;   // 4 elements
    if (g >= groups) return;
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(a.src_out) + g);
    const bool f16 = a.src_dtype == DT_FP16;
    float x[4];
    widen16x2(v.x, f16, x[0], x[1]);
    widen16x2(v.y, f16, x[2], x[3]);
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) o[i] = __float_as_uint(x[i]);
    __builtin_nontemporal_store(o, reinterpret_cast<u32x4*>(a.dst_out) + g);
    return;
  }
  const int runs = (a.Sq + lse_run - 1) / lse_run;
  const int b = blockIdx.x / runs;
  const int s0 = (blockIdx.x - b * runs) * lse_run;
  const int ns = min(lse_run, a.Sq - s0);
  const int n = ns * a.H;
  // element i of the piece in a layout's own order -> (h, s)
  auto decode = [&](bool bsh, int i, int& h, int& s) {
    if (bsh) { s = i / a.H; h = i - s * a.H; }
    else { h = i / ns; s = i - h * ns; }
  };
  for (int i = threadIdx.x; i < n; i += kConvThreads) {
    int h, s;
    decode(a.src_bsh != 0, i, h, s);
    conv_lds[h * ns + s] = a.src_lse[lse_index(a.src_bsh != 0, b, h, s0 + s, a.H, a.Sq)];
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += kConvThreads) {
    int h, s;
    decode(a.dst_bsh != 0, i, h, s);
    a.dst_lse[lse_index(a.dst_bsh != 0, b, h, s0 + s, a.H, a.Sq)] = conv_lds[h * ns + s];
  }
}

// Same dtype and same lse layout on both sides: the state is two flat byte ranges (out, lse).  A
// workgroup of 512 threads moves 8 KB: one 16-byte load per lane (1 KB contiguous per wavefront), both
// the load and the store non-temporal.  Measured against 2 / 4 / 8 loads per lane in flight, 256 and
// 1024 threads and grid-stride loops: more, simpler workgroups are the fastest copy on this part.
struct FlatCopyArgs {
  const uint8_t* src[2];
  uint8_t* dst[2];
  int64_t bytes[2];   // multiples of 4
  uint32_t wgs0;      // workgroups of the first range
};
constexpr int kFlatThreads = 512;
constexpr int kFlatWgBytes = kFlatThreads * 16;

__global__ __launch_bounds__(kFlatThreads) void flat_copy_kernel(const FlatCopyArgs a) {
  const int which = blockIdx.x >= a.wgs0 ? 1 : 0;
  const int64_t wg = which ? blockIdx.x - a.wgs0 : blockIdx.x;
  const uint8_t* src = a.src[which];
  uint8_t* dst = a.dst[which];
  const int64_t bytes = a.bytes[which];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t wave_base = wg * kFlatWgBytes + wave * 1024;
  const bool vec_ok = ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0;
  if (vec_ok && wave_base + 1024 <= bytes) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src + wave_base + lane * 16));
    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst + wave_base + lane * 16));
  } else {
    // the range's last, partial 1 KB (or a range that is not 16-byte aligned): 4 bytes at a time
    for (int64_t off = wave_base + lane * 4; off < bytes && off < wave_base + 1024; off += 256)
      *reinterpret_cast<uint32_t*>(dst + off) = *reinterpret_cast<const uint32_t*>(src + off);
  }
}

// One wavefront per (t, l) row: ballot + prefix popcount compaction.
__global__ __launch_bounds__(64) void build_schedule_kernel(const uint8_t* mask, int /*T*/, int /*L*/, int C, int row0,
                                                            int diag, int32_t* compute_ids, int32_t* reuse_ids,
                                                            int32_t* counts) {
  const int row = row0 + blockIdx.x;          // t*L + l
  const int orow = blockIdx.x;                // output row (0 for the single-row entry point)
  const uint8_t* m = mask + (int64_t)row * C;
  int32_t* comp = compute_ids + (int64_t)orow * C;
  int32_t* reu = reuse_ids + (int64_t)orow * C;
  const int lane = threadIdx.x;
  const bool has_diag = (diag >= 0 && diag < C);
  int n_comp = has_diag ? 1 : 0;
  int n_reu = 0;
  if (has_diag && lane == 0) comp[0] = diag;
  for (int c0 = 0; c0 < C; c0 += 64) {
    const int c = c0 + lane;
    const bool in = c < C && c != diag;
    const bool is_comp = in && m[c] == 0;
    const bool is_reu = in && m[c] != 0;
    const unsigned long long bc = __ballot(is_comp);
    const unsigned long long br = __ballot(is_reu);
    const unsigned long long lt = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    if (is_comp) comp[n_comp + __popcll(bc & lt)] = c;
    if (is_reu) reu[n_reu + __popcll(br & lt)] = c;
    n_comp += __popcll(bc);
    n_reu += __popcll(br);
  }
  for (int i = lane; i < C; i += 64) {
    if (i >= n_comp) comp[i] = -1;
    if (i >= n_reu) reu[i] = -1;
  }
  if (lane == 0) {
    counts[2 * orow] = n_comp;
    counts[2 * orow + 1] = n_reu;
  }
}

__global__ __launch_bounds__(kThreads) void rel_l1_sums_kernel(const float* a, const float* b, int64_t n,
                                                               double* sums) {
  float d = 0.f, sa = 0.f, sb = 0.f, cnt = 0.f;
  const int64_t stride = (int64_t)gridDim.x * kThreads * 4;
  for (int64_t i = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4; i < n; i += stride) {
    float xa[4], xb[4];
    if (i + 4 <= n) {
      const f32x4 va = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(a + i));
      const f32x4 vb = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(b + i));
      xa[0] = va.x; xa[1] = va.y; xa[2] = va.z; xa[3] = va.w;
      xb[0] = vb.x; xb[1] = vb.y; xb[2] = vb.z; xb[3] = vb.w;
    } else {
      for (int k = 0; k < 4; ++k) {
        const bool ok = i + k < n;
        xa[k] = ok ? a[i + k] : NAN;
        xb[k] = ok ? b[i + k] : NAN;
      }
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const bool ok = !(xa[k] != xa[k]) && !(xb[k] != xb[k]);
      if (ok) {
        d += fabsf(xa[k] - xb[k]);
        sa += fabsf(xa[k]);
        sb += fabsf(xb[k]);
        cnt += 1.f;
      }
    }
  }
  // wavefront reduction, workgroup reduction through the LDS, then ONE set of fp64 atomics per workgroup: the
  // four sums share a cache line, and atomics on one line are serialised (one set per wavefront of 2048
  // workgroups took 0.4 ms, seven times the streaming pass itself)
  double v[4] = {(double)d, (double)sa, (double)sb, (double)cnt};
#pragma unroll
  for (int k = 0; k < 4; ++k) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v[k] += __shfl_xor(v[k], off);
  }
  __shared__ double part[kThreads / 64][4];
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int k = 0; k < 4; ++k) part[wave][k] = v[k];
  }
  __syncthreads();
  if (threadIdx.x < 4) {
    double t = 0.0;
#pragma unroll
    for (int w = 0; w < kThreads / 64; ++w) t += part[w][threadIdx.x];
    atomicAdd(&sums[threadIdx.x], t);
  }
}

// Zeroes the 16-byte units behind row *first_row of a dense [n_rows, row_bytes] tensor (the rows of a packed
// batch that belong to no segment).  A fixed, small grid walks the range; with nothing to clear -- the usual
// case -- every lane leaves after one scalar load.
__global__ __launch_bounds__(kThreads) void zero_rows_from_kernel(u32x4* dst, int64_t n_rows, int64_t units_per_row,
                                                                 const int32_t* first_row) {
  int64_t first = *first_row;
  first = first < 0 ? 0 : (first > n_rows ? n_rows : first);
  const int64_t begin = first * units_per_row, end = n_rows * units_per_row;
  for (int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x; i < end; i += (int64_t)gridDim.x * kThreads)
    dst[i] = u32x4{0u, 0u, 0u, 0u};
}

// ---- host-side launchers ---------------------------------------------------------------

// Which mapping and how many passes a launch gets (A/B on one box, states rotating through HBM; TB/s):
//   * tiled wherever the tiles fit the head count (D = 128: 3 states 6.28 against 6.10 linear, 5 states 6.41
//     against 6.24, 8 states 6.52-6.56 against 6.43);
//   * D = 128: two passes from a full batch of states on (8 states 6.46 against 6.41 with one pass, 32 states
//     of 743 MB 5.88 against 5.74), one pass below (3 states 6.28 against 5.84 with two);
//   * D = 64: one pass while the launch is small (8 states of 14 MB: 5.6 against 5.2 with two
//     passes -- finer workgroups fill the last round of the chip better), two passes on large ones.
constexpr int64_t kTwoPassUnits = 1 << 20;

template <int D, int MAP, int P>
static void launch_merge_k(const MergeArgs& a, unsigned wgs, hipStream_t stream) {
  const uint64_t all = a.n >= 64 ? ~0ull : ((1ull << a.n) - 1);
  const dim3 grid(wgs), block(kThreads);
  // fewer states than a full batch: the instantiation with the small batch (its registers are sized for 4 states in
  // flight, which lets 5 wavefronts share a SIMD instead of 3 in the two-pass form: 6 or 7 states +14 % at D = 128,
  // 4 ... 7 states +10 ... 17 % at D = 64; from 8 states on the full batch is the faster one, by 2 ... 6 %)
  const bool small = a.n < kBatch;
  if (a.fp32_mask == 0 && a.f16_mask == 0) {
    if (small) hipLaunchKernelGGL((merge_states_kernel<D, 1, MAP, P, kBatchMixed>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((merge_states_kernel<D, 1, MAP, P, kBatch>), grid, block, 0, stream, a);
  } else if (a.f16_mask == all) {
    if (small) hipLaunchKernelGGL((merge_states_kernel<D, 2, MAP, P, kBatchMixed>), grid, block, 0, stream, a);
    else hipLaunchKernelGGL((merge_states_kernel<D, 2, MAP, P, kBatch>), grid, block, 0, stream, a);
  }
  else if (a.f16_mask == 0) hipLaunchKernelGGL((merge_states_kernel<D, 3, MAP, P, kBatchMixed>), grid, block, 0, stream, a);
  else hipLaunchKernelGGL((merge_states_kernel<D, 0, MAP, P, kBatchMixed>), grid, block, 0, stream, a);
}

template <int D>
static void launch_merge_d(const MergeArgs& a, bool tiled, int passes, unsigned wgs, hipStream_t stream) {
  if (tiled) {
    if (passes == 2) launch_merge_k<D, MAP_TILED, 2>(a, wgs, stream);
    else launch_merge_k<D, MAP_TILED, 1>(a, wgs, stream);
  } else {
    if (passes == 2) launch_merge_k<D, MAP_LINEAR, 2>(a, wgs, stream);
    else launch_merge_k<D, MAP_LINEAR, 1>(a, wgs, stream);
  }
}

int launch_merge(const MergeArgs& a, int D, hipStream_t stream) {
  if (D != 128 && D != 64) {
    set_error("head dim %d not built (64 and 128 are)", D);
    return DT_ERR_UNSUPPORTED;
  }
  const int R = 128 / D;   // rows per unit
  const int64_t units = ((int64_t)a.B * a.Sq * a.H + R - 1) / R;
  const bool tiled = unit_tiles_fit(a.H, D);
  int passes;
  if (D == 64) passes = units >= kTwoPassUnits ? 2 : 1;
  else passes = a.n >= kBatch ? 2 : 1;
  const int64_t wgs = unit_grid(a.B, a.Sq, a.H, D, tiled, passes);
  if (wgs <= 0) return DT_OK;
  if (wgs > 0x7fffffffLL) {
    set_error("merge grid too large");
    return DT_ERR_INVALID;
  }
  if (D == 128) launch_merge_d<128>(a, tiled, passes, (unsigned)wgs, stream);
  else launch_merge_d<64>(a, tiled, passes, (unsigned)wgs, stream);
  return hip_fail(hipGetLastError(), "merge_states launch");
}

// Picks the instantiation of a copy kernel for the (source, destination) dtypes of `a`.
template <template <int, int> class Launch>
static void dispatch_copy_dtypes(const CopyArgs& a, unsigned wgs, hipStream_t stream) {
#define DT_COPY_CASE(S, T) \
  if (a.src_dtype == S && a.dst_dtype == T) return Launch<S, T>::run(a, wgs, stream);
  DT_COPY_CASE(DT_BF16, DT_BF16) DT_COPY_CASE(DT_BF16, DT_FP32) DT_COPY_CASE(DT_BF16, DT_FP16)
  DT_COPY_CASE(DT_FP32, DT_BF16) DT_COPY_CASE(DT_FP32, DT_FP32) DT_COPY_CASE(DT_FP32, DT_FP16)
  DT_COPY_CASE(DT_FP16, DT_BF16) DT_COPY_CASE(DT_FP16, DT_FP32) DT_COPY_CASE(DT_FP16, DT_FP16)
#undef DT_COPY_CASE
}
template <int SRC, int DST>
struct LaunchCopyUnits64 {
  static void run(const CopyArgs& a, unsigned wgs, hipStream_t stream) {
    hipLaunchKernelGGL((state_copy_units_kernel<64, MAP_TILED, SRC, DST>), dim3(wgs), dim3(kThreads), 0, stream, a);
  }
};
template <int SRC, int DST>
struct LaunchCopyRows128 {
  static void run(const CopyArgs& a, unsigned wgs, hipStream_t stream) {
    hipLaunchKernelGGL((state_copy_kernel<128, SRC, DST>), dim3(wgs), dim3(kThreads), 0, stream, a);
  }
};
template <int SRC, int DST>
struct LaunchCopyRows64 {
  static void run(const CopyArgs& a, unsigned wgs, hipStream_t stream) {
    hipLaunchKernelGGL((state_copy_kernel<64, SRC, DST>), dim3(wgs), dim3(kThreads), 0, stream, a);
  }
};

int launch_copy(const CopyArgs& a, int D, hipStream_t stream) {
  const bool with_lse = a.dst_lse != nullptr && a.src_lse != nullptr;
  if (a.src_dtype == a.dst_dtype && (!with_lse || a.src_bsh == a.dst_bsh) && (D == 64 || D == 128)) {
    const int64_t rows = (int64_t)a.B * a.Sq * a.H;
    FlatCopyArgs f{};
    f.src[0] = static_cast<const uint8_t*>(a.src_out);
    f.dst[0] = static_cast<uint8_t*>(a.dst_out);
    f.bytes[0] = rows * D * (a.src_dtype == DT_FP32 ? 4 : 2);
    f.src[1] = reinterpret_cast<const uint8_t*>(a.src_lse);
    f.dst[1] = reinterpret_cast<uint8_t*>(a.dst_lse);
    f.bytes[1] = with_lse ? rows * 4 : 0;
    const int64_t w0 = (f.bytes[0] + kFlatWgBytes - 1) / kFlatWgBytes, w1 = (f.bytes[1] + kFlatWgBytes - 1) / kFlatWgBytes;
    if (w0 + w1 > 0x7fffffffLL) {
      set_error("copy grid too large");
      return DT_ERR_INVALID;
    }
    f.wgs0 = (uint32_t)w0;
    if (w0 + w1 > 0) hipLaunchKernelGGL(flat_copy_kernel, dim3((unsigned)(w0 + w1)), dim3(kFlatThreads), 0, stream, f);
    return hip_fail(hipGetLastError(), "flat_copy launch");
  }
  if (D != 64 && D != 128) {
    set_error("head dim %d not built (64 and 128 are)", D);
    return DT_ERR_UNSUPPORTED;
  }
  if (a.src_dtype != DT_FP32 && a.dst_dtype == DT_FP32) {
    const int64_t rows = (int64_t)a.B * a.Sq * a.H;
    const int64_t groups = rows * D / 4;
    const int64_t w_out = (groups + kConvThreads - 1) / kConvThreads;
    // Query positions per lse workgroup.  Runs of 64 floats per head read whole 256-byte lines of a [H][S] source,
    // but on a small state the few workgroups that result each walk a dozen dependent rounds of loads and finish
    // long after the streaming part (2222 x 48 heads: 35 workgroups of 3072 values, 16.6 us for a 42 MB launch
    // against 10 us with runs of 16); so a workgroup takes about 1024 values, in runs of at least 16 floats.
    int lse_run = a.H <= 256 ? 64 : std::max(1, 16384 / a.H);   // at most 64 KB of LDS
    if ((int64_t)a.B * a.Sq * a.H < (1 << 18)) lse_run = std::min(lse_run, std::max(16, 1024 / a.H / 16 * 16));
    const int64_t w_lse = with_lse ? (int64_t)a.B * ((a.Sq + lse_run - 1) / lse_run) : 0;
    if (w_out + w_lse <= 0) return DT_OK;
    if (w_out + w_lse > 0x7fffffffLL || (int64_t)lse_run * a.H * 4 > 65536) {
      set_error("copy grid too large");
      return DT_ERR_INVALID;
    }
    hipLaunchKernelGGL(state_widen_kernel, dim3((unsigned)(w_out + w_lse)), dim3(kConvThreads),
                       with_lse ? (size_t)lse_run * a.H * 4 : 0, stream, a, groups, (uint32_t)w_lse, lse_run);
    return hip_fail(hipGetLastError(), "state_widen launch");
  }
  if (D == 64 && unit_tiles_fit(a.H, D)) {
    // two neighbouring rows per lane group, query x head tiles (fp32 -> slot at 714 336 rows: 5.70 against 5.44 TB/s
    // for the row mapping; at D = 128 the row mapping with its contiguous lse runs is the faster one, 6.3 against 6.0)
    const int64_t wgs = unit_grid(a.B, a.Sq, a.H, D, true, 1);
    if (wgs <= 0) return DT_OK;
    if (wgs > 0x7fffffffLL) {
      set_error("copy grid too large");
      return DT_ERR_INVALID;
    }
    dispatch_copy_dtypes<LaunchCopyUnits64>(a, (unsigned)wgs, stream);
    return hip_fail(hipGetLastError(), "state_copy_units launch");
  }
  const int rows_per_wg = kThreads / (D / 8) * kCopyRows;
  const int n_st = (a.Sq + rows_per_wg - 1) / rows_per_wg;
  const int64_t wgs = (int64_t)a.B * a.H * n_st;
  if (wgs <= 0) return DT_OK;
  if (wgs > 0x7fffffffLL) {
    set_error("copy grid too large");
    return DT_ERR_INVALID;
  }
  if (D == 128) dispatch_copy_dtypes<LaunchCopyRows128>(a, (unsigned)wgs, stream);
  else dispatch_copy_dtypes<LaunchCopyRows64>(a, (unsigned)wgs, stream);
  return hip_fail(hipGetLastError(), "state_copy launch");
}

}  // namespace dt

using namespace dt;

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
static bool known_dtype(int32_t d) { return d == DT_BF16 || d == DT_FP32 || d == DT_FP16; }

static int check_dims(int32_t B, int32_t Sq, int32_t H, int32_t D) {
  if (B <= 0 || Sq <= 0 || H <= 0) {
    set_error("B, Sq, H must be positive (got %d, %d, %d)", B, Sq, H);
    return DT_ERR_INVALID;
  }
  if (D != 64 && D != 128) {
    set_error("head dim %d not built (64 and 128 are)", D);
    return DT_ERR_UNSUPPORTED;
  }
  return DT_OK;
}

extern "C" int dt_merge_states(int32_t n, const void* const* outs, const float* const* lses,
                               const int32_t* src_dtype, const int32_t* src_lse_layout, void* dst_out,
                               int32_t dst_dtype, float* dst_lse, int32_t dst_lse_layout, int32_t B, int32_t Sq,
                               int32_t H, int32_t D, void* stream) {
  if (int rc = check_dims(B, Sq, H, D)) return rc;
  if (n <= 0 || n > DT_MAX_MERGE) {
    set_error("merge of %d states: need 1..%d", n, DT_MAX_MERGE);
    return DT_ERR_INVALID;
  }
  if (!outs || !lses || !dst_out) {
    set_error("null pointer argument");
    return DT_ERR_INVALID;
  }
  MergeArgs a{};
  a.n = n;
  a.B = B; a.Sq = Sq; a.H = H;
  for (int i = 0; i < n; ++i) {
    if (!outs[i] || !lses[i] || !aligned16(outs[i])) {
      set_error("state %d: null or misaligned pointer", i);
      return DT_ERR_INVALID;
    }
    a.out[i] = outs[i];
    a.lse[i] = lses[i];
    const int dtp = src_dtype ? src_dtype[i] : DT_BF16;
    const int lay = src_lse_layout ? src_lse_layout[i] : DT_LSE_BHS;
    if (!known_dtype(dtp) || (lay != DT_LSE_BHS && lay != DT_LSE_BSH)) {
      set_error("state %d: bad dtype/layout code", i);
      return DT_ERR_INVALID;
    }
    if (dtp == DT_FP32) a.fp32_mask |= (1ull << i);
    if (dtp == DT_FP16) a.f16_mask |= (1ull << i);
    if (lay == DT_LSE_BSH) a.bsh_mask |= (1ull << i);
  }
  if (!aligned16(dst_out) || !known_dtype(dst_dtype) || (dst_lse_layout != DT_LSE_BHS && dst_lse_layout != DT_LSE_BSH)) {
    set_error("bad destination pointer/dtype/layout");
    return DT_ERR_INVALID;
  }
  a.dst_out = dst_out;
  a.dst_lse = dst_lse;
  a.dst_dtype = dst_dtype;
  a.dst_bsh = dst_lse_layout == DT_LSE_BSH;
  return launch_merge(a, D, (hipStream_t)stream);
}

static int state_copy(const void* src_out, int32_t src_dtype, const float* src_lse, int32_t src_layout, void* dst_out,
                      int32_t dst_dtype, float* dst_lse, int32_t dst_layout, int32_t B, int32_t Sq, int32_t H,
                      int32_t D, void* stream) {
  if (int rc = check_dims(B, Sq, H, D)) return rc;
  if (!src_out || !dst_out || !aligned16(src_out) || !aligned16(dst_out)) {
    set_error("null or misaligned state pointer");
    return DT_ERR_INVALID;
  }
  if (!known_dtype(src_dtype) || !known_dtype(dst_dtype) ||
      (src_layout != DT_LSE_BHS && src_layout != DT_LSE_BSH) || (dst_layout != DT_LSE_BHS && dst_layout != DT_LSE_BSH)) {
    set_error("bad dtype/layout code");
    return DT_ERR_INVALID;
  }
  CopyArgs a{};
  a.src_out = src_out; a.src_lse = src_lse; a.dst_out = dst_out; a.dst_lse = dst_lse;
  a.B = B; a.Sq = Sq; a.H = H;
  a.src_dtype = src_dtype; a.src_bsh = src_layout == DT_LSE_BSH;
  a.dst_dtype = dst_dtype; a.dst_bsh = dst_layout == DT_LSE_BSH;
  return launch_copy(a, D, (hipStream_t)stream);
}

extern "C" int dt_cache_store(const void* src_out, int32_t src_dtype, const float* src_lse, int32_t src_lse_layout,
                              void* slot_out, float* slot_lse, int32_t B, int32_t Sq, int32_t H, int32_t D,
                              void* stream) {
  return state_copy(src_out, src_dtype, src_lse, src_lse_layout, slot_out, DT_BF16, slot_lse, DT_LSE_BHS, B, Sq, H, D,
                    stream);
}

extern "C" int dt_cache_load(const void* slot_out, const float* slot_lse, void* dst_out, int32_t dst_dtype,
                             float* dst_lse, int32_t dst_lse_layout, int32_t B, int32_t Sq, int32_t H, int32_t D,
                             void* stream) {
  return state_copy(slot_out, DT_BF16, slot_lse, DT_LSE_BHS, dst_out, dst_dtype, dst_lse, dst_lse_layout, B, Sq, H, D,
                    stream);
}

extern "C" int dt_state_copy(const void* src_out, int32_t src_dtype, const float* src_lse, int32_t src_lse_layout,
                             void* dst_out, int32_t dst_dtype, float* dst_lse, int32_t dst_lse_layout, int32_t B,
                             int32_t Sq, int32_t H, int32_t D, void* stream) {
  return state_copy(src_out, src_dtype, src_lse, src_lse_layout, dst_out, dst_dtype, dst_lse, dst_lse_layout, B, Sq, H, D,
                    stream);
}

static int check_sched(const uint8_t* mask, int32_t T, int32_t L, int32_t C, const void* a, const void* b,
                       const void* c) {
  if (!mask || !a || !b || !c) {
    set_error("null pointer argument");
    return DT_ERR_INVALID;
  }
  if (T <= 0 || L <= 0 || C <= 0 || C > 1024) {
    set_error("schedule dims T=%d L=%d C=%d out of range (C <= 1024)", T, L, C);
    return DT_ERR_INVALID;
  }
  return DT_OK;
}

extern "C" int dt_build_schedule(const uint8_t* mask, int32_t T, int32_t L, int32_t C, int32_t t, int32_t l,
                                 int32_t diag, int32_t* compute_ids, int32_t* reuse_ids, int32_t* counts,
                                 void* stream) {
  if (int rc = check_sched(mask, T, L, C, compute_ids, reuse_ids, counts)) return rc;
  if (t < 0 || t >= T || l < 0 || l >= L) {
    set_error("(t,l)=(%d,%d) outside [0,%d)x[0,%d)", t, l, T, L);
    return DT_ERR_INVALID;
  }
  hipLaunchKernelGGL(build_schedule_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, mask, T, L, C, t * L + l, diag,
                     compute_ids, reuse_ids, counts);
  return hip_fail(hipGetLastError(), "build_schedule launch");
}

extern "C" int dt_build_schedule_table(const uint8_t* mask, int32_t T, int32_t L, int32_t C, int32_t diag,
                                       int32_t* compute_ids, int32_t* reuse_ids, int32_t* counts, void* stream) {
  if (int rc = check_sched(mask, T, L, C, compute_ids, reuse_ids, counts)) return rc;
  hipLaunchKernelGGL(build_schedule_kernel, dim3((unsigned)(T * L)), dim3(64), 0, (hipStream_t)stream, mask, T, L, C,
                     0, diag, compute_ids, reuse_ids, counts);
  return hip_fail(hipGetLastError(), "build_schedule_table launch");
}

extern "C" int dt_zero_rows_from(void* dst, int64_t n_rows, int64_t row_bytes, const int32_t* first_row, void* stream) {
  if (!dst || !first_row || !aligned16(dst) || n_rows < 0 || row_bytes <= 0 || (row_bytes % 16)) {
    set_error("zero_rows_from: need a 16-byte aligned tensor, rows of a positive multiple of 16 bytes and a device row index");
    return DT_ERR_INVALID;
  }
  if (n_rows == 0) return DT_OK;
  hipLaunchKernelGGL(zero_rows_from_kernel, dim3(512), dim3(kThreads), 0, (hipStream_t)stream, static_cast<u32x4*>(dst),
                     n_rows, row_bytes / 16, first_row);
  return hip_fail(hipGetLastError(), "zero_rows_from launch");
}

extern "C" int dt_rel_l1_sums(const float* a, const float* b, int64_t n, double* sums, void* stream) {
  if (!a || !b || !sums || n < 0) {
    set_error("null pointer or negative length");
    return DT_ERR_INVALID;
  }
  if (!aligned16(a) || !aligned16(b)) {
    set_error("inputs must be 16-byte aligned");
    return DT_ERR_INVALID;
  }
  if (n == 0) return DT_OK;
  int64_t wgs = (n / 4 + kThreads - 1) / kThreads;
  if (wgs > 1024) wgs = 1024;   // 4 per CU: enough loads in flight, few atomics
  if (wgs < 1) wgs = 1;
  hipLaunchKernelGGL(rel_l1_sums_kernel, dim3((unsigned)wgs), dim3(kThreads), 0, (hipStream_t)stream, a, b, n, sums);
  return hip_fail(hipGetLastError(), "rel_l1_sums launch");
}
