// Chunk attention forward for gfx950 (MI355X): out = softmax(q k^T * scale) v and
// the natural-log lse of one query shard against one or several KV chunks.
//
// Stands in for flash_attn_func as called at core/attention.py:137-143,185-191
// of the reference.
//
// Shape of the computation
//   * One workgroup = 8 wavefronts = 256 queries of one (batch, head); each
//     wavefront owns 32 queries.  D = 128: one workgroup per CU, two wavefronts per
//     SIMD (256 VGPRs each); D = 64: two workgroups per CU (128 VGPRs each).
//   * The 8 wavefronts form two groups of 4 that run the same loop ONE PHASE
//     APART ("ping-pong"): while group A issues the MFMAs of a tile
//     (O^T += V^T P^T of the previous tile, then S^T = K Q^T of this one), group B
//     runs the VALU half (online softmax of its tile, issuing the loads of a later
//     K/V tile), and vice versa; a workgroup barrier separates the
//     phases.  Each SIMD holds one wavefront of either group, so its matrix pipe
//     and its vector ALU are busy at the same time instead of taking turns.
//   * KV is consumed in tiles of 64 keys, staged in LDS as they come, [key][d],
//     four buffers per operand.  A tile goes from global memory STRAIGHT into
//     LDS (buffer loads with the LDS as destination: no registers, no LDS write
//     instructions, no wait for them in the softmax), issued three (K) and two
//     (V) tiles ahead of their first use.  Staging through registers cost a
//     fifth of the loop's cycles: the fill's LDS writes queue up in front of the
//     operand reads of the wavefronts that are issuing MFMAs.  Such a load writes
//     1 KB of consecutive LDS bytes, so rows are not padded but XOR-swizzled (the
//     lane picks which 16 bytes of global memory it fetches); operand reads stay
//     bank-conflict free and use immediate offsets from a few per-lane address
//     registers.  The second MFMA needs V^T; the transposition is done by the
//     LDS read itself (ds_read_b64_tr_b16).  The buffer descriptor lives in
//     scalar registers, and rows past the end of a chunk arrive as zeros.
//   * Scores are computed TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16:
//     in the accumulator layout a lane then owns ONE query (column lane%32) and
//     16 of the 32 keys of the tile, so the online-softmax max/sum are
//     in-register reductions plus a single exchange with lane^32.
//   * The rows of the K operand are permuted (bits 2 and 3 of the row index
//     swapped) so that the 8 accumulator registers a lane holds for a half tile
//     are 8 CONSECUTIVE keys.  Rounded to bf16 they are directly the B operand
//     of the second MFMA, O^T += V^T P^T, whose A operand (8 consecutive keys of
//     one d column) is two transposing reads of 4 keys each.
//   * O^T stays in registers as [d][query]: a rescale is a multiply by a per-lane
//     scalar.  The reference maximum the accumulators are scaled to may lag behind
//     the true row maximum (the lse stays exact): the common path computes no row
//     maximum at all, the fp32 row sum it needs anyway is the overflow detector,
//     and only a tile whose sum exceeds 2^12 is redone with its exact maximum.  The epilogue
//     transposes through LDS so that the global stores are 16 bytes per lane.
//   * Workgroups are mapped to (head, query tile) so that the 8 XCDs each work
//     through a contiguous range of heads: the workgroups that share an XCD's
//     L2 stream the same K/V.
#include <algorithm>
#include <mutex>
#include <type_traits>

#include "attn_schedule.h"
#include "dt_common.h"

namespace dt {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// The 16-bit element type of q, K, V, P and the output states: bfloat16, or IEEE half (kHalf).  Loads, LDS
// layout, swizzles and the transposing reads only see 16-bit elements; the type decides the MFMA and the
// roundings of P and of the output.
template <bool kHalf>
struct Elem {
  typedef __bf16 t;
  typedef __bf16 x8 __attribute__((ext_vector_type(8)));
  typedef __bf16 x4 __attribute__((ext_vector_type(4)));
  typedef __bf16 x2 __attribute__((ext_vector_type(2)));
  __device__ static __forceinline__ f32x16 mfma(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  // two packed elements of a 32-bit word, widened
  __device__ static __forceinline__ f32x2 widen(uint32_t w) {
    f32x2 f;
    f.x = __builtin_bit_cast(float, w << 16);
    f.y = __builtin_bit_cast(float, w & 0xffff0000u);
    return f;
  }
};
template <>
struct Elem<true> {
  typedef _Float16 t;
  typedef _Float16 x8 __attribute__((ext_vector_type(8)));
  typedef _Float16 x4 __attribute__((ext_vector_type(4)));
  typedef _Float16 x2 __attribute__((ext_vector_type(2)));
  __device__ static __forceinline__ f32x16 mfma(x8 a, x8 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  __device__ static __forceinline__ f32x2 widen(uint32_t w) {
    return __builtin_convertvector(__builtin_bit_cast(x2, w), f32x2);
  }
};

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * 64;
constexpr int kBQ = kWaves * 32;  // queries per workgroup
constexpr int kBK = 64;           // keys per tile
constexpr int kXcds = 8;
constexpr int kNumBuf = DT_SCHED_NUM_BUF;  // LDS buffers per operand; a tile uses buffer (tile & 3)
static_assert(kNumBuf == 4, "buffer indices are computed with & 3 and the loop is unrolled by four");
constexpr int kRingDepth = 4;     // operand fragments the LDS reads of a matrix phase run ahead of its MFMAs (2 and 6 measured: no gain)
// Row permutation of the K operand: MFMA row i -> key (within a 32-key half tile).
__device__ __forceinline__ int key_of_row(int i) {
  return (i & 19) | ((i & 4) << 1) | ((i & 8) >> 1);
}

// Raw buffer descriptor word 3 for gfx9-family targets (32-bit data format, no swizzle).
constexpr int kRsrcFlags = 0x00020000;

// Workgroup barrier between the phases.  Waits for this wavefront's LDS traffic only:
// global loads issued for a later tile stay in flight across it.
__device__ __forceinline__ void phase_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
  __builtin_amdgcn_sched_barrier(0);
}
// Waits until at most N of this wavefront's tile loads are still in flight.  N comes from attn_schedule.h.
template <int N>
__device__ __forceinline__ void wait_tile_loads() {
#define DT_WAIT_VMCNT(K) asm volatile("s_waitcnt vmcnt(" #K ")" ::: "memory")
  if constexpr (N == 0) DT_WAIT_VMCNT(0);
  else if constexpr (N == 3) DT_WAIT_VMCNT(3);
  else if constexpr (N == 4) DT_WAIT_VMCNT(4);
  else if constexpr (N == 5) DT_WAIT_VMCNT(5);
  else if constexpr (N == 6) DT_WAIT_VMCNT(6);
  else if constexpr (N == 8) DT_WAIT_VMCNT(8);
  else {
    static_assert(N == 10, "add the immediate for this wait count");
    DT_WAIT_VMCNT(10);
  }
#undef DT_WAIT_VMCNT
}
// The same barrier with the results of the finished phase routed through it as in/out
// operands.  Register-only code may otherwise migrate across an asm statement; tied to it,
// the phase's work stays on its own side (the vector phase produces P^T, the matrix phase
// produces S^T and updates O^T).
// After a vector phase the wavefront also waits for the direct-to-LDS tile loads it issued earlier,
// all but the kInFlight newest: behind the barrier they are visible to every wavefront.
template <int kInFlight, typename V>
__device__ __forceinline__ void phase_barrier_after_vector(V (&p)[2][2]) {
  __builtin_amdgcn_sched_barrier(0);
#define DT_VECTOR_BARRIER(N)                                                      \
  asm volatile("s_waitcnt vmcnt(" #N ") lgkmcnt(0)\n\ts_barrier"                   \
               : "+v"(p[0][0]), "+v"(p[0][1]), "+v"(p[1][0]), "+v"(p[1][1])       \
               :                                                                  \
               : "memory")
  if constexpr (kInFlight == 6) DT_VECTOR_BARRIER(6);
  else if constexpr (kInFlight == 3) DT_VECTOR_BARRIER(3);
  else if constexpr (kInFlight == 2) DT_VECTOR_BARRIER(2);
  else {
    static_assert(kInFlight == 1, "loads in flight across the barrier: 1, 2, 3 or 6");
    DT_VECTOR_BARRIER(1);
  }
#undef DT_VECTOR_BARRIER
  __builtin_amdgcn_sched_barrier(0);
}
template <typename V, int NO>
__device__ __forceinline__ void phase_barrier_after_matrix(V (&sa)[2], V (&oa)[NO]) {
  __builtin_amdgcn_sched_barrier(0);
  if constexpr (NO == 4) {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier"
                 : "+v"(sa[0]), "+v"(sa[1]), "+v"(oa[0]), "+v"(oa[1]), "+v"(oa[2]), "+v"(oa[3])
                 :
                 : "memory");
  } else {
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier"
                 : "+v"(sa[0]), "+v"(sa[1]), "+v"(oa[0]), "+v"(oa[1])
                 :
                 : "memory");
  }
  __builtin_amdgcn_sched_barrier(0);
}

// A tile's per-lane sum of probabilities (32 of them) above which the tile is redone with an
// exact row maximum.  Below it every probability is at most 2^12: harmless for the bf16
// operand (same relative precision at any exponent), inside the range of the fp16 operand (largest
// finite value 65504; the reference never exceeds the row's true maximum, so a probability is at least its
// true softmax weight and loses no more to fp16's small end than under an exact maximum) and for the fp32
// accumulators.
constexpr float kSumLimit = 4096.0f;
// The same for queries that come with softmax_scale * log2(e) folded in (kPre): rows keep the
// reference 0 while the maximum of their first tile lies in [kBandLo, kBandHi] (powers of two;
// 2^-40 .. 2^24 neither underflows nor overflows anything downstream), so a probability is then
// simply exp2(score), and a tile is redone when its sum exceeds 2^40.
constexpr float kSumLimitPre = 1099511627776.0f;
constexpr float kBandLo = -40.f, kBandHi = 24.f;

template <int D>
struct Tile {
  // Both tiles sit in LDS as [key][d] rows WITHOUT padding: a tile arrives through direct-to-LDS
  // buffer loads, and one such instruction writes 1 KB of consecutive LDS bytes (lane L -> bytes
  // 16 L .. 16 L + 15), so rows cannot be padded.  Bank conflicts are avoided by swizzling instead:
  // which 16 bytes of global memory a lane fetches is free, so a row's 16-byte chunks (K) or
  // 64-byte segments (V) are stored XOR-permuted by a function of the row.
  //   K: chunk c of row r sits at chunk position c ^ swz_k(r); the 16 lanes of a ds_read_b128 pass
  //      read 16 rows at the same c and land in 16 distinct 16-byte bank groups.
  //   V: segment g of row r sits at segment position g ^ swz_v(r); a transposing 8-byte read pass
  //      touches 4 rows x one 64-byte segment, which land in the four quarters of the banks.
  // swz_v only depends on row bits that the immediate row steps of the operand reads (multiples
  // of 4 rows) leave alone; the per-lane part of the swizzle is folded into a few precomputed
  // address registers (one per k-step for K, one per 32 columns for V).
  static constexpr int kRowBytes = D * 2;
  static constexpr int kChunks = D / 8;               // 16-byte chunks per row
  static constexpr int kSegs = D / 32;                // 64-byte segments per row
  static constexpr int kBytesK = kBK * kRowBytes;
  static constexpr int kBytesV = kBK * kRowBytes;
  static constexpr int kOffV = kNumBuf * kBytesK;     // V buffers follow the K buffers
  static constexpr int kBlocks = kBytesK / 1024;      // direct-load instructions per tile and operand
  static constexpr int kLoads = kBlocks / kWaves;     // ... per wavefront (2 or 1)
  static constexpr int kRowsPerBlock = 1024 / kRowBytes;
  static constexpr int kPitchO = D * 2 + 16;          // epilogue row pitch
  static constexpr int kLdsTiles = kNumBuf * (kBytesK + kBytesV);
  static constexpr int kLdsEpilogue = kWaves * 32 * kPitchO;
  static constexpr int kLdsBytes = kLdsTiles > kLdsEpilogue ? kLdsTiles : kLdsEpilogue;
  static_assert(D == 128 || D == 64, "swizzles are written for these two head dimensions");
  __device__ static constexpr int swz_k(int row) { return D == 128 ? (row & 15) : ((row >> 1) & 7); }
  __device__ static constexpr int swz_v(int row) { return D == 128 ? (row & 3) : ((row >> 1) & 1); }
};

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
// Transposing LDS read (ds_read_b64_tr_b16).  Within each block of 16 lanes the 16 x 4 matrix of
// 16-bit elements [source lane][element] is read as 4 rows of 16 (source lane 4j+m supplies
// row j, columns 4m..4m+3) and lane i receives column i: element j = row j, column i.
__device__ __forceinline__ s16x4 lds_read_tr(const uint8_t* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16(
      (s16x4 __attribute__((address_space(3)))*)(p));
}

// Raw buffer descriptor: base address, stride 0, number of valid bytes, flags.
__device__ __forceinline__ u32x4 make_rsrc(const void* base, uint32_t valid_bytes) {
  const uint64_t p = reinterpret_cast<uint64_t>(base);
  u32x4 r;   // uniform by construction; say so, the descriptor then lives in scalar registers
  r.x = __builtin_amdgcn_readfirstlane((uint32_t)p);
  r.y = __builtin_amdgcn_readfirstlane((uint32_t)(p >> 32) & 0xffffu);
  r.z = __builtin_amdgcn_readfirstlane(valid_bytes);
  r.w = (uint32_t)kRsrcFlags;
  return r;
}
// One 16-byte-per-lane buffer load whose destination is the LDS: lane L's bytes land at
// lds_addr + 16 L (lds_addr, through M0, is uniform).  Written as inline assembly on purpose: the
// compiler, when it sees such a load, makes every later LDS read of the wavefront wait for ALL
// outstanding loads (it cannot tell that the reads touch other buffers), which turns a prefetch
// several phases deep into one that must land within the phase.  Here the waits are the explicit
// vmcnt in front of the barriers.  (Loads the compiler does not know of only make its own vmcnt
// waits for other loads stricter, never too weak: the counter retires in order.)
__device__ __forceinline__ void load_block_to_lds(u32x4 rsrc, uint32_t lane_off, uint32_t uniform_off, uint32_t lds_addr) {
  // (the uniform operands are uniform by construction; say so, or a value the compiler happens to
  // hold in a vector register ends up in the instruction as one)
  u32x4 r;
  r.x = __builtin_amdgcn_readfirstlane(rsrc.x);
  r.y = __builtin_amdgcn_readfirstlane(rsrc.y);
  r.z = __builtin_amdgcn_readfirstlane(rsrc.z);
  r.w = __builtin_amdgcn_readfirstlane(rsrc.w);
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds"
               :
               : "v"(lane_off), "s"(r), "s"(__builtin_amdgcn_readfirstlane(uniform_off)),
                 "s"(__builtin_amdgcn_readfirstlane(lds_addr))
               : "memory", "m0");
}
// The wavefront's next 1 KB block of the same tile: same M0, the instruction's immediate offset moves both the LDS
// address and the global address on by 1 KB (lane_off is reduced by as much where the global side should not move).
// Rewriting M0 between two such loads costs about 17 cycles each time: the write waits until the load before it
// has read the register.
__device__ __forceinline__ void load_next_block_to_lds(u32x4 rsrc, uint32_t lane_off, uint32_t uniform_off) {
  u32x4 r;
  r.x = __builtin_amdgcn_readfirstlane(rsrc.x);
  r.y = __builtin_amdgcn_readfirstlane(rsrc.y);
  r.z = __builtin_amdgcn_readfirstlane(rsrc.z);
  r.w = __builtin_amdgcn_readfirstlane(rsrc.w);
  asm volatile("buffer_load_dwordx4 %0, %1, %2 offen offset:1024 lds"
               :
               : "v"(lane_off), "s"(r), "s"(__builtin_amdgcn_readfirstlane(uniform_off))
               : "memory");
}

// Wavefronts per SIMD the register budget is set for.  D = 128: two (one workgroup per CU: its LDS
// tiles fill the CU).  D = 64: four, i.e. TWO workgroups per CU (64 KB of LDS and at most 128
// registers each): the second workgroup's wavefronts issue into the barrier waits, the start-up and
// the epilogue of the first, which at 35 key tiles per work item are a tenth of its time (+10 %).
constexpr int kWavesPerSimdD64 = 4;
template <int D, bool kPre, bool kHalf>
__global__ __launch_bounds__(kThreads, D == 64 ? kWavesPerSimdD64 : 2) void attn_fwd_kernel(const AttnArgs args_by_value) {
  using T = Tile<D>;
  using E = Elem<kHalf>;
  typedef typename E::t elem_t;
  typedef typename E::x8 ex8;
  typedef typename E::x4 ex4;
  typedef typename E::x2 ex2;
  static_assert(!(kPre && kHalf), "the prescaled softmax keeps probabilities up to 2^40: bf16 only");
  // The arguments are read where they arrive: in the kernarg segment (constant address space, scalar loads),
  // through its base pointer -- AttnArgs is the kernel's only parameter, so it sits at offset 0.  Going through the
  // by-value parameter instead leaves it to the optimiser to prove that its private copy of the 3.6 KB struct is
  // never needed; with the tables indexed at run time from several branches it sometimes cannot, and every lane
  // then copies the whole struct into scratch memory before it starts (seven times the run time of a short launch).
  typedef const AttnArgs __attribute__((address_space(4))) KernArgs;
  KernArgs& a = *(KernArgs*)__builtin_amdgcn_kernarg_segment_ptr();
  (void)args_by_value;
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];

  // ---- which (job, batch, head, query tile) ------------------------------------------
  int job = blockIdx.y;
  const int xcd = blockIdx.x & (kXcds - 1);
  int idx = blockIdx.x >> 3;
  int part = 0;          // which of the part_ways key-tile ranges of a tail item
  bool is_part = false;  // this workgroup computes one part of a tail item
  if (job >= a.n_jobs) {
    // planes behind the jobs hold the parts of the tail items, in dispatch order
    const int pi = (job - a.n_jobs) * (int)(gridDim.x >> 3) + idx;
    if (pi >= a.tail_items * a.part_ways) return;
    job = a.tail_job;
    const int u = pi / a.part_ways;
    part = pi - u * a.part_ways;
    idx = a.tail_idx0 + u;
    is_part = true;
  } else if (job == a.tail_job && idx >= a.tail_idx0) {
    return;  // runs as parts
  }
  const int item = xcd * a.per_xcd + idx;
  if (idx >= a.per_xcd || item >= a.total) return;
  const int bh = item / a.nqt;
  const int qt = item - bh * a.nqt;
  const int b = bh / a.H;
  const int h = bh - b * a.H;

  int seg_begin, seg_end, single = -1;
  int q_begin = 0, q_end = a.Sq;   // query rows of this job
  uint16_t* out_ptr;
  float* lse_ptr;
  int vseg = -1;  // segment of a packed variable-length batch (device-listed jobs only)
  int dseg = -1;  // segment whose boundaries are read from device memory (a.cu_q != nullptr)
  if (a.dev_ids != nullptr) {
    int slot = job;
    if (a.n_seg > 0) {
      slot = job / a.n_seg;
      vseg = job - slot * a.n_seg;
    }
    if (slot >= *a.dev_count) return;
    single = __builtin_amdgcn_readfirstlane(a.dev_ids[slot]);  // uniform by construction; tell the compiler
    if (single < 0 || single >= a.n_chunks) return;  // never index the tables with a bad id
    seg_begin = 0;
    seg_end = 1;
    if (single == a.diag) {
      out_ptr = a.diag_out;
      lse_ptr = a.diag_lse;
    } else {
      out_ptr = a.slot_out + (int64_t)single * a.slot_out_stride;
      lse_ptr = a.slot_lse + (int64_t)single * a.slot_lse_stride;
    }
    if (vseg >= 0) {
      if (a.cu_q != nullptr) {
        dseg = vseg;
      } else {
        q_begin = a.seg_q_begin[vseg];
        q_end = q_begin + a.seg_q_len[vseg];
      }
    }
  } else {
    seg_begin = a.job_begin[job];
    seg_end = a.job_begin[job + 1];
    out_ptr = a.job_out[job];
    lse_ptr = a.job_lse[job];
    if (a.cu_q != nullptr) {
      dseg = a.job_q_begin[job];
    } else {
      q_begin = a.job_q_begin[job];
      q_end = q_begin + a.job_q_len[job];
    }
  }
  // Segment boundaries are read through the constant address space, i.e. with scalar loads: the lists were
  // written before the launch and the address is uniform.  (As a vector load the compiler follows it with
  // vmcnt(0), which inside the loop would also wait for every tile load in flight.)
  typedef const int32_t __attribute__((address_space(4))) ConstI32;
  auto boundary = [](const int32_t* list, int i) __attribute__((always_inline)) -> int { return ((ConstI32*)list)[i]; };
  if (dseg >= 0) {
    // boundaries from device memory: nothing on the host has looked at them, so they are clamped
    // to the rows that exist (a malformed list then yields wrong rows, never a stray access)
    q_begin = min(max(boundary(a.cu_q, dseg), 0), a.Sq);
    q_end = min(max(boundary(a.cu_q, dseg + 1), q_begin), a.Sq);
  }
  if (qt * kBQ >= q_end - q_begin) return;  // the grid is sized for the longest job / segment
  auto chunk_of = [&](int seg) __attribute__((always_inline)) -> int { return single >= 0 ? single : a.job_chunks[seg]; };
  // keys [begin, begin + len) of chunk reference `seg`
  auto kv_begin_of = [&](int seg) __attribute__((always_inline)) -> int {
    if (dseg >= 0) {
      const int cid = chunk_of(seg);
      return min(max(boundary(a.cu_kv[cid], dseg), 0), a.kv_len[cid]);
    }
    if (single < 0) return a.entry_kv_begin[seg];
    return vseg >= 0 ? a.entry_kv_begin[single * a.n_seg + vseg] : 0;
  };
  auto kv_len_of = [&](int seg) __attribute__((always_inline)) -> int {
    if (dseg >= 0) {
      const int cid = chunk_of(seg);
      const int lo = min(max(boundary(a.cu_kv[cid], dseg), 0), a.kv_len[cid]);
      const int hi = min(max(boundary(a.cu_kv[cid], dseg + 1), lo), a.kv_len[cid]);
      return hi - lo;
    }
    if (single < 0) return a.entry_kv_len[seg];
    return vseg >= 0 ? a.entry_kv_len[single * a.n_seg + vseg] : a.kv_len[single];
  };

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: keeps group/buffer arithmetic scalar
  const int group = wave >> 2;  // 0: leads, 1: runs one phase behind
  const int col = lane & 31;    // query column (B operand) / operand row (A operand)
  const int hh = lane >> 5;     // which half of the contraction dimension this lane feeds
  const int q0 = q_begin + qt * kBQ + wave * 32;

  // ---- Q fragments: B operand of S^T = K Q^T, kept in registers ----------------------
  ex8 qf[D / 16];
  {
    int qrow = q0 + col;
    if (qrow > q_end - 1) qrow = q_end - 1;
    const uint16_t* qp = a.q + (int64_t)b * a.q_sb + (int64_t)qrow * a.q_ss + (int64_t)h * a.q_sh + 8 * hh;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) qf[s] = *reinterpret_cast<const ex8*>(qp + 16 * s);
  }
  // Route the fragments through an empty asm: they are then defined by it, not by loads.  The
  // compiler otherwise keeps "Q may still be in flight" alive round the loop and waits for ALL
  // outstanding vector-memory loads (including the K/V prefetch just issued) before the first
  // MFMA that reads Q in every iteration.
#pragma unroll
  for (int s = 0; s < D / 16; ++s) asm volatile("" : "+v"(qf[s]));

  // ---- tile bookkeeping -----------------------------------------------------------------
  int n_tiles = 0;
  for (int s = seg_begin; s < seg_end; ++s) n_tiles += (kv_len_of(s) + kBK - 1) / kBK;

  // Two cursors walk the job's chunks tile by tile, all in scalar registers: the load cursor
  // (ahead of the compute cursor: base pointers of the tile and keys left in its chunk) and
  // the compute cursor (keys left in the chunk of the tile whose scores are being computed).
  int ld_seg = seg_begin - 1, ld_left = 0;
  int cp_seg = seg_begin - 1, cp_left = 0;
  // The load cursor addresses a tile as (buffer descriptor of its chunk, byte offset of its first key from the
  // chunk's first key).  The descriptors (base of the chunk's keys for this batch and head, number of valid
  // bytes) only change with the chunk; per tile the cursor moves one scalar offset.  A chunk's (batch, head)
  // plane is below 2 GiB (checked on the host), so offsets fit 32 bits with room for the lane's part.
  const uint32_t row_bytes = (uint32_t)a.kv_ss * 2u;
  const uint32_t tile_bytes = (uint32_t)kBK * row_bytes;
  u32x4 rk = make_rsrc(nullptr, 0u), rv = rk;   // K and V of the chunk under the load cursor
  uint32_t k_off = 0u;
  auto ld_next_chunk = [&]() __attribute__((always_inline)) {
    do { ++ld_seg; } while (ld_seg < seg_end && kv_len_of(ld_seg) == 0);
    k_off = 0u;
    if (ld_seg < seg_end) {
      const int cid = chunk_of(ld_seg);
      const int64_t head_off =
          (int64_t)b * a.kv_sb[cid] + (int64_t)h * a.kv_sh + (int64_t)kv_begin_of(ld_seg) * a.kv_ss;
      ld_left = kv_len_of(ld_seg);
      const uint32_t valid = (uint32_t)(ld_left - 1) * row_bytes + (uint32_t)(D * 2);
      rk = make_rsrc(a.k[cid] + head_off, valid);
      rv = make_rsrc(a.v[cid] + head_off, valid);
    } else {
      // past the last chunk: an empty descriptor, loads store zeros without touching memory
      rk = make_rsrc(nullptr, 0u);
      rv = rk;
    }
  };
  auto cp_next_chunk = [&]() __attribute__((always_inline)) {
    do { ++cp_seg; } while (cp_seg < seg_end && kv_len_of(cp_seg) == 0);
    if (cp_seg < seg_end) cp_left = kv_len_of(cp_seg);
  };
  ld_next_chunk();
  cp_next_chunk();
  if (is_part) {
    // this workgroup covers key tiles [t0, t1) of the item: walk both cursors to t0
    const int t0 = (int)((int64_t)n_tiles * part / a.part_ways);
    const int t1 = (int)((int64_t)n_tiles * (part + 1) / a.part_ways);
    int skip = t0;
    while (skip > 0 && ld_seg < seg_end) {
      const int in_chunk = (ld_left + kBK - 1) / kBK;
      if (skip >= in_chunk) {
        skip -= in_chunk;
        ld_next_chunk();
      } else {
        k_off += (uint32_t)skip * tile_bytes;
        ld_left -= skip * kBK;
        skip = 0;
      }
    }
    skip = t0;
    while (skip > 0 && cp_seg < seg_end) {
      const int in_chunk = (cp_left + kBK - 1) / kBK;
      if (skip >= in_chunk) {
        skip -= in_chunk;
        cp_next_chunk();
      } else {
        cp_left -= skip * kBK;
        skip = 0;
      }
    }
    n_tiles = t1 - t0;
  }

  // ---- tile loads: global memory -> LDS without passing through registers ---------------
  // A wavefront brings in kLoads consecutive 1 KB blocks of every K tile and of every V tile (blocks
  // kLoads * wave + i = rows kRowsPerBlock * (kLoads * wave + i) ...; consecutive, so that one M0 value serves
  // all of them).  Lane L of a load lands at LDS bytes
  // 16 L .. 16 L + 15 of the block, i.e. at row L / kChunks, chunk position L % kChunks; it
  // therefore fetches the chunk of global memory that the swizzle assigns to that position.
  // Raw buffer loads: the descriptor (base of the chunk's first key for this batch and head,
  // number of valid bytes) lives in scalar registers, the tile's offset from there travels as the
  // load's scalar offset (which the range check includes), and rows past the end of the chunk fail
  // the hardware bounds check and arrive as zeros (their scores are masked to -inf; zero V rows
  // add nothing).
  // this lane's byte offset from the tile's first key for its i-th block, loop invariant; less the 1 KB per block
  // that the immediate offset of load_next_block_to_lds adds back (a block's rows start at least that far in)
  uint32_t k_goff[T::kLoads], v_goff[T::kLoads];
#pragma unroll
  for (int i = 0; i < T::kLoads; ++i) {
    const int lrow = T::kRowsPerBlock * (T::kLoads * wave + i) + lane / T::kChunks;
    const int pos = lane % T::kChunks;
    k_goff[i] = (uint32_t)lrow * row_bytes + 16u * (uint32_t)(pos ^ T::swz_k(lrow)) - 1024u * i;
    v_goff[i] = (uint32_t)lrow * row_bytes + 16u * (uint32_t)((((pos >> 2) ^ T::swz_v(lrow)) << 2) | (pos & 3)) - 1024u * i;
  }
  static_assert(T::kLoads <= 2 && T::kRowsPerBlock * T::kRowBytes == 1024, "one immediate offset of 1 KB, whole rows per block");
  typedef __attribute__((address_space(3))) uint8_t* lds_ptr_t;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
  // Issues this wavefront's loads of V of the tile before the one under the load cursor and of
  // K of the tile under it (tile X, into K buffer X & 3; V is needed two phases later than K, so
  // its loads run one tile behind), and moves the cursor on.  Past the last tile the loads are still
  // issued, against an empty descriptor (they store zeros without touching memory): with the same
  // number of loads in every iteration the counter the barrier waits on is static.
  // V of the previous tile: its offset, and -- only in the call after the cursor changed chunks -- the
  // descriptor of the chunk it belongs to.
  uint32_t v_off = 0u;
  u32x4 rv_old = make_rsrc(nullptr, 0u);   // the very first call has no previous tile: zeros into a buffer nobody reads
  bool v_lags = true;
  auto load_tile = [&](int kbuf) __attribute__((always_inline)) {
    const int vbuf = (kbuf + kNumBuf - 1) & (kNumBuf - 1);
    const uint32_t kdst = lds_base + kbuf * T::kBytesK + wave * (1024 * T::kLoads);
    const uint32_t vdst = lds_base + T::kOffV + vbuf * T::kBytesV + wave * (1024 * T::kLoads);
    auto load_blocks = [&](const u32x4& rsrc, const uint32_t (&goff)[T::kLoads], uint32_t off, uint32_t dst) __attribute__((always_inline)) {
      load_block_to_lds(rsrc, goff[0], off, dst);
      if constexpr (T::kLoads == 2) load_next_block_to_lds(rsrc, goff[1], off);
    };
    // V first: the barrier waits let the K half of a call stay in flight one vector phase longer
    if (__builtin_expect(v_lags, 0)) {
      load_blocks(rv_old, v_goff, v_off, vdst);
      v_lags = false;
    } else {
      load_blocks(rv, v_goff, v_off, vdst);
    }
    load_blocks(rk, k_goff, k_off, kdst);
    v_off = k_off;
    k_off += tile_bytes;
    ld_left -= kBK;
    if (__builtin_expect(ld_left <= 0 && ld_seg < seg_end, 0)) {
      rv_old = rv;
      v_lags = true;
      ld_next_chunk();
    }
  };

  // ---- accumulators ---------------------------------------------------------------------
  f32x16 o_acc[D / 32];
#pragma unroll
  for (int i = 0; i < D / 32; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[i][r] = 0.f;
  // reference (raw scores; kPre: log2 units) the accumulators are scaled to
  float m_ref = kPre ? 0.f : -INFINITY;
  float rs_bias = kPre ? INFINITY : 0.f;  // kPre: inf until the row has seen a key (forces the exact path)
  bool any_off = false;                   // kPre: some row of this wavefront has a reference other than 0
  float l_run = 0.f;        // running sum over THIS lane's keys (halves combined at the end)
  const float c = kPre ? 1.f : a.scale_log2;

  // operand read addresses of this lane within a K / V buffer (the lane's part of the swizzle)
  uint32_t kld[D / 16];  // K fragment of k-step s: row key_of_row(col) (+32 for the second half tile)
  {
    const int krow = key_of_row(col);
#pragma unroll
    for (int s = 0; s < D / 16; ++s) kld[s] = krow * T::kRowBytes + 16 * ((2 * s + hh) ^ T::swz_k(krow));
  }
  // V operand: this lane is source lane 4j+m of its 16-lane block and supplies keys 8*hh + j,
  // d columns 16*(block parity) + 4m .. +3 of the fragment's 32-column segment
  uint32_t vld[T::kSegs];
  {
    const int vrow = 8 * hh + ((lane & 15) >> 2);
#pragma unroll
    for (int g = 0; g < T::kSegs; ++g)
      vld[g] = T::kOffV + vrow * T::kRowBytes + 64 * (g ^ T::swz_v(vrow)) + (16 * ((lane >> 4) & 1) + 4 * (lane & 3)) * 2;
  }

  f32x16 s_acc[2];       // S^T of the tile whose softmax comes next
  ex8 p_frag[2][2];      // P^T of the tile whose P V product comes next
  int cp_valid = 0;      // keys that exist in the tile held in s_acc

  // S^T = K Q^T for tile 0 only (first matrix phase)
  auto qk_only = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s_acc[kb][r] = 0.f;
#pragma unroll
      for (int s = 0; s < D / 16; ++s) {
        const ex8 ka = *reinterpret_cast<const ex8*>(lds + kld[s] + kb * 32 * T::kRowBytes);
        s_acc[kb] = E::mfma(ka, qf[s], s_acc[kb]);
      }
    }
  };

  // One matrix phase: O^T += V^T P^T for tile `tile`, then S^T = K Q^T for tile `tile + 1`,
  // as ONE stream of MFMAs fed by a ring of LDS reads kept kRing fragments ahead, so that the
  // single wavefront of this SIMD that is in its matrix phase never waits for LDS latency.
  // (After the last tile the second half recomputes scores on a stale K buffer; they are unused.)
  // U = tile & 3 picks the buffers at compile time: all operand reads use immediate offsets.
  constexpr int kPV = D / 32 * 4;       // fragments of the P V product
  constexpr int kQK = 2 * (D / 16);     // fragments of the score product
  constexpr int kFrags = kPV + kQK;
  constexpr int kRing = kRingDepth;
  // Where a wavefront issues its tile loads: at the start of its vector phase, or behind the
  // MFMAs of its matrix phase (one phase later, and then awaited one call earlier).  At D = 64
  // the vector phase is the longer one (half the MFMAs per softmax element) and the matrix
  // phase has the room (measured +16 %); at D = 128 it is the other way round (+1.5 %).
  constexpr bool kLoadAfterMatrix = (D == 64 ? DT_SCHED_LOAD_AFTER_MATRIX_D64 : DT_SCHED_LOAD_AFTER_MATRIX_D128) != 0;
  static_assert(T::kLoads == (D == 64 ? DT_SCHED_LOADS_D64 : DT_SCHED_LOADS_D128),
                "attn_schedule.h states how many load instructions a wavefront issues per tile and operand");
  // shares of tile loads that may stay in flight across the barrier that ends a vector phase
  constexpr int kVectorInFlight = D == 64 ? DT_SCHED_VECTOR_BARRIER_INFLIGHT_D64 : DT_SCHED_VECTOR_BARRIER_INFLIGHT_D128;
  static_assert(DT_SCHED_PROLOGUE_CALLS_LEADING == DT_SCHED_CALL_AHEAD && DT_SCHED_PROLOGUE_CALLS_TRAILING == DT_SCHED_CALL_AHEAD + 1,
                "the prologue issues exactly the calls the loop's first phase pair assumes: tiles 0 .. 2 + group");
  // The operand ring lives across the barrier in front of a matrix phase: its first kRing
  // fragments (V fragments of a tile completed at least a phase ago) are read at the END of the
  // preceding vector phase, so their LDS latency passes while the wavefront waits at the barrier
  // instead of in front of the first MFMA.
  ex8 ring[kRing];
  auto v_frag = [&](int vbuf, int i) __attribute__((always_inline)) -> ex8 {
    // 8 consecutive keys of one d column = two transposing reads of 4 keys each
    const int db = i % (D / 32), kb = (i / (D / 32)) >> 1, half = (i / (D / 32)) & 1;
    const uint8_t* p = lds + vld[db] + vbuf * T::kBytesV + (32 * kb + 16 * half) * T::kRowBytes;
    const s16x4 lo = lds_read_tr(p);
    const s16x4 hi = lds_read_tr(p + 4 * T::kRowBytes);
    const s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(ex8, both);
  };
  auto ring_prefill = [&](auto u_tag) __attribute__((always_inline)) {
    constexpr int kU = decltype(u_tag)::value;
#pragma unroll
    for (int i = 0; i < kRing; ++i) ring[i] = v_frag(kU, i);
  };
  auto matrix_phase = [&](auto u_tag) __attribute__((always_inline)) {
    constexpr int kU = decltype(u_tag)::value;         // V buffer of this tile
    constexpr int kUK = (kU + 1) & (kNumBuf - 1);      // K buffer of the next tile
    auto frag = [&](int i) -> ex8 {
      if (i < kPV) return v_frag(kU, i);
      const int j = i - kPV;
      const int kb = j & 1, sidx = j >> 1;
      return *reinterpret_cast<const ex8*>(lds + kld[sidx] + kUK * T::kBytesK + kb * 32 * T::kRowBytes);
    };
#pragma unroll
    for (int i = 0; i < kFrags; ++i) {
      const ex8 cur = ring[i % kRing];
      if (i + kRing < kFrags) ring[i % kRing] = frag(i + kRing);
      if (i < kPV) {
        const int db = i % (D / 32), kb = (i / (D / 32)) >> 1, half = (i / (D / 32)) & 1;
        o_acc[db] = E::mfma(cur, p_frag[kb][half], o_acc[db]);
      } else {
        const int j = i - kPV;
        const int kb = j & 1, sidx = j >> 1;
        if (sidx == 0) {
          f32x16 zero;
#pragma unroll
          for (int r = 0; r < 16; ++r) zero[r] = 0.f;
          s_acc[kb] = E::mfma(cur, qf[sidx], zero);
        } else {
          s_acc[kb] = E::mfma(cur, qf[sidx], s_acc[kb]);
        }
      }
    }
    // pin the order: the reads of kRing fragments up front (a V fragment is two reads), then the
    // reads of one more fragment behind every MFMA
    static_assert(kRing <= kPV, "the prefill is assumed to consist of V fragments");
#pragma unroll
    for (int i = 0; i < kPV - kRing; ++i) {   // MFMAs whose refill is a V fragment
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
#pragma unroll
    for (int i = 0; i < kQK; ++i) {           // MFMAs whose refill is a K fragment
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, kRing, 0);
  };

  // ---- prologue ---------------------------------------------------------------------------
  // Schedule of the loads (phases are separated by workgroup barriers; group g runs the vector
  // phase of tile t in phase 2t + g and its matrix phase in phase 2t + g + 1):
  //   * K of tile X is read in phases 2X-1 and 2X (scores, matrix phases of tile X-1), V of tile X
  //     at the end of phases 2X and 2X+1 (the operand ring's prefill) and in phases 2X+1 and 2X+2.
  //   * A call of load_tile issues V of tile Y-1 and then K of tile Y.  In the vector phase of
  //     tile t a wavefront of group g makes the call Y = t+3+g: with four buffers per operand the
  //     slot a load overwrites (K of tile Y-4: last read in phase 2Y-8; V of tile Y-5: phase 2Y-8)
  //     is free since the barrier before the phase the load is issued in (2Y-6 or 2Y-7).
  //   * The barrier that ends a vector phase waits for all of the wavefront's loads but the newest
  //     call and the K half of the call before: V of tile t+1+g and K of tile t+1+g are then in
  //     the LDS for everybody, i.e. V one barrier before its first reader (the prefill in phase
  //     2(t+1) + g at the earliest) after three phases in flight, K after five.
  //   * At D = 64 the calls are made behind the MFMAs of the matrix phase instead (see
  //     kLoadAfterMatrix); the barrier of the next vector phase then lets only the K half of the
  //     newest call stay in flight.
  // Here: the calls Y = 0..2 (group 1: ..3) -- the V half of the first has no tile, it stores
  // zeros into a buffer nobody reads -- of which K of tile 0 (first scores) and V of tile 0 (first
  // prefill) are awaited; the trailing group then waits one phase, which staggers the two groups.
  using U0 = std::integral_constant<int, 0>;
  using U1 = std::integral_constant<int, 1>;
  using U2 = std::integral_constant<int, 2>;
  using U3 = std::integral_constant<int, 3>;
#pragma unroll
  for (int y = 0; y < DT_SCHED_PROLOGUE_CALLS_LEADING; ++y) load_tile(y);
  if (group == 1) {
#pragma unroll
    for (int y = DT_SCHED_PROLOGUE_CALLS_LEADING; y < DT_SCHED_PROLOGUE_CALLS_TRAILING; ++y) load_tile(y);
  }
  // in flight behind this wait: K of tile 1 and the calls after it (kLoads + 2 kLoads (1 + g) loads)
  if (group == 0) wait_tile_loads<DT_SCHED_PROLOGUE_INFLIGHT_LEADING * T::kLoads>();
  else wait_tile_loads<DT_SCHED_PROLOGUE_INFLIGHT_TRAILING * T::kLoads>();
  phase_barrier();
  if (group == 1) phase_barrier();
  // first matrix phase: scores of tile 0
  if (n_tiles > 0) {
    qk_only();
    cp_valid = cp_left;
    cp_left -= kBK;
    if (cp_left <= 0) cp_next_chunk();
  }
  // Behind this barrier the leading group computes the scores of tile 1, so K of tile 1 has to be in
  // the LDS from ALL wavefronts.  The leading group waits for its share at the end of its vector
  // phase; the trailing group is in its score-only phase here and has no vector phase in between,
  // so it waits for its share now (of its 8 kLoads loads, the 4 kLoads oldest: V(-1), K0, V0, K1).
  // From tile 2 on, the wait that ends a group's vector phase covers the tile the other group
  // reads next.
  if (group == 1) wait_tile_loads<DT_SCHED_TRAILING_K1_INFLIGHT * T::kLoads>();
  phase_barrier_after_matrix(s_acc, o_acc);

  // one iteration = vector phase of tile t, then matrix phase (P V of tile t, scores of t+1)
  auto iteration = [&](int t, auto u_tag) __attribute__((always_inline)) {
    constexpr int kU = decltype(u_tag)::value;  // t & 3
    // ======== vector phase: tile loads for later, online softmax of tile t ========
    // The vector phase runs at raised wave priority: where the two wavefronts of a SIMD compete for
    // the vector issue port, the one doing the softmax goes first.  With equal priorities the older
    // wavefront wins in either role and the phases of the two groups come out unequal (measured
    // 1.43k vs 1.24k cycles of vector work), so every other barrier waits for a squeezed softmax.
    // (D = 64: four wavefronts of two workgroups share the SIMD and the raised priority only gets in
    // the way of the other workgroup's matrix phase: measured -3 %, so it is left at 0 there)
    __builtin_amdgcn_s_setprio(D == 64 ? 0 : 1);
    if constexpr (!kLoadAfterMatrix) load_tile((kU + DT_SCHED_CALL_AHEAD + group) & (kNumBuf - 1));
    // (kPre: the same rare branch takes the reference off the scores of a wavefront in which some
    // row has left the band; everywhere else the reference is 0 and there is nothing to subtract)
    if (__builtin_expect(cp_valid < kBK || (kPre && any_off), 0)) {
      // the empty asm has side effects as far as the compiler knows, which keeps this a real
      // branch: otherwise the selects below are hoisted out and run for every tile
      asm volatile("" ::: "memory");
      const int lim = cp_valid;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = 32 * kb + 16 * (r >> 3) + 8 * hh + (r & 7);
          if (key >= lim) s_acc[kb][r] = -INFINITY;
          if constexpr (kPre) s_acc[kb][r] -= m_ref;
        }
    }
    // Probabilities relative to the reference maximum the accumulators are scaled to.  The
    // maximum of the tile is NOT computed on this path: the row sum, needed anyway, doubles as
    // the overflow detector.  While it stays below kSumLimit every probability is bounded and a
    // lagging reference is harmless (the lse stays exact); otherwise -- including the first tile,
    // where the reference is -inf and the sum comes out inf or NaN -- the tile is redone below
    // with its exact maximum.
    float mc = m_ref * c;
    float rs0 = rs_bias, rs1 = 0.f;
    // The first tile of a work item always takes the exact path below (its reference is still -inf), so its pass
    // through the common path is thrown away: skip it.  Results are bit-identical; +0.4-0.5 % at D = 128.  (At
    // D = 64 the extra branch costs registers the kernel does not have: 36 spills, -18 %; it keeps the plain form.)
    if (D == 128 && __builtin_expect(t == 0, 0)) {
      asm volatile("" ::: "memory");   // keeps this a real branch
      rs0 = INFINITY;
    } else
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; r += 2) {
        f32x2 p;
        if constexpr (kPre) {
          p.x = __builtin_amdgcn_exp2f(s_acc[kb][r]);
          p.y = __builtin_amdgcn_exp2f(s_acc[kb][r + 1]);
        } else {
          p.x = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kb][r], c, -mc));
          p.y = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kb][r + 1], c, -mc));
        }
        if (!kPre && kb == 0 && r == 0) {   // the sums start from these two (0 + p is not folded: it would turn -0 into +0)
          rs0 = p.x;
          rs1 = p.y;
        } else {
          rs0 += p.x;
          rs1 += p.y;
        }
        const ex2 pb = __builtin_convertvector(p, ex2);
        p_frag[kb][r >> 3][r & 7] = pb.x;
        p_frag[kb][r >> 3][(r & 7) + 1] = pb.y;
      }
    if (__builtin_expect(__any(!(rs0 + rs1 <= (kPre ? kSumLimitPre : kSumLimit))), 0)) {
      float mx = s_acc[0][0];
#pragma unroll
      for (int r = 1; r < 16; ++r) mx = fmaxf(mx, s_acc[0][r]);
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s_acc[1][r]);
      mx = fmaxf(mx, __shfl_xor(mx, 32));
      float m_new, alpha;
      if constexpr (kPre) {
        float rs_tot = rs0 + rs1;
        rs_tot += __shfl_xor(rs_tot, 32);
        const bool first = rs_bias != 0.f;
        const float mx_true = mx + m_ref;
        if (first) m_new = (mx_true >= kBandLo && mx_true <= kBandHi) || !(mx_true > -INFINITY) ? 0.f : mx_true;
        else m_new = !(rs_tot <= kSumLimitPre) ? fmaxf(m_ref, mx_true) : m_ref;
        alpha = first ? 1.f : __builtin_amdgcn_exp2f(m_ref - m_new);
        rs_bias = first && !(mx > -INFINITY) ? INFINITY : 0.f;
        mx = m_new - m_ref;  // what the scores in s_acc still have to lose
      } else {
        m_new = fmaxf(m_ref, mx);
        alpha = m_new > -INFINITY ? __builtin_amdgcn_exp2f((m_ref - m_new) * c) : 1.f;
      }
      m_ref = m_new;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < D / 32; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[i][r] *= alpha;
      // a row whose keys are all masked so far keeps m_ref = -inf: use 0 so that exp2(-inf - 0) = 0
      mc = kPre ? mx : (m_new > -INFINITY ? m_new * c : 0.f);
      if constexpr (kPre) any_off = any_off || __any(m_ref != 0.f);
      rs0 = 0.f;
      rs1 = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; r += 2) {
          f32x2 p;
          p.x = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kb][r], c, -mc));
          p.y = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[kb][r + 1], c, -mc));
          rs0 += p.x;
          rs1 += p.y;
          const ex2 pb = __builtin_convertvector(p, ex2);
          p_frag[kb][r >> 3][r & 7] = pb.x;
          p_frag[kb][r >> 3][(r & 7) + 1] = pb.y;
        }
    }
    l_run += rs0 + rs1;
    ring_prefill(u_tag);
    phase_barrier_after_vector<kVectorInFlight * T::kLoads>(p_frag);

    // ======== matrix phase: O^T += V^T P^T (tile t), S^T = K Q^T (tile t+1) ========
    __builtin_amdgcn_s_setprio(0);
    matrix_phase(u_tag);
    if constexpr (kLoadAfterMatrix) load_tile((kU + DT_SCHED_CALL_AHEAD + group) & (kNumBuf - 1));
    // the tile after the last one of this workgroup's range has no keys for it (its scores are
    // computed on whatever the buffer holds and never used; it may belong to the next part of a
    // split item)
    cp_valid = t + 1 < n_tiles ? cp_left : 0;
    cp_left -= kBK;
    if (cp_left <= 0) cp_next_chunk();
    phase_barrier_after_matrix(s_acc, o_acc);
  };
  // Iterations come in fours (one per LDS buffer, so that buffer offsets are immediates); the last
  // round stops after the last tile.
  for (int t = 0; t < n_tiles; t += 4) {
    iteration(t, U0{});
    if (t + 1 >= n_tiles) break;
    iteration(t + 1, U1{});
    if (t + 2 >= n_tiles) break;
    iteration(t + 2, U2{});
    if (t + 3 >= n_tiles) break;
    iteration(t + 3, U3{});
  }
  // tile loads issued for tiles past the end are still on their way (they store zeros): let them
  // land before the epilogue reuses the tile buffers
  wait_tile_loads<0>();
  // the leading group waits out the phase it is ahead
  if (group == 0) phase_barrier();

  // ---- epilogue -------------------------------------------------------------------------
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  const float lse = l_tot > 0.f ? (m_ref * c + __builtin_amdgcn_logf(l_tot)) * 0.6931471805599453f : -INFINITY;
  const int qrow = q0 + col;
  // tail launch: the partial state goes to this workgroup's workspace slot, [256 queries][D] + [256]
  const int64_t ws_slot = (((int64_t)(idx - a.tail_idx0) * kXcds + xcd) * a.part_ways + part);
  if (is_part) {
    if (hh == 0) a.ws_lse[ws_slot * kBQ + wave * 32 + col] = lse;
  } else if (hh == 0 && qrow < q_end) {
    lse_ptr[((int64_t)b * a.H + h) * a.Sq + qrow] = lse;
  }

  // O^T (registers, [d][query]) -> LDS [query][d] in the element type -> coalesced 16-byte stores.
  phase_barrier();  // every wavefront is done with the tile buffers
  uint8_t* ol = lds + wave * (32 * T::kPitchO);
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x2 lo, hi;
      lo.x = o_acc[db][4 * g + 0] * inv;
      lo.y = o_acc[db][4 * g + 1] * inv;
      hi.x = o_acc[db][4 * g + 2] * inv;
      hi.y = o_acc[db][4 * g + 3] * inv;
      const ex2 l2 = __builtin_convertvector(lo, ex2);
      const ex2 h2 = __builtin_convertvector(hi, ex2);
      ex4 pk;
      pk.x = l2.x; pk.y = l2.y; pk.z = h2.x; pk.w = h2.y;
      const int d = 32 * db + 8 * g + 4 * hh;
      *reinterpret_cast<ex4*>(ol + col * T::kPitchO + d * 2) = pk;
    }
  phase_barrier();
  constexpr int kLanesPerRow = D / 8;
  constexpr int kRowsPerPass = 64 / kLanesPerRow;
  const int rr = lane / kLanesPerRow;
  const int cc = lane % kLanesPerRow;
#pragma unroll
  for (int p = 0; p < 32 / kRowsPerPass; ++p) {
    const int row = p * kRowsPerPass + rr;
    const int qg = q0 + row;
    const u32x4 val = *reinterpret_cast<const u32x4*>(ol + row * T::kPitchO + cc * 16);
    if (is_part) {
      uint16_t* dst = a.ws_out + (ws_slot * kBQ + wave * 32 + row) * D + cc * 8;
      *reinterpret_cast<u32x4*>(dst) = val;
    } else if (qg < q_end) {
      uint16_t* dst = out_ptr + (((int64_t)b * a.Sq + qg) * a.H + h) * D + cc * 8;
      __builtin_nontemporal_store(val, reinterpret_cast<u32x4*>(dst));
    }
  }
}

// Folds the part_ways partial states of every tail item into the item's rows of its destination.
// One workgroup per item and slice of 256 / (D/8) rows; a group of D/8 lanes owns a row.
template <int D, bool kHalf>
__global__ __launch_bounds__(256) void attn_tail_fold_kernel(const AttnArgs a) {
  using E = Elem<kHalf>;
  constexpr int kSlices = kBQ / (256 / (D / 8));
  const int slot_id = blockIdx.x / kSlices;
  const int slice = blockIdx.x - slot_id * kSlices;
  const int xcd = slot_id & (kXcds - 1);
  const int u = slot_id >> 3;
  const int idx = a.tail_idx0 + u;
  const int item = xcd * a.per_xcd + idx;
  if (idx >= a.per_xcd || item >= a.total) return;
  const int bh = item / a.nqt;
  const int qt = item - bh * a.nqt;
  const int b = bh / a.H;
  const int h = bh - b * a.H;
  const int job = a.tail_job;
  uint16_t* out_ptr;
  float* lse_ptr;
  if (a.dev_ids != nullptr) {
    if (job >= *a.dev_count) return;
    const int single = a.dev_ids[job];
    if (single < 0 || single >= a.n_chunks) return;
    out_ptr = single == a.diag ? a.diag_out : a.slot_out + (int64_t)single * a.slot_out_stride;
    lse_ptr = single == a.diag ? a.diag_lse : a.slot_lse + (int64_t)single * a.slot_lse_stride;
  } else {
    out_ptr = a.job_out[job];
    lse_ptr = a.job_lse[job];
  }
  constexpr int kLanes = D / 8;
  constexpr int kRows = 256 / kLanes;
  const int rr = threadIdx.x / kLanes;
  const int cc = threadIdx.x % kLanes;
  const int64_t slot0 = ((int64_t)u * kXcds + xcd) * a.part_ways;
  {
    const int row = slice * kRows + rr;
    const int qg = qt * kBQ + row;
    if (qg >= a.Sq) return;
    float m = -INFINITY;
    for (int p = 0; p < a.part_ways; ++p) m = fmaxf(m, a.ws_lse[(slot0 + p) * kBQ + row]);
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    float den = 0.f;
    if (m > -INFINITY) {
      for (int p = 0; p < a.part_ways; ++p) {
        const float w = __expf(a.ws_lse[(slot0 + p) * kBQ + row] - m);
        const u32x4 v = *reinterpret_cast<const u32x4*>(a.ws_out + ((slot0 + p) * kBQ + row) * D + cc * 8);
        const uint32_t e[4] = {v.x, v.y, v.z, v.w};
        den += w;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const f32x2 x = E::widen(e[k]);
          acc[2 * k] = __builtin_fmaf(w, x.x, acc[2 * k]);
          acc[2 * k + 1] = __builtin_fmaf(w, x.y, acc[2 * k + 1]);
        }
      }
    }
    const float inv = den > 0.f ? 1.f / den : 0.f;
    u32x4 o;
    uint32_t pk[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      f32x2 f;
      f.x = acc[2 * k] * inv;
      f.y = acc[2 * k + 1] * inv;
      pk[k] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, typename E::x2));
    }
    o.x = pk[0]; o.y = pk[1]; o.z = pk[2]; o.w = pk[3];
    *reinterpret_cast<u32x4*>(out_ptr + (((int64_t)b * a.Sq + qg) * a.H + h) * D + cc * 8) = o;
    if (cc == 0) lse_ptr[((int64_t)b * a.H + h) * a.Sq + qg] = den > 0.f ? m + __logf(den) : -INFINITY;
  }
}

static_assert(Tile<128>::kLdsBytes == kAttnLdsBytes128 && Tile<64>::kLdsBytes == kAttnLdsBytes64,
              "dt_common.h states the LDS footprint of the attention kernel");

template <int D, bool kPre, bool kHalf>
static int launch_one(const AttnArgs& a, dim3 grid, hipStream_t stream) {
  // more than 64 KB of dynamic LDS has to be allowed once per kernel and device
  static thread_local int allowed_dev = -1;
  int dev = 0;
  if (int rc = hip_fail(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (allowed_dev != dev) {
    if (int rc = hip_fail(hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_fwd_kernel<D, kPre, kHalf>),
                                              hipFuncAttributeMaxDynamicSharedMemorySize, Tile<D>::kLdsBytes),
                          "hipFuncSetAttribute"))
      return rc;
    allowed_dev = dev;
  }
  hipLaunchKernelGGL((attn_fwd_kernel<D, kPre, kHalf>), grid, dim3(kThreads), Tile<D>::kLdsBytes, stream, a);
  return hip_fail(hipGetLastError(), "attn_fwd launch");
}

static int launch_dim(const AttnArgs& a, int D, dim3 grid, hipStream_t stream) {
  if (a.elem_f16) {
    if (D == 128) return launch_one<128, false, true>(a, grid, stream);
    return launch_one<64, false, true>(a, grid, stream);
  }
  if (a.q_prescaled) {
    if (D == 128) return launch_one<128, true, false>(a, grid, stream);
    return launch_one<64, true, false>(a, grid, stream);
  }
  if (D == 128) return launch_one<128, false, false>(a, grid, stream);
  return launch_one<64, false, false>(a, grid, stream);
}

// Number of CUs of the current device (one workgroup of the attention kernel per CU at a time).
static int cu_count() {
  static thread_local int cached_dev = -1, cached = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (dev != cached_dev) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached = n;
    cached_dev = dev;
  }
  return cached;
}

// Scratch of the allocation-free entry point: the tail-balancing workspace as a device array that
// lives as long as the code object (one copy per GPU, at that GPU's own address).  Host code never
// uses the array's name as an address: static_tail_scratch() asks the runtime for the device
// address once per device and hands that out.
static __device__ __align__(256) uint8_t g_tail_scratch[kStaticTailBytes];

int static_tail_scratch(void** ptr, int64_t* bytes) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* addr[kMaxDevices] = {};
  int dev = 0;
  if (int rc = hip_fail(hipGetDevice(&dev), "hipGetDevice")) return rc;
  if (dev < 0 || dev >= kMaxDevices) {
    set_error("device ordinal %d outside the %d the static scratch table covers", dev, kMaxDevices);
    return DT_ERR_UNSUPPORTED;
  }
  std::lock_guard<std::mutex> lock(mu);
  if (addr[dev] == nullptr) {
    void* p = nullptr;
    if (int rc = hip_fail(hipGetSymbolAddress(&p, HIP_SYMBOL(g_tail_scratch)), "hipGetSymbolAddress(tail scratch)"))
      return rc;
    if (p == nullptr || (reinterpret_cast<uintptr_t>(p) & 255) != 0) {
      set_error("the runtime returned an unusable address for the static tail scratch");
      return DT_ERR_HIP;
    }
    addr[dev] = p;
  }
  *ptr = addr[dev];
  *bytes = kStaticTailBytes;
  return DT_OK;
}

int launch_attn(const AttnArgs& a_in, int D, int n_jobs, hipStream_t stream, void* workspace,
                int64_t workspace_bytes, bool balance) {
  if (n_jobs <= 0 || a_in.total <= 0) return DT_OK;
  if (D != 128 && D != 64) {
    set_error("head dim %d not built (64 and 128 are)", D);
    return DT_ERR_UNSUPPORTED;
  }
  if (a_in.elem_f16 && a_in.q_prescaled) {
    set_error("fp16 tensors and a prescaled q do not combine (the prescaled softmax keeps probabilities beyond fp16's range)");
    return DT_ERR_UNSUPPORTED;
  }
  AttnArgs a = a_in;
  a.n_jobs = n_jobs;
  a.tail_job = -1;
  a.tail_idx0 = 0;
  a.tail_items = 0;
  a.part_ways = 0;
  const int slots_per_job = a.per_xcd * kXcds;
  // ---- tail balancing: is the last round of workgroups worth splitting? -------------------
  // Time is counted in key tiles.  Unsplit, the launch takes ceil(n / cus) rounds of one item
  // (n_tiles tiles each).  With the last `rem` items cut into w parts, the parts are handed to
  // CUs as they come free (same launch, no barrier in between), so the tail takes
  // ceil(rem * w / cus) rounds of (n_tiles / w + kPartOverhead) tiles plus the fold kernel.
  int tail = 0, ways = 0;
  const int cus = balance && workspace ? cu_count() : 0;
  const int64_t slot_bytes = (int64_t)kBQ * D * 2 + (int64_t)kBQ * 4;
  if (cus >= 64 && cus % kXcds == 0 && a.total == slots_per_job) {
    int n_tiles = 0;  // key tiles of one item of the last job (device-listed jobs: of the longest chunk)
    if (a.dev_ids != nullptr) {
      for (int c = 0; c < a.n_chunks; ++c) n_tiles = std::max(n_tiles, (a.kv_len[c] + kBK - 1) / kBK);
    } else {
      for (int e = a.job_begin[n_jobs - 1]; e < a.job_begin[n_jobs]; ++e) n_tiles += (a.entry_kv_len[e] + kBK - 1) / kBK;
    }
    // Measured on the HunyuanVideo, Step-Video and CogVideoX shares: a part costs about 6 tiles on
    // top of its own (start-up, epilogue, partial state) when all parts run at once and about 10
    // when they take several rounds, so many small parts only pay in the first case.
    constexpr double kPartOverheadOneRound = 6.0, kPartOverheadRounds = 10.0;
    constexpr double kFoldOverhead = 4.0;  // the fold kernel's launch
    const int64_t n = (int64_t)n_jobs * slots_per_job;
    const int rem = (int)(n % cus);
    const int64_t cap = std::min<int64_t>(workspace_bytes / slot_bytes, kMaxTailSlots);
    if (rem > 0 && rem <= slots_per_job && rem < n && n_tiles >= 16) {
      double best = 0.1 * n_tiles;  // least gain worth the extra kernel
      for (int w = 2; w <= 16; ++w) {
        if ((int64_t)rem * w > cap || n_tiles / w < 6) break;
        const int rounds = (int)(((int64_t)rem * w + cus - 1) / cus);
        const double split = rounds * ((double)n_tiles / w + (rounds == 1 ? kPartOverheadOneRound : kPartOverheadRounds)) + kFoldOverhead;
        if (n_tiles - split > best) {
          best = n_tiles - split;
          tail = rem;
          ways = w;
        }
      }
    }
  }
  if (tail == 0) return launch_dim(a, D, dim3((unsigned)slots_per_job, (unsigned)n_jobs, 1), stream);
  // (the planner only considers splits of at most `cap` slots, so this cannot fire; it guards later edits to it)
  if ((int64_t)tail * ways * slot_bytes > workspace_bytes) {
    set_error("internal: tail split of %d items x %d parts needs %lld bytes of scratch, %lld are there", tail, ways,
              (long long)((int64_t)tail * ways * slot_bytes), (long long)workspace_bytes);
    return DT_ERR_INVALID;
  }
  a.tail_job = n_jobs - 1;
  a.tail_idx0 = a.per_xcd - tail / kXcds;
  a.tail_items = tail / kXcds;
  a.part_ways = ways;
  a.ws_out = static_cast<uint16_t*>(workspace);
  a.ws_lse = reinterpret_cast<float*>(static_cast<uint8_t*>(workspace) + (int64_t)tail * ways * kBQ * D * 2);
  // parts per XCD lane of the grid: tail / 8 items x ways parts, spread over extra planes of per_xcd entries
  const int part_planes = (a.tail_items * ways + a.per_xcd - 1) / a.per_xcd;
  if (int rc = launch_dim(a, D, dim3((unsigned)slots_per_job, (unsigned)(n_jobs + part_planes), 1), stream)) return rc;
  if (D == 128) {
    if (a.elem_f16) hipLaunchKernelGGL((attn_tail_fold_kernel<128, true>), dim3((unsigned)tail * 16), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((attn_tail_fold_kernel<128, false>), dim3((unsigned)tail * 16), dim3(256), 0, stream, a);
  } else {
    if (a.elem_f16) hipLaunchKernelGGL((attn_tail_fold_kernel<64, true>), dim3((unsigned)tail * 8), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL((attn_tail_fold_kernel<64, false>), dim3((unsigned)tail * 8), dim3(256), 0, stream, a);
  }
  return hip_fail(hipGetLastError(), "attn tail fold launch");
}

}  // namespace dt
