// A caller of libditango_hip.so that knows nothing but the C header and the HIP runtime: two KV chunks of
// attention (dt_attn_jobs_fwd), their merge (dt_merge_states), a trip through a cache slot
// (dt_cache_store / dt_cache_load), a device-built schedule (dt_build_schedule) and a packed variable-length
// batch whose segment boundaries live in device memory (dt_attn_varlen_jobs_fwd, dt_zero_rows_from), each checked
// against plain host loops in double precision.  Exit status 0 = everything within the library's stated bounds
// (out 2e-2, lse 1e-3, integer results exact).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

#include "ditango_hip.h"

#define HIP_OK(call)                                                                        \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));                \
      return 2;                                                                             \
    }                                                                                       \
  } while (0)
#define DT_CHECK(call)                                                                      \
  do {                                                                                      \
    int rc_ = (call);                                                                       \
    if (rc_ != DT_OK) {                                                                     \
      std::fprintf(stderr, "%s returned %d: %s\n", #call, rc_, dt_last_error());            \
      return 3;                                                                             \
    }                                                                                       \
  } while (0)

static uint16_t to_bf16(float x) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &x, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float x;
  std::memcpy(&x, &u, 4);
  return x;
}
static float rnd(uint64_t& s) {  // uniform in [-1, 1)
  s = s * 6364136223846793005ull + 1442695040888963407ull;
  return (float)((s >> 40) & 0xffffff) / 8388608.0f - 1.0f;
}

int main() {
  const int B = 1, H = 8, D = 64, Sq = 70, n_chunks = 2;
  const int Sk[2] = {100, 37};
  uint64_t seed = 12345;
  std::vector<uint16_t> q((size_t)B * Sq * H * D);
  for (auto& x : q) x = to_bf16(rnd(seed));
  std::vector<uint16_t> k[2], v[2];
  for (int c = 0; c < n_chunks; ++c) {
    k[c].resize((size_t)B * Sk[c] * H * D);
    v[c].resize(k[c].size());
    for (auto& x : k[c]) x = to_bf16(2.0f * rnd(seed));
    for (auto& x : v[c]) x = to_bf16(rnd(seed));
  }
  auto at = [&](const std::vector<uint16_t>& t, int s, int h, int d) { return (double)from_bf16(t[((size_t)s * H + h) * D + d]); };

  // ---- host reference: per-chunk states and the full result -------------------------------------
  const double scale = 1.0 / std::sqrt((double)D);
  std::vector<double> ref_out((size_t)Sq * H * D, 0.0), ref_lse((size_t)H * Sq, 0.0);
  std::vector<double> ref_clse[2];
  for (int c = 0; c < n_chunks; ++c) ref_clse[c].assign((size_t)H * Sq, 0.0);
  for (int h = 0; h < H; ++h)
    for (int s = 0; s < Sq; ++s) {
      std::vector<double> sc;
      double mx = -1e300;
      for (int c = 0; c < n_chunks; ++c)
        for (int j = 0; j < Sk[c]; ++j) {
          double d = 0;
          for (int e = 0; e < D; ++e) d += at(q, s, h, e) * at(k[c], j, h, e);
          sc.push_back(d * scale);
          mx = std::fmax(mx, d * scale);
        }
      double den = 0;
      size_t i = 0;
      for (int c = 0; c < n_chunks; ++c) {
        double dc = 0;
        for (int j = 0; j < Sk[c]; ++j, ++i) {
          const double p = std::exp(sc[i] - mx);
          dc += p;
          for (int e = 0; e < D; ++e) ref_out[((size_t)s * H + h) * D + e] += p * at(v[c], j, h, e);
        }
        ref_clse[c][(size_t)h * Sq + s] = mx + std::log(dc);
        den += dc;
      }
      for (int e = 0; e < D; ++e) ref_out[((size_t)s * H + h) * D + e] /= den;
      ref_lse[(size_t)h * Sq + s] = mx + std::log(den);
    }

  // ---- device buffers ----------------------------------------------------------------------------
  void *dq, *dk[2], *dv[2], *dso[2], *dout, *slot_o, *back_o;
  float *dsl[2], *dlse, *slot_l, *back_l;
  const size_t state_elems = (size_t)B * Sq * H * D, lse_elems = (size_t)B * H * Sq;
  HIP_OK(hipMalloc(&dq, q.size() * 2));
  HIP_OK(hipMemcpy(dq, q.data(), q.size() * 2, hipMemcpyHostToDevice));
  for (int c = 0; c < n_chunks; ++c) {
    HIP_OK(hipMalloc(&dk[c], k[c].size() * 2));
    HIP_OK(hipMalloc(&dv[c], v[c].size() * 2));
    HIP_OK(hipMemcpy(dk[c], k[c].data(), k[c].size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dv[c], v[c].data(), v[c].size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMalloc(&dso[c], state_elems * 2));
    HIP_OK(hipMalloc((void**)&dsl[c], lse_elems * 4));
  }
  HIP_OK(hipMalloc(&dout, state_elems * 4));
  HIP_OK(hipMalloc((void**)&dlse, lse_elems * 4));
  HIP_OK(hipMalloc(&slot_o, state_elems * 2));
  HIP_OK(hipMalloc((void**)&slot_l, lse_elems * 4));
  HIP_OK(hipMalloc(&back_o, state_elems * 4));
  HIP_OK(hipMalloc((void**)&back_l, lse_elems * 4));
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));

  // ---- one launch: a state per chunk ---------------------------------------------------------------
  const void* kp[2] = {dk[0], dk[1]};
  const void* vp[2] = {dv[0], dv[1]};
  const int32_t lens[2] = {Sk[0], Sk[1]};
  const int64_t kv_sb[2] = {(int64_t)Sk[0] * H * D, (int64_t)Sk[1] * H * D};
  const int32_t job_begin[3] = {0, 1, 2}, job_chunks[2] = {0, 1};
  void* outs[2] = {dso[0], dso[1]};
  float* lses[2] = {dsl[0], dsl[1]};
  DT_CHECK(dt_attn_jobs_fwd(dq, B, Sq, H, D, (int64_t)Sq * H * D, (int64_t)H * D, D, n_chunks, kp, vp, lens, kv_sb,
                            (int64_t)H * D, D, 2, job_begin, job_chunks, outs, lses, 0.f, stream));
  // ---- merge of the two states into an fp32 result ---------------------------------------------------
  const void* mo[2] = {dso[0], dso[1]};
  const float* ml[2] = {dsl[0], dsl[1]};
  DT_CHECK(dt_merge_states(2, mo, ml, nullptr, nullptr, dout, DT_FP32, dlse, DT_LSE_BHS, B, Sq, H, D, stream));
  // ---- the fp32 result through a cache slot and back ---------------------------------------------------
  DT_CHECK(dt_cache_store(dout, DT_FP32, dlse, DT_LSE_BHS, slot_o, slot_l, B, Sq, H, D, stream));
  DT_CHECK(dt_cache_load(slot_o, slot_l, back_o, DT_FP32, back_l, DT_LSE_BHS, B, Sq, H, D, stream));
  // ---- a schedule row built on the device ---------------------------------------------------------------
  const int T = 2, L = 3, C = 8;
  std::vector<uint8_t> mask((size_t)T * L * C);
  for (auto& m : mask) m = rnd(seed) > 0.f ? 1 : 0;
  uint8_t* dmask;
  int32_t *dcomp, *dreu, *dcnt;
  HIP_OK(hipMalloc((void**)&dmask, mask.size()));
  HIP_OK(hipMemcpy(dmask, mask.data(), mask.size(), hipMemcpyHostToDevice));
  HIP_OK(hipMalloc((void**)&dcomp, C * 4));
  HIP_OK(hipMalloc((void**)&dreu, C * 4));
  HIP_OK(hipMalloc((void**)&dcnt, 2 * 4));
  const int t = 1, l = 2, diag = 3;
  DT_CHECK(dt_build_schedule(dmask, T, L, C, t, l, diag, dcomp, dreu, dcnt, stream));
  // ---- a packed batch of two segments against chunk 0, boundaries in device memory (never read on the host) ----
  const int32_t cu_q[3] = {0, 50, 64}, cu_k[3] = {0, 60, 100};      // rows 64..69 belong to no segment
  int32_t *d_cu_q, *d_cu_k;
  void* dvar_o;
  float* dvar_l;
  HIP_OK(hipMalloc((void**)&d_cu_q, sizeof cu_q));
  HIP_OK(hipMalloc((void**)&d_cu_k, sizeof cu_k));
  HIP_OK(hipMemcpy(d_cu_q, cu_q, sizeof cu_q, hipMemcpyHostToDevice));
  HIP_OK(hipMemcpy(d_cu_k, cu_k, sizeof cu_k, hipMemcpyHostToDevice));
  HIP_OK(hipMalloc(&dvar_o, state_elems * 2));
  HIP_OK(hipMalloc((void**)&dvar_l, lse_elems * 4));
  HIP_OK(hipMemset(dvar_o, 0xff, state_elems * 2));                  // NaN patterns: rows outside the segments must be zeroed
  const int32_t vjob_begin[3] = {0, 1, 2}, vjob_chunks[2] = {0, 0}, vjob_seg[2] = {0, 1};
  const int32_t* cu_kv_tab[2] = {d_cu_k, nullptr};                   // chunk 1 is not referenced
  void* vouts[2] = {dvar_o, dvar_o};
  float* vlses[2] = {dvar_l, dvar_l};
  const int32_t one_len[2] = {Sk[0], 0};
  DT_CHECK(dt_attn_varlen_jobs_fwd(dq, B, Sq, H, D, (int64_t)Sq * H * D, (int64_t)H * D, D, n_chunks, kp, vp, one_len, kv_sb,
                                   (int64_t)H * D, D, 2, vjob_begin, vjob_chunks, vjob_seg, 2, d_cu_q, cu_kv_tab, 50, vouts, vlses,
                                   0.f, 0, stream));
  DT_CHECK(dt_zero_rows_from(dvar_o, Sq, (int64_t)H * D * 2, d_cu_q + 2, stream));
  HIP_OK(hipStreamSynchronize(stream));

  // ---- checks --------------------------------------------------------------------------------------------
  std::vector<float> out(state_elems), lse(lse_elems), bo(state_elems), bl(lse_elems), cl(lse_elems);
  std::vector<uint16_t> so(state_elems);
  HIP_OK(hipMemcpy(out.data(), dout, state_elems * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(lse.data(), dlse, lse_elems * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(bo.data(), back_o, state_elems * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(bl.data(), back_l, lse_elems * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(so.data(), slot_o, state_elems * 2, hipMemcpyDeviceToHost));
  double e_out = 0, e_lse = 0, e_clse = 0;
  for (size_t i = 0; i < state_elems; ++i) e_out = std::fmax(e_out, std::fabs(out[i] - ref_out[i]));
  for (size_t i = 0; i < lse_elems; ++i) e_lse = std::fmax(e_lse, std::fabs(lse[i] - ref_lse[i]));
  for (int c = 0; c < n_chunks; ++c) {
    HIP_OK(hipMemcpy(cl.data(), dsl[c], lse_elems * 4, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < lse_elems; ++i) e_clse = std::fmax(e_clse, std::fabs(cl[i] - ref_clse[c][i]));
  }
  int bad = 0;
  for (size_t i = 0; i < state_elems; ++i) {
    if (so[i] != to_bf16(out[i])) ++bad;            // the slot holds the rounded result ...
    if (bo[i] != from_bf16(so[i])) ++bad;           // ... and the load widens it bit for bit
  }
  for (size_t i = 0; i < lse_elems; ++i)
    if (bl[i] != lse[i]) ++bad;
  std::vector<int32_t> comp(C), reu(C), cnt(2), want_comp, want_reu;
  HIP_OK(hipMemcpy(comp.data(), dcomp, C * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(reu.data(), dreu, C * 4, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(cnt.data(), dcnt, 8, hipMemcpyDeviceToHost));
  want_comp.push_back(diag);   // the diagonal chunk is always computed, first
  for (int c = 0; c < C; ++c) {
    if (c == diag) continue;
    (mask[((size_t)t * L + l) * C + c] ? want_reu : want_comp).push_back(c);
  }
  int sched_bad = (cnt[0] != (int)want_comp.size()) + (cnt[1] != (int)want_reu.size());
  for (size_t i = 0; i < want_comp.size() && i < (size_t)C; ++i) sched_bad += comp[i] != want_comp[i];
  for (size_t i = 0; i < want_reu.size() && i < (size_t)C; ++i) sched_bad += reu[i] != want_reu[i];

  // the packed batch: segment s of the queries against segment s of chunk 0's keys; zero rows behind the last boundary
  std::vector<uint16_t> vo(state_elems);
  std::vector<float> vl(lse_elems);
  HIP_OK(hipMemcpy(vo.data(), dvar_o, state_elems * 2, hipMemcpyDeviceToHost));
  HIP_OK(hipMemcpy(vl.data(), dvar_l, lse_elems * 4, hipMemcpyDeviceToHost));
  double e_var = 0, e_vlse = 0;
  int var_bad = 0;
  for (int h = 0; h < H; ++h)
    for (int sq = 0; sq < Sq; ++sq) {
      int seg = -1;
      for (int g = 0; g < 2; ++g)
        if (sq >= cu_q[g] && sq < cu_q[g + 1]) seg = g;
      if (seg < 0) {
        for (int e = 0; e < D; ++e) var_bad += vo[((size_t)sq * H + h) * D + e] != 0;
        continue;
      }
      std::vector<double> sc;
      double mx = -1e300, den = 0;
      for (int j = cu_k[seg]; j < cu_k[seg + 1]; ++j) {
        double d = 0;
        for (int e = 0; e < D; ++e) d += at(q, sq, h, e) * at(k[0], j, h, e);
        sc.push_back(d * scale);
        mx = std::fmax(mx, d * scale);
      }
      std::vector<double> o(D, 0.0);
      for (int j = cu_k[seg]; j < cu_k[seg + 1]; ++j) {
        const double p = std::exp(sc[j - cu_k[seg]] - mx);
        den += p;
        for (int e = 0; e < D; ++e) o[e] += p * at(v[0], j, h, e);
      }
      for (int e = 0; e < D; ++e) e_var = std::fmax(e_var, std::fabs(from_bf16(vo[((size_t)sq * H + h) * D + e]) - o[e] / den));
      e_vlse = std::fmax(e_vlse, std::fabs(vl[(size_t)h * Sq + sq] - (mx + std::log(den))));
    }
  std::printf("capi demo: packed batch with device-resident boundaries: out max-abs %.3e, lse max-abs %.3e, non-zero rows outside "
              "the segments %d\n", e_var, e_vlse, var_bad);

  std::printf("capi demo: version %d, out max-abs %.3e, merged lse max-abs %.3e, chunk lse max-abs %.3e, "
              "slot round trip mismatches %d, schedule mismatches %d\n",
              dt_version(), e_out, e_lse, e_clse, bad, sched_bad);
  // an invalid request comes back as an error code with a message, not as a fault
  const int rc = dt_merge_states(0, mo, ml, nullptr, nullptr, dout, DT_FP32, dlse, DT_LSE_BHS, B, Sq, H, D, stream);
  const bool err_ok = rc == DT_ERR_INVALID && std::strlen(dt_last_error()) > 0;
  if (!err_ok) std::fprintf(stderr, "expected DT_ERR_INVALID with a message for a merge of 0 states, got %d\n", rc);
  const bool ok = e_out <= 2e-2 && e_lse <= 1e-3 && e_clse <= 1e-3 && bad == 0 && sched_bad == 0 && err_ok &&
                  e_var <= 2e-2 && e_vlse <= 1e-3 && var_bad == 0;
  std::printf(ok ? "capi demo ok\n" : "capi demo FAILED\n");
  return ok ? 0 : 1;
}
