// Launchers for the channels-last InstanceNorm kernels, templated on the storage type.
#pragma once

#include "cl_kernels.hip.h"
#include "cl_single_kernels.hip.h"
#include "plan.h"
#include "status.h"

namespace atexn {

static_assert(kPlanClSingleMaxCap == kClSingleMaxCap && kPlanClSingleMaxSlabs == kClSingleMaxSlabs &&
                  kPlanClSingleMaxOwned == kClSingleMaxOwned,
              "the planner and the single-launch kernels must agree on their limits");

static_assert(kPlanClFoldRegs == 2 * kClFoldRegs, "the planner and the kernels must agree on the fold's register limit");

// Whether every register-resident slab of the plan holds exactly U pixels per pixel slot and
// every channel tile is complete (the kernels' FULL instantiations: no lane is ever masked).
inline bool cl_slabs_full(const ClPlan& p, int64_t C, int64_t D) {
  const int64_t ppb = kClThreads >> p.tpp_shift;
  return p.U > 0 && C % (int64_t(p.TPP) * p.V) == 0 && D % p.slab_len == 0 && p.slab_len == int64_t(p.U) * ppb;
}

template <typename T, int V>
int cl_fwd_v(const T* x, const float* gamma, const float* beta, int64_t N, int64_t C, int64_t D,
             float eps, T* y, float* mean, float* rstd, void* ws, size_t ws_bytes,
             hipStream_t st) {
  const ClPlan p = plan_cl(false, V, N, C, D, cu_count());
  ATEXN_REQUIRE(ws != nullptr && ws_bytes >= p.ws_bytes,
                "workspace too small: need %zu bytes, got %zu", p.ws_bytes, ws_bytes);
  float* pstat = reinterpret_cast<float*>(static_cast<char*>(ws) + p.off_a);
  float* folded = reinterpret_cast<float*>(static_cast<char*>(ws) + p.off_fold);
  const int Ci = static_cast<int>(C);
  // one workgroup column per instance: the launch's x extent N * 256 must stay below 2^32
  ATEXN_REQUIRE(N < (int64_t(1) << 24), "batch size %lld too large (channels-last limit 2^24 - 1)",
                (long long)N);
  // channel tiles of 2048 channels are the launch's z extent
  ATEXN_REQUIRE(p.CT <= 65535, "channel count %lld too large (channels-last limit 65535 * 2048)",
                (long long)C);
  const dim3 grid(static_cast<unsigned>(N), p.S, p.CT);
#define ATEXN_CL_FWD(U_, RG_, ...)                                                             \
  do {                                                                                        \
    cl_fwd_stats<T, V, U_, RG_, ##__VA_ARGS__><<<grid, kClThreads, 0, st>>>(x, pstat, D, Ci, p.S, p.tpp_shift,  \
                                                       p.slab_len);                           \
    ATEXN_CHECK_LAUNCH("cl_fwd_stats");                                                       \
    if (p.fold) {                                                                             \
      const dim3 mgrid(static_cast<unsigned>(div_up(C, kClMergeChannels)),                    \
                       static_cast<unsigned>(N));                                             \
      cl_merge_stats<<<mgrid, kClThreads, 0, st>>>(pstat, folded, D, Ci, p.S, p.slab_len);    \
      ATEXN_CHECK_LAUNCH("cl_merge_stats");                                                   \
    }                                                                                         \
    cl_fwd_apply<T, V, U_, RG_, ##__VA_ARGS__><<<grid, kClThreads, 0, st>>>(x, p.fold ? folded : pstat, gamma,  \
                                                       beta, y, mean, rstd, D, Ci,            \
                                                       p.fold ? 1 : p.S,                      \
                                                       p.fold ? D : p.slab_len, p.tpp_shift,  \
                                                       p.slab_len, eps,                       \
                                                       tuning().reverse_second_pass);         \
    ATEXN_CHECK_LAUNCH("cl_fwd_apply");                                                       \
  } while (0)
  if constexpr (V > 1) {
    if (p.fused) {
      const dim3 fgrid(static_cast<unsigned>(N), 1, p.CT);
#define ATEXN_CL_FWD_FUSED(U_)                                                                 \
  do {                                                                                        \
    if (C % V != 0)                                                                           \
      cl_fwd_fused<T, V, U_, true><<<fgrid, kClThreads, 0, st>>>(x, gamma, beta, y, mean,     \
                                                                  rstd, D, Ci, p.tpp_shift,   \
                                                                  eps);                       \
    else                                                                                      \
      cl_fwd_fused<T, V, U_, false><<<fgrid, kClThreads, 0, st>>>(x, gamma, beta, y, mean,    \
                                                                   rstd, D, Ci, p.tpp_shift,  \
                                                                   eps);                      \
  } while (0)
      switch (p.fused_u) {
        case 1: ATEXN_CL_FWD_FUSED(1); break;
        case 2: ATEXN_CL_FWD_FUSED(2); break;
        case 4: ATEXN_CL_FWD_FUSED(4); break;
        case 8: ATEXN_CL_FWD_FUSED(8); break;
        default: ATEXN_CL_FWD_FUSED(16); break;
      }
#undef ATEXN_CL_FWD_FUSED
      ATEXN_CHECK_LAUNCH("cl_fwd_fused");
      return ATEXN_OK;
    }
    if (p.single && static_cast<const void*>(y) != static_cast<const void*>(x) && exchange_allowed(st)) {
      char* w = static_cast<char*>(ws);
      cl_word* tagged = reinterpret_cast<cl_word*>(w + p.off_tagged);
      cl_word* finals = reinterpret_cast<cl_word*>(w + p.off_finals);
      unsigned* claims = reinterpret_cast<unsigned*>(w + p.off_claims);
      unsigned* trouble = exchange_trouble_word();
      const unsigned tag = next_call_tag();
      const int polls = tuning().cl_single_polls;
      const dim3 sgrid = p.single_xm ? dim3(static_cast<unsigned>(p.xm_grid), 1, 1) : grid;
      const int xm_tiles = p.single_xm ? p.CT : 0;
      // more instances than the chip holds at once: the kernel compiled for more workgroups per CU
      // (16-bit data; the float32 kernel needs fewer registers to begin with and gains nothing)
      const bool occ = p.single_xm && !p.xm_resident && sizeof(T) == 2 && tuning().cl_single_occ;
#define ATEXN_CL_FWD_SINGLE(U_, FULL_)                                                          \
  do {                                                                                          \
    auto fn = occ ? cl_fwd_single<T, V, U_, FULL_, true> : cl_fwd_single<T, V, U_, FULL_, false>; \
    fn<<<sgrid, kClThreads, 0, st>>>(x, tagged, finals, claims, gamma, beta, y, mean, rstd, N, D, Ci, p.S, \
                                     p.tpp_shift, p.slab_len, eps, tag, polls, xm_tiles, trouble); \
  } while (0)
      if (cl_slabs_full(p, C, D)) {
        if (p.U == 4) ATEXN_CL_FWD_SINGLE(4, true);
        else ATEXN_CL_FWD_SINGLE(8, true);
      } else {
        if (p.U == 4) ATEXN_CL_FWD_SINGLE(4, false);
        else ATEXN_CL_FWD_SINGLE(8, false);
      }
#undef ATEXN_CL_FWD_SINGLE
      ATEXN_CHECK_LAUNCH("cl_fwd_single");
      return ATEXN_OK;
    }
    // a channel count that is not a multiple of V: the last channel vector of a pixel overlaps
    // its neighbour and owns only its last C % V elements
    if (C % V != 0) {
      if (p.U == 4) { ATEXN_CL_FWD(4, true); return ATEXN_OK; }
      if (p.U == 8) { ATEXN_CL_FWD(8, true); return ATEXN_OK; }
      if (p.U == 16) { ATEXN_CL_FWD(16, true); return ATEXN_OK; }
      ATEXN_CL_FWD(0, true);
      return ATEXN_OK;
    }
    // every slab has exactly U pixels per slot and every channel tile is complete: no masks
    if (cl_slabs_full(p, C, D)) {
      if (p.U == 4) { ATEXN_CL_FWD(4, false, true); return ATEXN_OK; }
      if (p.U == 8) { ATEXN_CL_FWD(8, false, true); return ATEXN_OK; }
      if (p.U == 16) { ATEXN_CL_FWD(16, false, true); return ATEXN_OK; }
    }
    if (p.U == 4) { ATEXN_CL_FWD(4, false); return ATEXN_OK; }
    if (p.U == 8) { ATEXN_CL_FWD(8, false); return ATEXN_OK; }
    if (p.U == 16) { ATEXN_CL_FWD(16, false); return ATEXN_OK; }
  }
  ATEXN_CL_FWD(0, false);
#undef ATEXN_CL_FWD
  return ATEXN_OK;
}

template <typename T, int V>
int cl_bwd_v(const T* dy, const T* x, const float* gamma, const float* mean, const float* rstd,
             int64_t N, int64_t C, int64_t D, T* dx, float* dgamma, float* dbeta, void* ws,
             size_t ws_bytes, hipStream_t st) {
  const ClPlan p = plan_cl(true, V, N, C, D, cu_count());
  ATEXN_REQUIRE(ws != nullptr && ws_bytes >= p.ws_bytes,
                "workspace too small: need %zu bytes, got %zu", p.ws_bytes, ws_bytes);
  float* part = static_cast<float*>(ws);
  float* folded = reinterpret_cast<float*>(static_cast<char*>(ws) + p.off_fold);
  const int Ci = static_cast<int>(C);
  // one workgroup column per instance: the launch's x extent N * 256 must stay below 2^32
  ATEXN_REQUIRE(N < (int64_t(1) << 24), "batch size %lld too large (channels-last limit 2^24 - 1)",
                (long long)N);
  // channel tiles of 2048 channels are the launch's z extent
  ATEXN_REQUIRE(p.CT <= 65535, "channel count %lld too large (channels-last limit 65535 * 2048)",
                (long long)C);
  const dim3 grid(static_cast<unsigned>(N), p.S, p.CT);
  // how stage 2 deals the dgamma / dbeta columns to its workgroups (after the fold launch a
  // partial row per instance is left)
  const int cw_shift = cl_dparam_chunk_shift(p.fold ? N : N * p.S, 2 * C, N * p.S * p.CT);
#define ATEXN_CL_BWD(U_, RG_, ...)                                                             \
  do {                                                                                        \
    cl_bwd_sums<T, V, U_, RG_, ##__VA_ARGS__><<<grid, kClThreads, 0, st>>>(dy, x, mean, rstd, part, D, Ci, p.S, \
                                                      p.tpp_shift, p.slab_len);               \
    ATEXN_CHECK_LAUNCH("cl_bwd_sums");                                                        \
    if (p.fold) {                                                                             \
      const int rc = launch_col_reduce(part, folded, folded + C, p.S, C, st,                  \
                                       static_cast<int>(N), int64_t(p.S) * 2 * C, 2 * C);     \
      if (rc != ATEXN_OK) return rc;                                                          \
    }                                                                                         \
    cl_bwd_apply<T, V, U_, RG_, ##__VA_ARGS__><<<grid, kClThreads, 0, st>>>(dy, x, gamma, mean, rstd,           \
                                                       p.fold ? folded : part, dx,            \
                                                       dgamma, dbeta, N, D, Ci,               \
                                                       p.fold ? 1 : p.S,                      \
                                                       p.tpp_shift, p.slab_len,               \
                                                       tuning().reverse_second_pass,          \
                                                       cw_shift);                             \
    ATEXN_CHECK_LAUNCH("cl_bwd_apply");                                                       \
  } while (0)
  if constexpr (V > 1) {
    if (p.fused) {
      const dim3 fgrid(static_cast<unsigned>(N), 1, p.CT);
      // a single instance: its sums are dgamma / dbeta; else per-instance rows for col_reduce
      float* o0 = N == 1 ? dgamma : part;
      float* o1 = N == 1 ? dbeta : part + C;
      const int64_t stride = N == 1 ? 0 : 2 * C;
#define ATEXN_CL_BWD_FUSED(U_)                                                                 \
  do {                                                                                        \
    if (C % V != 0)                                                                           \
      cl_bwd_fused<T, V, U_, true><<<fgrid, kClThreads, 0, st>>>(dy, x, gamma, mean, rstd,    \
                                                                  dx, o0, o1, stride, D, Ci,  \
                                                                  p.tpp_shift);               \
    else                                                                                      \
      cl_bwd_fused<T, V, U_, false><<<fgrid, kClThreads, 0, st>>>(dy, x, gamma, mean, rstd,   \
                                                                   dx, o0, o1, stride, D, Ci, \
                                                                   p.tpp_shift);              \
  } while (0)
      switch (p.fused_u) {
        case 1: ATEXN_CL_BWD_FUSED(1); break;
        case 2: ATEXN_CL_BWD_FUSED(2); break;
        case 4: ATEXN_CL_BWD_FUSED(4); break;
        default: ATEXN_CL_BWD_FUSED(8); break;
      }
#undef ATEXN_CL_BWD_FUSED
      ATEXN_CHECK_LAUNCH("cl_bwd_fused");
      if (N > 1) return launch_col_reduce(part, dgamma, dbeta, static_cast<int>(N), C, st);
      return ATEXN_OK;
    }
    if (p.single && static_cast<const void*>(dx) != static_cast<const void*>(dy) && exchange_allowed(st)) {
      char* w = static_cast<char*>(ws);
      cl_word* tagged = reinterpret_cast<cl_word*>(w + p.off_tagged);
      cl_word* finals = reinterpret_cast<cl_word*>(w + p.off_finals);
      cl_word* finals_dev = reinterpret_cast<cl_word*>(w + p.off_finals_dev);
      unsigned* claims = reinterpret_cast<unsigned*>(w + p.off_claims);
      unsigned* trouble = exchange_trouble_word();
      const unsigned tag = next_call_tag();
      const int polls = tuning().cl_single_polls;
      const int Ni = static_cast<int>(N);
      // XCD-major grid: no fold over the instances in the kernel; a single instance's sums are
      // dgamma / dbeta, else per-instance rows for col_reduce
      const dim3 sgrid = p.single_xm ? dim3(static_cast<unsigned>(p.xm_grid), 1, 1) : grid;
      const int xm_tiles = p.single_xm ? p.CT : 0;
      float* xpart = reinterpret_cast<float*>(w + p.off_xm_part);
      float* o0 = N == 1 ? dgamma : xpart;
      float* o1 = N == 1 ? dbeta : xpart + C;
      const int64_t o_stride = N == 1 ? 0 : 2 * C;
      if (p.single_xm && !p.xm_fold) finals_dev = nullptr;
      // (the backward, which runs three workgroups per CU as it is, only with more than 32 slabs
      // per instance and more than two instances per XCD: [64, 128^2, 64] fp16 94 -> 87 us; with
      // fewer slabs it loses, [128, 64^2, 64] 44.0 -> 46.8 us, [32, 128^2, 32] 23.1 -> 23.8 us, and
      // with two instances per XCD the step does, [16, 128^2, 64] 39.1 -> 40.2 us)
      const bool occ = p.single_xm && !p.xm_resident && p.S > 32 && static_cast<int64_t>(Ni) * p.CT > 16 &&
                       tuning().cl_single_occ;
#define ATEXN_CL_BWD_SINGLE(U_, FULL_)                                                          \
  do {                                                                                          \
    /* (ragged slabs keep the plain build: under the bound of 128 registers theirs spills 96) */ \
    auto fn = occ ? cl_bwd_single<T, V, U_, FULL_, FULL_> : cl_bwd_single<T, V, U_, FULL_, false>; \
    fn<<<sgrid, kClThreads, 0, st>>>(dy, x, gamma, mean, rstd, tagged, finals, finals_dev, claims, dx, dgamma, \
                                     dbeta, Ni, D, Ci, p.S, p.tpp_shift, p.slab_len, tag, polls, \
                                     xm_tiles, o0, o1, o_stride, trouble);             \
  } while (0)
      if (cl_slabs_full(p, C, D)) {
        if (p.U == 4) ATEXN_CL_BWD_SINGLE(4, true);
        else ATEXN_CL_BWD_SINGLE(8, true);
      } else {
        if (p.U == 4) ATEXN_CL_BWD_SINGLE(4, false);
        else ATEXN_CL_BWD_SINGLE(8, false);
      }
#undef ATEXN_CL_BWD_SINGLE
      ATEXN_CHECK_LAUNCH("cl_bwd_single");
      if (p.single_xm && !p.xm_fold && N > 1) return launch_col_reduce(xpart, dgamma, dbeta, static_cast<int>(N), C, st);
      return ATEXN_OK;
    }
    if (C % V != 0) {
      if (p.U == 4) { ATEXN_CL_BWD(4, true); return ATEXN_OK; }
      if (p.U == 8) { ATEXN_CL_BWD(8, true); return ATEXN_OK; }
      ATEXN_CL_BWD(0, true);
      return ATEXN_OK;
    }
    if (cl_slabs_full(p, C, D)) {
      if (p.U == 4) { ATEXN_CL_BWD(4, false, true); return ATEXN_OK; }
      if (p.U == 8) { ATEXN_CL_BWD(8, false, true); return ATEXN_OK; }
    }
    if (p.U == 4) { ATEXN_CL_BWD(4, false); return ATEXN_OK; }
    if (p.U == 8) { ATEXN_CL_BWD(8, false); return ATEXN_OK; }
  }
  ATEXN_CL_BWD(0, false);
#undef ATEXN_CL_BWD
  return ATEXN_OK;
}

template <typename T>
int cl_fwd_t(const void* x_, const float* gamma, const float* beta, int64_t N, int64_t C,
             int64_t D, float eps, void* y_, float* mean, float* rstd, void* ws, size_t ws_bytes,
             hipStream_t st) {
  constexpr int VEC = VecOf<T>::value;
  const T* x = static_cast<const T*>(x_);
  T* y = static_cast<T*>(y_);
  // 16-byte accesses work at element alignment; a C that is not a multiple of the vector
  // width is covered by an overlapping last vector
  const bool vec = C >= VEC;
  return vec ? cl_fwd_v<T, VEC>(x, gamma, beta, N, C, D, eps, y, mean, rstd, ws, ws_bytes, st)
             : cl_fwd_v<T, 1>(x, gamma, beta, N, C, D, eps, y, mean, rstd, ws, ws_bytes, st);
}

template <typename T>
int cl_bwd_t(const void* dy_, const void* x_, const float* gamma, const float* mean,
             const float* rstd, int64_t N, int64_t C, int64_t D, void* dx_, float* dgamma,
             float* dbeta, void* ws, size_t ws_bytes, hipStream_t st) {
  constexpr int VEC = VecOf<T>::value;
  const T* x = static_cast<const T*>(x_);
  const T* dy = static_cast<const T*>(dy_);
  T* dx = static_cast<T*>(dx_);
  const bool vec = C >= VEC;
  return vec ? cl_bwd_v<T, VEC>(dy, x, gamma, mean, rstd, N, C, D, dx, dgamma, dbeta, ws, ws_bytes, st)
             : cl_bwd_v<T, 1>(dy, x, gamma, mean, rstd, N, C, D, dx, dgamma, dbeta, ws, ws_bytes, st);
}

#define ATEXN_INSTANTIATE_CL(T)                                                                  \
  template int cl_fwd_t<T>(const void*, const float*, const float*, int64_t, int64_t, int64_t,   \
                           float, void*, float*, float*, void*, size_t, hipStream_t);            \
  template int cl_bwd_t<T>(const void*, const void*, const float*, const float*, const float*,   \
                           int64_t, int64_t, int64_t, void*, float*, float*, void*, size_t,      \
                           hipStream_t);

}  // namespace atexn
