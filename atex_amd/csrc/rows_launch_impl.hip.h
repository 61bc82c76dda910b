// Launchers for the contiguous-row kernels, templated on the storage type; one
// translation unit per dtype instantiates them (rows_launch_*.hip).
#pragma once

#include "plan.h"
#include "rows_kernels.hip.h"
#include "plane_single_kernels.hip.h"
#include "small_kernels.hip.h"
#include "tiles_kernels.hip.h"

#include <atomic>
#include "status.h"

namespace atexn {

static_assert(kAffineFoldMaxStep == kPlanAffineFoldMaxStep && kAffineFoldMaxPairs == kPlanAffineFoldMaxPairs,
              "the planner admits the in-kernel batch fold with the kernels' limits");
static_assert(kFoldLdsBytes == kPlanFoldLdsBytes && kFoldMaxWaves == kPlanFoldMaxWaves,
              "the planner sizes the fold's LDS with the kernels' constants");

template <typename T, int V, bool AFF>
using FwdResidentFn = void (*)(const T*, const float*, const float*, T*, float*, float*, int64_t,
                               int, int, float);
template <typename T, int V, bool AFF>
using BwdResidentFn = void (*)(const T*, const T*, const float*, const float*, const float*, T*,
                               float*, int64_t, int, int, AffineFold);

// Row batching (RB > 1) exists for the vector path and rows of at most one wave; the
// predicate-free EXACT variants exist for the vector path.
// The kernels that keep a row (or its accumulators) in LDS ask for more dynamic LDS than a
// launch gets by default: the limit is raised once per kernel and device.
template <auto Kernel>
inline hipError_t allow_large_lds() {
  static std::atomic<uint64_t> done{0};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    dev = -1;
  }
  if (dev >= 0 && ((done.load(std::memory_order_acquire) >> dev) & 1)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(kPlanLdsBytes - kPlanBwdLdsReserve));
  if (e == hipSuccess && dev >= 0) done.fetch_or(uint64_t(1) << dev, std::memory_order_release);
  if (e != hipSuccess) (void)hipGetLastError();
  return e;
}

template <typename T, int V, int TPR, int VPT, bool AFF>
FwdResidentFn<T, V, AFF> fwd_variant(int rb, bool exact, bool ragged) {
  if constexpr (V > 1) {
    if (ragged) {
      // short ragged rows (one vector per lane) keep their row batching
      if constexpr (TPR != 0 && TPR <= 64 && VPT == 1) {
        if (rb == 2) return rows_fwd_resident<T, V, TPR, VPT, 2, false, AFF, true>;
        if (rb == 4) return rows_fwd_resident<T, V, TPR, VPT, 4, false, AFF, true>;
      }
      return rb == 1 ? rows_fwd_resident<T, V, TPR, VPT, 1, false, AFF, true> : nullptr;
    }
    if constexpr (TPR != 0) {
      if (rb == 2) return exact ? rows_fwd_resident<T, V, TPR, VPT, 2, true, AFF> : rows_fwd_resident<T, V, TPR, VPT, 2, false, AFF>;
      if (rb == 4) return exact ? rows_fwd_resident<T, V, TPR, VPT, 4, true, AFF> : rows_fwd_resident<T, V, TPR, VPT, 4, false, AFF>;
    }
    if (rb == 1 && exact) return rows_fwd_resident<T, V, TPR, VPT, 1, true, AFF>;
  }
  return rb == 1 ? rows_fwd_resident<T, V, TPR, VPT, 1, false, AFF> : nullptr;
}
template <typename T, int V, int TPR, int VPT, bool AFF>
BwdResidentFn<T, V, AFF> bwd_variant(int rb, bool exact, bool ragged) {
  if constexpr (V > 1) {
    if (ragged) {
      if constexpr (TPR != 0 && TPR <= 64 && VPT == 1) {
        if (rb == 2) return rows_bwd_resident<T, V, TPR, VPT, 2, false, AFF, true>;
      }
      return rb == 1 ? rows_bwd_resident<T, V, TPR, VPT, 1, false, AFF, true> : nullptr;
    }
    // (the planner batches backward rows only with one vector per lane: with two or three the
    // batched kernels need more than 256 registers)
    if constexpr (TPR != 0 && TPR <= 64 && VPT == 1) {
      if (rb == 2) return exact ? rows_bwd_resident<T, V, TPR, VPT, 2, true, AFF> : rows_bwd_resident<T, V, TPR, VPT, 2, false, AFF>;
    }
    if (rb == 1 && exact) return rows_bwd_resident<T, V, TPR, VPT, 1, true, AFF>;
  }
  return rb == 1 ? rows_bwd_resident<T, V, TPR, VPT, 1, false, AFF> : nullptr;
}

template <typename T, int V, bool AFF>
FwdResidentFn<T, V, AFF> pick_fwd_resident(int tpr, int vpt, int rb, bool exact, bool ragged) {
  // element-wise rows are only the ones shorter than a vector
  if constexpr (V == 1) {
    return tpr == 8 && vpt == 1 ? fwd_variant<T, V, 8, 1, AFF>(rb, exact, false) : nullptr;
  } else {
  if (vpt == 3) {
    if (tpr == 8) return fwd_variant<T, V, 8, 3, AFF>(rb, exact, ragged);
    if (tpr == 16) return fwd_variant<T, V, 16, 3, AFF>(rb, exact, ragged);
    if (tpr == 32) return fwd_variant<T, V, 32, 3, AFF>(rb, exact, ragged);
    if (tpr == 64) return fwd_variant<T, V, 64, 3, AFF>(rb, exact, ragged);
    return nullptr;
  }
  if (tpr == 8) return fwd_variant<T, V, 8, 1, AFF>(rb, exact, ragged);
  if (tpr == 16) return fwd_variant<T, V, 16, 1, AFF>(rb, exact, ragged);
  if (tpr == 32) return fwd_variant<T, V, 32, 1, AFF>(rb, exact, ragged);
  if (tpr == 64 && vpt == 1) return fwd_variant<T, V, 64, 1, AFF>(rb, exact, ragged);
  if (tpr == 64 && vpt == 2) return fwd_variant<T, V, 64, 2, AFF>(rb, exact, ragged);
  if (tpr == 0 && vpt == 2) return fwd_variant<T, V, 0, 2, AFF>(rb, exact, ragged);
  if (tpr == 0 && vpt == 4) return fwd_variant<T, V, 0, 4, AFF>(rb, exact, ragged);
  if (tpr == 0 && vpt == 8) return fwd_variant<T, V, 0, 8, AFF>(rb, exact, ragged);
  return nullptr;
  }
}

template <typename T, int V, bool AFF>
BwdResidentFn<T, V, AFF> pick_bwd_resident(int tpr, int vpt, int rb, bool exact, bool ragged) {
  if constexpr (V == 1) {
    return tpr == 8 && vpt == 1 ? bwd_variant<T, V, 8, 1, AFF>(rb, exact, false) : nullptr;
  } else {
  if (vpt == 3) {
    if (tpr == 8) return bwd_variant<T, V, 8, 3, AFF>(rb, exact, ragged);
    if (tpr == 16) return bwd_variant<T, V, 16, 3, AFF>(rb, exact, ragged);
    if (tpr == 32) return bwd_variant<T, V, 32, 3, AFF>(rb, exact, ragged);
    if (tpr == 64) return bwd_variant<T, V, 64, 3, AFF>(rb, exact, ragged);
    if constexpr (!AFF) {
      if (tpr == 128) return bwd_variant<T, V, 128, 3, AFF>(1, exact, ragged);
    }
    return nullptr;
  }
  if (tpr == 8) return bwd_variant<T, V, 8, 1, AFF>(rb, exact, ragged);
  if (tpr == 16) return bwd_variant<T, V, 16, 1, AFF>(rb, exact, ragged);
  if (tpr == 32) return bwd_variant<T, V, 32, 1, AFF>(rb, exact, ragged);
  if (tpr == 64 && vpt == 1) return bwd_variant<T, V, 64, 1, AFF>(rb, exact, ragged);
  if (tpr == 64 && vpt == 2) return bwd_variant<T, V, 64, 2, AFF>(rb, exact, ragged);
  if constexpr (!AFF) {  // LayerNorm: rows held by 2 or 4 waves of a 512-thread block
    if (tpr == 128 && vpt == 2) return bwd_variant<T, V, 128, 2, AFF>(1, exact, ragged);
    if (tpr == 256 && vpt == 2) return bwd_variant<T, V, 256, 2, AFF>(1, exact, ragged);
  }
  if (tpr == 0 && vpt == 2) return bwd_variant<T, V, 0, 2, AFF>(rb, exact, ragged);
  if (tpr == 0 && vpt == 4) return bwd_variant<T, V, 0, 4, AFF>(rb, exact, ragged);
  if constexpr (AFF) {
    if (tpr == 0 && vpt == 8) return bwd_variant<T, V, 0, 8, AFF>(rb, exact, ragged);
  }
  return nullptr;
  }
}

template <typename T, int V, bool AFF>
int rows_fwd_v(const T* x, const float* gamma, const float* beta, int64_t n_rows, int64_t D,
               int C, float eps, T* y, float* mean, float* rstd, void* ws, size_t ws_bytes,
               hipStream_t st) {
  const RowsPlan p = plan_rows(RowsKind::kFwd, V, n_rows, D, AFF ? C : 0, cu_count());
  ATEXN_REQUIRE(ws_bytes >= p.ws_bytes && (p.ws_bytes == 0 || ws != nullptr),
                "workspace too small: need %zu bytes, got %zu", p.ws_bytes, ws_bytes);
  if (p.resident) {
    auto fn = pick_fwd_resident<T, V, AFF>(p.tpr, p.vpt, p.rb, p.exact, p.ragged);
    if (!fn) return set_error(ATEXN_LAUNCH_ERROR, "no resident forward kernel for tpr=%d vpt=%d", p.tpr, p.vpt);
    fn<<<p.grid, p.threads, 0, st>>>(x, gamma, beta, y, mean, rstd, n_rows, static_cast<int>(D), C,
                                     eps);
    ATEXN_CHECK_LAUNCH("rows_fwd_resident");
    return ATEXN_OK;
  }
  if constexpr (AFF && V > 1) {
    if (p.plane_single && static_cast<const void*>(y) != static_cast<const void*>(x) && exchange_allowed(st)) {
      static_assert(kPlaneThreads == kPlanPlaneThreads && kPlaneMaxChunks == kPlanPlaneMaxChunks && kPlaneXcds == kPlanXcdCount,
                    "plan_rows sizes the plane_*_single launches");
      cl_word* tagged = reinterpret_cast<cl_word*>(static_cast<char*>(ws) + p.off_ps_tagged);
      const int n_vec = static_cast<int>(D / V);
      const bool nt = n_rows * D * int64_t(sizeof(T)) >= int64_t(tuning().plane_nt_min_mb) << 20;
      auto fn = p.ps_full ? (nt ? plane_fwd_single<T, V, kPlanPlaneVpt, true, true> : plane_fwd_single<T, V, kPlanPlaneVpt, true, false>)
                          : (nt ? plane_fwd_single<T, V, kPlanPlaneVpt, false, true> : plane_fwd_single<T, V, kPlanPlaneVpt, false, false>);
      unsigned* claims = reinterpret_cast<unsigned*>(static_cast<char*>(ws) + p.off_ps_claims);
      fn<<<p.ps_grid, kPlaneThreads, 0, st>>>(x, tagged, claims, gamma, beta, y, mean, rstd, n_rows, n_vec, p.ps_S,
                                              p.ps_chunk_vec, C, eps, next_call_tag(), tuning().plane_single_polls,
                                              exchange_trouble_word());
      ATEXN_CHECK_LAUNCH("plane_fwd_single");
      return ATEXN_OK;
    }
  }
  if constexpr (AFF && V > 1) {
    if (p.staged) {
      static_assert(kStagedThreads == kPlanStagedThreads && kStagedRegVec == kPlanStagedRegVec, "plan_rows sizes the staged launches");
      const bool lds_ok = allow_large_lds<rows_fwd_staged<T, V>>() == hipSuccess;
      ATEXN_REQUIRE(lds_ok, "this device does not give a workgroup %zu bytes of LDS", kPlanLdsBytes - kPlanBwdLdsReserve);
      rows_fwd_staged<T, V><<<p.grid, p.threads, p.fold_lds, st>>>(x, gamma, beta, y, mean, rstd, n_rows,
                                                                        static_cast<int>(D), C, eps, p.nv_lds);
      ATEXN_CHECK_LAUNCH("rows_fwd_staged");
      return ATEXN_OK;
    }
  }
  if constexpr (AFF && V > 1) {
    float2* stats = reinterpret_cast<float2*>(static_cast<char*>(ws) + p.off_pairs);
    split_fwd_stats<T, V><<<p.split_grid, kSplitThreads, 0, st>>>(x, stats, n_rows, D, p.S, p.chunk);
    ATEXN_CHECK_LAUNCH("split_fwd_stats");
    split_fwd_apply<T, V, true><<<p.split_grid, kSplitThreads, 0, st>>>(x, stats, gamma, beta, y, mean, rstd,
                                                             n_rows, D, p.S, p.chunk, C, eps,
                                                             tuning().reverse_second_pass);
    ATEXN_CHECK_LAUNCH("split_fwd_apply");
    return ATEXN_OK;
  } else {
    return set_error(ATEXN_LAUNCH_ERROR, "rows of %lld elements have no split kernel on this path", (long long)D);
  }
}

// Many rows of at most four vectors: one thread per row (small_kernels.hip.h).
template <typename T, bool AFF>
int small_fwd_launch(const T* x, const float* gamma, const float* beta, int64_t n_rows, int64_t D,
                     int C, float eps, T* y, float* mean, float* rstd, hipStream_t st) {
  constexpr int V = VecOf<T>::value;
  const SmallPlan p = plan_small(RowsKind::kFwd, V, n_rows, D, C, cu_count());
  const int Di = static_cast<int>(D);
  switch (p.NV) {
    case 1: small_fwd<T, V, 1, AFF><<<p.grid, kSmallThreads, 0, st>>>(x, gamma, beta, y, mean, rstd, n_rows, Di, C, eps); break;
    case 2: small_fwd<T, V, 2, AFF><<<p.grid, kSmallThreads, 0, st>>>(x, gamma, beta, y, mean, rstd, n_rows, Di, C, eps); break;
    case 3: small_fwd<T, V, 3, AFF><<<p.grid, kSmallThreads, 0, st>>>(x, gamma, beta, y, mean, rstd, n_rows, Di, C, eps); break;
    default: small_fwd<T, V, 4, AFF><<<p.grid, kSmallThreads, 0, st>>>(x, gamma, beta, y, mean, rstd, n_rows, Di, C, eps); break;
  }
  ATEXN_CHECK_LAUNCH("small_fwd");
  return ATEXN_OK;
}

template <typename T, bool AFF>
int small_bwd_launch(const T* dy, const T* x, const float* gamma, const float* mean,
                     const float* rstd, int64_t n_rows, int64_t D, int C, T* dx, float* dgamma,
                     float* dbeta, void* ws, size_t ws_bytes, hipStream_t st) {
  constexpr int V = VecOf<T>::value;
  const SmallPlan p = plan_small(AFF ? RowsKind::kBwdAffine : RowsKind::kBwdCols, V, n_rows, D, C, cu_count());
  ATEXN_REQUIRE(ws_bytes >= p.ws_bytes && ws != nullptr,
                "workspace too small: need %zu bytes, got %zu", p.ws_bytes, ws_bytes);
  float* part = static_cast<float*>(ws);
  const int Di = static_cast<int>(D);
  if (bwd_stage_mask() & 1) {
    switch (p.NV) {
      case 1: small_bwd<T, V, 1, AFF><<<p.grid, kSmallThreads, 0, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di, C); break;
      case 2: small_bwd<T, V, 2, AFF><<<p.grid, kSmallThreads, 0, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di, C); break;
      case 3: small_bwd<T, V, 3, AFF><<<p.grid, kSmallThreads, 0, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di, C); break;
      default: small_bwd<T, V, 4, AFF><<<p.grid, kSmallThreads, 0, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di, C); break;
    }
    ATEXN_CHECK_LAUNCH("small_bwd");
  }
  if (!(bwd_stage_mask() & 2)) return ATEXN_OK;
  return launch_col_reduce(part, dgamma, dbeta, p.part_rows, AFF ? C : D, st);
}

// LayerNorm rows too long for registers, any D and alignment (tiles_kernels.hip.h).
template <typename T>
int tiles_fwd(const T* x, const float* gamma, const float* beta, int64_t n_rows, int64_t D,
              float eps, T* y, float* mean, float* rstd, void* ws, size_t ws_bytes,
              hipStream_t st) {
  constexpr int V = VecOf<T>::value;
  const TilePlan p = plan_tiles(false, V, n_rows, D, cu_count());
  ATEXN_REQUIRE(ws_bytes >= p.ws_bytes && ws != nullptr,
                "workspace too small: need %zu bytes, got %zu", p.ws_bytes, ws_bytes);
  float2* stats = reinterpret_cast<float2*>(static_cast<char*>(ws) + p.off_pairs);
  split_fwd_stats<T, V><<<p.stats_grid, kSplitThreads, 0, st>>>(x, stats, n_rows, D, p.S, p.chunk);
  ATEXN_CHECK_LAUNCH("split_fwd_stats");
  merge_row_stats<4><<<static_cast<unsigned>(div_up(n_rows, 4)), 256, 0, st>>>(stats, mean, rstd, n_rows,
                                                                        D, p.S, p.chunk, eps);
  ATEXN_CHECK_LAUNCH("merge_row_stats");
  const dim3 grid(p.CT, p.RS);
  tile_fwd_apply<T, V><<<grid, kTileThreads, 0, st>>>(x, gamma, beta, mean, rstd, y, n_rows, D, p.R,
                                                     tuning().reverse_second_pass);
  ATEXN_CHECK_LAUNCH("tile_fwd_apply");
  return ATEXN_OK;
}

template <typename T>
int tiles_bwd(const T* dy, const T* x, const float* gamma, const float* mean, const float* rstd,
              int64_t n_rows, int64_t D, T* dx, float* dgamma, float* dbeta, void* ws,
              size_t ws_bytes, hipStream_t st) {
  constexpr int V = VecOf<T>::value;
  const TilePlan p = plan_tiles(true, V, n_rows, D, cu_count());
  ATEXN_REQUIRE(ws_bytes >= p.ws_bytes && ws != nullptr,
                "workspace too small: need %zu bytes, got %zu", p.ws_bytes, ws_bytes);
  char* base = static_cast<char*>(ws);
  float2* sums = reinterpret_cast<float2*>(base + p.off_pairs);
  float2* rowsum = reinterpret_cast<float2*>(base + p.off_rowsum);
  float* part = reinterpret_cast<float*>(base + p.off_part);
  const dim3 grid(p.CT, p.RS);
  const dim3 sgrid(p.sums_CT, p.sums_RS);
  const bool direct = p.sums_RS == 1;  // one row slab: the column sums are final
  float* og = direct ? dgamma : part;
  float* ob = direct ? dbeta : part + D;
  const int64_t sstride = direct ? 0 : 2 * D;
  switch (p.sums_vpt) {
    case 4: tile_bwd_sums<T, V, 4><<<sgrid, kTileThreads, 0, st>>>(dy, x, gamma, mean, rstd, sums, og, ob, sstride, n_rows, D, p.sums_R); break;
    case 2: tile_bwd_sums<T, V, 2><<<sgrid, kTileThreads, 0, st>>>(dy, x, gamma, mean, rstd, sums, og, ob, sstride, n_rows, D, p.sums_R); break;
    default: tile_bwd_sums<T, V, 1><<<sgrid, kTileThreads, 0, st>>>(dy, x, gamma, mean, rstd, sums, og, ob, sstride, n_rows, D, p.sums_R); break;
  }
  ATEXN_CHECK_LAUNCH("tile_bwd_sums");
  merge_row_sums<4><<<static_cast<unsigned>(div_up(n_rows, 4)), 256, 0, st>>>(sums, rowsum, n_rows, p.sums_CT);
  ATEXN_CHECK_LAUNCH("merge_row_sums");
  tile_bwd_apply<T, V><<<grid, kTileThreads, 0, st>>>(dy, x, gamma, mean, rstd, rowsum, dx, n_rows,
                                                     D, p.R, tuning().reverse_second_pass);
  ATEXN_CHECK_LAUNCH("tile_bwd_apply");
  if (direct) return ATEXN_OK;
  return launch_col_reduce(part, dgamma, dbeta, p.sums_RS, D, st);
}

template <typename T, int V, bool AFF>
int rows_bwd_v(const T* dy, const T* x, const float* gamma, const float* mean, const float* rstd,
               int64_t n_rows, int64_t D, int C, T* dx, float* dgamma, float* dbeta, void* ws,
               size_t ws_bytes, hipStream_t st) {
  const RowsPlan p =
      plan_rows(AFF ? RowsKind::kBwdAffine : RowsKind::kBwdCols, V, n_rows, D, AFF ? C : 0, cu_count());
  ATEXN_REQUIRE(ws_bytes >= p.ws_bytes && ws != nullptr,
                "workspace too small: need %zu bytes, got %zu", p.ws_bytes, ws_bytes);
  float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + p.off_part);
  const int64_t W = AFF ? C : D;
  if constexpr (!AFF && V > 1) {
    if (p.acc_lds) {
      const bool lds_ok = allow_large_lds<rows_bwd_lds<T, V, false>>() == hipSuccess &&
                          allow_large_lds<rows_bwd_lds<T, V, true>>() == hipSuccess;
      ATEXN_REQUIRE(lds_ok, "this device does not give a workgroup %zu bytes of LDS", kPlanLdsBytes - kPlanBwdLdsReserve);
      static_assert(kBwdLdsThreads == 512 && kBwdLdsVpt == 8, "plan_rows sizes rows_bwd_lds launches");
      const int stages = bwd_stage_mask();
      if (stages & 1) {
        const int Di = static_cast<int>(D);
        if (p.vpt == 4) {
          (void)allow_large_lds<rows_bwd_lds<T, V, false, 4>>();
          (void)allow_large_lds<rows_bwd_lds<T, V, true, 4>>();
          if (p.ragged) rows_bwd_lds<T, V, true, 4><<<p.grid, p.threads, p.fold_lds, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di);
          else rows_bwd_lds<T, V, false, 4><<<p.grid, p.threads, p.fold_lds, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di);
        } else if (p.ragged) {
          rows_bwd_lds<T, V, true><<<p.grid, p.threads, p.fold_lds, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di);
        } else {
          rows_bwd_lds<T, V, false><<<p.grid, p.threads, p.fold_lds, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows, Di);
        }
        ATEXN_CHECK_LAUNCH("rows_bwd_lds");
      }
      if (!(stages & 2)) return ATEXN_OK;
      return launch_col_reduce(part, dgamma, dbeta, p.part_rows, W, st);
    }
  }
  if (p.resident) {
    auto fn = pick_bwd_resident<T, V, AFF>(p.tpr, p.vpt, p.rb, p.exact, p.ragged);
    if (!fn) return set_error(ATEXN_LAUNCH_ERROR, "no resident backward kernel for tpr=%d vpt=%d", p.tpr, p.vpt);
    AffineFold fold;
    if (AFF && p.affine_fold && static_cast<const void*>(dx) != static_cast<const void*>(dy) &&
        exchange_allowed(st)) {
      // the plane sums are folded over the batch inside the row kernel: no col_reduce
      fold.tagged = reinterpret_cast<cl_word*>(static_cast<char*>(ws) + p.off_tagged);
      fold.dgamma = dgamma;
      fold.dbeta = dbeta;
      fold.tag = next_call_tag();
      fold.max_polls = tuning().affine_fold_polls;
      fold.N = p.part_rows;
      fn<<<p.grid, p.threads, p.fold_lds, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows,
                                                static_cast<int>(D), C, fold);
      ATEXN_CHECK_LAUNCH("rows_bwd_resident");
      return ATEXN_OK;
    }
    const int stages = bwd_stage_mask();
    if (stages & 1) {
      fn<<<p.grid, p.threads, p.fold_lds, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows,
                                                static_cast<int>(D), C, fold);
      ATEXN_CHECK_LAUNCH("rows_bwd_resident");
    }
    if (!(stages & 2)) return ATEXN_OK;
    return launch_col_reduce(part, dgamma, dbeta, p.part_rows, W, st);
  }
  if constexpr (AFF && V > 1) {
    if (p.plane_single && static_cast<const void*>(dx) != static_cast<const void*>(dy) && exchange_allowed(st)) {
      cl_word* tagged = reinterpret_cast<cl_word*>(static_cast<char*>(ws) + p.off_ps_tagged);
      const int n_vec = static_cast<int>(D / V);
      // (three workgroups per CU when the two of an XCD's CUs would all hold chunks of one plane)
      const bool occ = p.ps_full && tuning().plane_single_occ && p.ps_S > 32;
      auto fn = occ         ? plane_bwd_single<T, V, kPlanPlaneVpt, true, true>
                : p.ps_full ? plane_bwd_single<T, V, kPlanPlaneVpt, true, false>
                            : plane_bwd_single<T, V, kPlanPlaneVpt, false, false>;
      PlaneFold pf{nullptr, dgamma, dbeta, p.part_rows};
      if (p.ps_fold) pf.tagged = reinterpret_cast<cl_word*>(static_cast<char*>(ws) + p.off_ps_fold);
      unsigned* claims = reinterpret_cast<unsigned*>(static_cast<char*>(ws) + p.off_ps_claims);
      fn<<<p.ps_grid, kPlaneThreads, 0, st>>>(dy, x, gamma, mean, rstd, tagged, claims, dx, part, n_rows, n_vec, p.ps_S,
                                              p.ps_chunk_vec, C, next_call_tag(), tuning().plane_single_polls, pf,
                                              exchange_trouble_word());
      ATEXN_CHECK_LAUNCH("plane_bwd_single");
      if (p.ps_fold) return ATEXN_OK;
      return launch_col_reduce(part, dgamma, dbeta, p.part_rows, W, st);
    }
  }
  if constexpr (AFF && V > 1) {
    if (p.staged) {
      const bool lds_ok = allow_large_lds<rows_bwd_staged<T, V>>() == hipSuccess;
      ATEXN_REQUIRE(lds_ok, "this device does not give a workgroup %zu bytes of LDS", kPlanLdsBytes - kPlanBwdLdsReserve);
      if (bwd_stage_mask() & 1) {
        rows_bwd_staged<T, V><<<p.grid, p.threads, p.fold_lds, st>>>(dy, x, gamma, mean, rstd, dx, part, n_rows,
                                                                     static_cast<int>(D), C, p.nv_lds);
        ATEXN_CHECK_LAUNCH("rows_bwd_staged");
      }
      if (!(bwd_stage_mask() & 2)) return ATEXN_OK;
      return launch_col_reduce(part, dgamma, dbeta, p.part_rows, W, st);
    }
    float2* sums = reinterpret_cast<float2*>(static_cast<char*>(ws) + p.off_pairs);
    split_bwd_sums<T, V, true><<<p.split_grid, kSplitThreads, 0, st>>>(dy, x, gamma, mean, rstd, sums, n_rows,
                                                            D, p.S, p.chunk);
    ATEXN_CHECK_LAUNCH("split_bwd_sums");
    split_bwd_apply<T, V, true><<<p.split_grid, kSplitThreads, 0, st>>>(dy, x, gamma, mean, rstd, sums, dx,
                                                             part, n_rows, D, p.S, p.chunk, C,
                                                             tuning().reverse_second_pass);
    ATEXN_CHECK_LAUNCH("split_bwd_apply");
    return launch_col_reduce(part, dgamma, dbeta, p.part_rows, W, st);
  } else {
    return set_error(ATEXN_LAUNCH_ERROR, "rows of %lld elements have no split kernel on this path", (long long)D);
  }
}

template <typename T>
int rows_fwd_t(bool affine, const void* x_, const float* gamma, const float* beta, int64_t n_rows,
               int64_t D, int C, float eps, void* y_, float* mean, float* rstd, void* ws,
               size_t ws_bytes, hipStream_t st) {
  constexpr int VEC = VecOf<T>::value;
  const T* x = static_cast<const T*>(x_);
  T* y = static_cast<T*>(y_);
  // 16-byte accesses need no pointer alignment beyond the element's
  const RowsRoute route = route_rows(RowsKind::kFwd, !affine, VEC, n_rows, D);
  if (route.small) {
    return affine ? small_fwd_launch<T, true>(x, gamma, beta, n_rows, D, C, eps, y, mean, rstd, st)
                  : small_fwd_launch<T, false>(x, gamma, beta, n_rows, D, C, eps, y, mean, rstd, st);
  }
  if (route.tiles) {
    return tiles_fwd<T>(x, gamma, beta, n_rows, D, eps, y, mean, rstd, ws, ws_bytes, st);
  }
  if (route.V > 1) {
    return affine ? rows_fwd_v<T, VEC, true>(x, gamma, beta, n_rows, D, C, eps, y, mean, rstd, ws, ws_bytes, st)
                  : rows_fwd_v<T, VEC, false>(x, gamma, beta, n_rows, D, C, eps, y, mean, rstd, ws, ws_bytes, st);
  }
  return affine ? rows_fwd_v<T, 1, true>(x, gamma, beta, n_rows, D, C, eps, y, mean, rstd, ws, ws_bytes, st)
                : rows_fwd_v<T, 1, false>(x, gamma, beta, n_rows, D, C, eps, y, mean, rstd, ws, ws_bytes, st);
}

template <typename T>
int rows_bwd_t(bool affine, const void* dy_, const void* x_, const float* gamma, const float* mean,
               const float* rstd, int64_t n_rows, int64_t D, int C, void* dx_, float* dgamma,
               float* dbeta, void* ws, size_t ws_bytes, hipStream_t st) {
  constexpr int VEC = VecOf<T>::value;
  const T* x = static_cast<const T*>(x_);
  const T* dy = static_cast<const T*>(dy_);
  T* dx = static_cast<T*>(dx_);
  const RowsRoute route =
      route_rows(affine ? RowsKind::kBwdAffine : RowsKind::kBwdCols, !affine, VEC, n_rows, D);
  if (route.small) {
    return affine ? small_bwd_launch<T, true>(dy, x, gamma, mean, rstd, n_rows, D, C, dx, dgamma, dbeta, ws, ws_bytes, st)
                  : small_bwd_launch<T, false>(dy, x, gamma, mean, rstd, n_rows, D, C, dx, dgamma, dbeta, ws, ws_bytes, st);
  }
  if (route.tiles) {
    return tiles_bwd<T>(dy, x, gamma, mean, rstd, n_rows, D, dx, dgamma, dbeta, ws, ws_bytes, st);
  }
  if (route.V > 1) {
    return affine ? rows_bwd_v<T, VEC, true>(dy, x, gamma, mean, rstd, n_rows, D, C, dx, dgamma, dbeta, ws, ws_bytes, st)
                  : rows_bwd_v<T, VEC, false>(dy, x, gamma, mean, rstd, n_rows, D, C, dx, dgamma, dbeta, ws, ws_bytes, st);
  }
  return affine ? rows_bwd_v<T, 1, true>(dy, x, gamma, mean, rstd, n_rows, D, C, dx, dgamma, dbeta, ws, ws_bytes, st)
                : rows_bwd_v<T, 1, false>(dy, x, gamma, mean, rstd, n_rows, D, C, dx, dgamma, dbeta, ws, ws_bytes, st);
}

#define ATEXN_INSTANTIATE_ROWS(T)                                                              \
  template int rows_fwd_t<T>(bool, const void*, const float*, const float*, int64_t, int64_t,  \
                             int, float, void*, float*, float*, void*, size_t, hipStream_t);   \
  template int rows_bwd_t<T>(bool, const void*, const void*, const float*, const float*,       \
                             const float*, int64_t, int64_t, int, void*, float*, float*, void*, \
                             size_t, hipStream_t);

}  // namespace atexn
