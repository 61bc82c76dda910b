// dtype dispatch, shared helper kernels, error state and tunables.
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstdarg>
#include <cstdio>
#include <cstring>

#include "norm_common.hip.h"
#include "plan.h"
#include "rows_kernels.hip.h"
#include "status.h"

namespace atexn {

// --------------------------------------------------------------------- error state
namespace {
thread_local char g_last_error[512] = "";
}

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

const char* last_error() { return g_last_error; }

#ifdef ATEXN_BENCH_BUILD
Tuning& tuning() {
  static Tuning t;
  return t;
}
#else
const Tuning& tuning() {
  static const Tuning t;
  return t;
}
#endif

unsigned next_call_tag() {
  static std::atomic<unsigned> counter{
      static_cast<unsigned>(std::chrono::steady_clock::now().time_since_epoch().count()) | 1u};
  unsigned t = counter.fetch_add(1, std::memory_order_relaxed);
  return t == 0 ? counter.fetch_add(1, std::memory_order_relaxed) : t;
}

bool exchange_allowed(void* st) {
  static const bool disabled = [] {
    const char* v = std::getenv("ATEXN_NO_EXCHANGE");
    return v != nullptr && v[0] != '\0' && !(v[0] == '0' && v[1] == '\0');
  }();
  if (disabled) return false;
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(static_cast<hipStream_t>(st), &status) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return status == hipStreamCaptureStatusNone;
}

namespace {
// tag of the last call on this device in which a patient wait for a peer's results ran out
__device__ unsigned g_exchange_trouble;
}  // namespace

unsigned* exchange_trouble_word() {
  static std::atomic<unsigned*> cached[64];
  static std::atomic<bool> failed[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return nullptr;
  }
  unsigned* p = cached[dev].load(std::memory_order_acquire);
  if (p != nullptr || failed[dev].load(std::memory_order_relaxed)) return p;
  void* q = nullptr;
  if (hipGetSymbolAddress(&q, HIP_SYMBOL(g_exchange_trouble)) != hipSuccess || q == nullptr) {
    (void)hipGetLastError();
    failed[dev].store(true, std::memory_order_relaxed);
    return nullptr;
  }
  // (racing threads look the same address up: the stores agree)
  cached[dev].store(static_cast<unsigned*>(q), std::memory_order_release);
  return static_cast<unsigned*>(q);
}

int cu_count() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    (void)hipGetLastError();
    return 256;
  }
  int v = cached[dev].load(std::memory_order_relaxed);
  if (v > 0) return v;
  int cus = 0;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
      cus <= 0) {
    (void)hipGetLastError();
    return 256;
  }
  cached[dev].store(cus, std::memory_order_relaxed);
  return cus;
}

// --------------------------------------------------------------------- small kernels
__global__ void fill_zero_kernel(float* out, int64_t n) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    out[i] = 0.f;
  }
}

int fill_zero(float* out, int64_t n, hipStream_t st) {
  if (n <= 0) return ATEXN_OK;
  const int grid = static_cast<int>(std::min<int64_t>(div_up(n, 256), 1024));
  fill_zero_kernel<<<grid, 256, 0, st>>>(out, n);
  ATEXN_CHECK_LAUNCH("fill_zero");
  return ATEXN_OK;
}

int launch_col_reduce(const float* part, float* out0, float* out1, int G, int64_t W,
                      hipStream_t st, int batch, int64_t part_stride, int64_t out_stride) {
  ATEXN_REQUIRE(2 * W < (int64_t(1) << 31), "column count %lld too large", (long long)W);
  const int Wi = static_cast<int>(W);
  // Column groups per block (CX): the more, the longer the contiguous run a wave reads per
  // partial row, but the fewer blocks and the fewer rows in parallel (256 / CX).  Take the
  // largest CX that still gives every CU a block and every row-lane at least two rows.
  const int cus = cu_count();
  auto fits = [&](int cw, int cx) {
    return div_up(2 * W, int64_t(cw) * cx) * batch >= cus && (256 / cx) * 2 <= std::max(G, 2);
  };
#define ATEXN_COL_REDUCE(CW_, CX_)                                                              \
  col_reduce<CW_, CX_><<<dim3(static_cast<unsigned>(div_up(2 * W, int64_t(CW_) * CX_)), batch),  \
                         kColReduceThreads, 0, st>>>(part, out0, out1, G, Wi, part_stride,      \
                                                     out_stride)
  if (W % 4 == 0) {
    if (fits(4, 256) || G < 8) {
      ATEXN_COL_REDUCE(4, 256);
    } else if (fits(4, 64)) {
      ATEXN_COL_REDUCE(4, 64);
    } else if (fits(4, 16)) {
      ATEXN_COL_REDUCE(4, 16);
    } else {
      ATEXN_COL_REDUCE(4, 4);
    }
  } else {
    if (fits(1, 256) || G < 8) {
      ATEXN_COL_REDUCE(1, 256);
    } else {
      ATEXN_COL_REDUCE(1, 16);
    }
  }
#undef ATEXN_COL_REDUCE
  ATEXN_CHECK_LAUNCH("col_reduce");
  return ATEXN_OK;
}

// --------------------------------------------------------------------- dtype dispatch
template <typename T>
int rows_fwd_t(bool, const void*, const float*, const float*, int64_t, int64_t, int, float, void*,
               float*, float*, void*, size_t, hipStream_t);
template <typename T>
int rows_bwd_t(bool, const void*, const void*, const float*, const float*, const float*, int64_t,
               int64_t, int, void*, float*, float*, void*, size_t, hipStream_t);
template <typename T>
int cl_fwd_t(const void*, const float*, const float*, int64_t, int64_t, int64_t, float, void*,
             float*, float*, void*, size_t, hipStream_t);
template <typename T>
int cl_bwd_t(const void*, const void*, const float*, const float*, const float*, int64_t, int64_t,
             int64_t, void*, float*, float*, void*, size_t, hipStream_t);

extern template int rows_fwd_t<float>(bool, const void*, const float*, const float*, int64_t, int64_t, int, float, void*, float*, float*, void*, size_t, hipStream_t);
extern template int rows_fwd_t<f16_t>(bool, const void*, const float*, const float*, int64_t, int64_t, int, float, void*, float*, float*, void*, size_t, hipStream_t);
extern template int rows_fwd_t<bf16_t>(bool, const void*, const float*, const float*, int64_t, int64_t, int, float, void*, float*, float*, void*, size_t, hipStream_t);
extern template int rows_bwd_t<float>(bool, const void*, const void*, const float*, const float*, const float*, int64_t, int64_t, int, void*, float*, float*, void*, size_t, hipStream_t);
extern template int rows_bwd_t<f16_t>(bool, const void*, const void*, const float*, const float*, const float*, int64_t, int64_t, int, void*, float*, float*, void*, size_t, hipStream_t);
extern template int rows_bwd_t<bf16_t>(bool, const void*, const void*, const float*, const float*, const float*, int64_t, int64_t, int, void*, float*, float*, void*, size_t, hipStream_t);
extern template int cl_fwd_t<float>(const void*, const float*, const float*, int64_t, int64_t, int64_t, float, void*, float*, float*, void*, size_t, hipStream_t);
extern template int cl_fwd_t<f16_t>(const void*, const float*, const float*, int64_t, int64_t, int64_t, float, void*, float*, float*, void*, size_t, hipStream_t);
extern template int cl_fwd_t<bf16_t>(const void*, const float*, const float*, int64_t, int64_t, int64_t, float, void*, float*, float*, void*, size_t, hipStream_t);
extern template int cl_bwd_t<float>(const void*, const void*, const float*, const float*, const float*, int64_t, int64_t, int64_t, void*, float*, float*, void*, size_t, hipStream_t);
extern template int cl_bwd_t<f16_t>(const void*, const void*, const float*, const float*, const float*, int64_t, int64_t, int64_t, void*, float*, float*, void*, size_t, hipStream_t);
extern template int cl_bwd_t<bf16_t>(const void*, const void*, const float*, const float*, const float*, int64_t, int64_t, int64_t, void*, float*, float*, void*, size_t, hipStream_t);

#define ATEXN_DISPATCH(dtype, CALL)                                        \
  switch (dtype) {                                                         \
    case ATEXN_F32: { using T = float; return CALL; }                      \
    case ATEXN_F16: { using T = f16_t; return CALL; }                      \
    case ATEXN_BF16: { using T = bf16_t; return CALL; }                    \
    default: return set_error(ATEXN_INVALID_ARGUMENT, "bad dtype %d", dtype); \
  }

int rows_fwd(int dtype, bool affine, const void* x, const float* gamma, const float* beta,
             int64_t n_rows, int64_t D, int C, float eps, void* y, float* mean, float* rstd,
             void* ws, size_t ws_bytes, hipStream_t st) {
  ATEXN_DISPATCH(dtype, rows_fwd_t<T>(affine, x, gamma, beta, n_rows, D, C, eps, y, mean, rstd, ws, ws_bytes, st));
}
int rows_bwd(int dtype, bool affine, const void* dy, const void* x, const float* gamma,
             const float* mean, const float* rstd, int64_t n_rows, int64_t D, int C, void* dx,
             float* dgamma, float* dbeta, void* ws, size_t ws_bytes, hipStream_t st) {
  ATEXN_DISPATCH(dtype, rows_bwd_t<T>(affine, dy, x, gamma, mean, rstd, n_rows, D, C, dx, dgamma, dbeta, ws, ws_bytes, st));
}
int cl_fwd(int dtype, const void* x, const float* gamma, const float* beta, int64_t N, int64_t C,
           int64_t D, float eps, void* y, float* mean, float* rstd, void* ws, size_t ws_bytes,
           hipStream_t st) {
  ATEXN_DISPATCH(dtype, cl_fwd_t<T>(x, gamma, beta, N, C, D, eps, y, mean, rstd, ws, ws_bytes, st));
}
int cl_bwd(int dtype, const void* dy, const void* x, const float* gamma, const float* mean,
           const float* rstd, int64_t N, int64_t C, int64_t D, void* dx, float* dgamma,
           float* dbeta, void* ws, size_t ws_bytes, hipStream_t st) {
  ATEXN_DISPATCH(dtype, cl_bwd_t<T>(dy, x, gamma, mean, rstd, N, C, D, dx, dgamma, dbeta, ws, ws_bytes, st));
}

// Workspace: the same choice of path as the launchers make (it depends on sizes only).
static size_t rows_ws(RowsKind kind, int dtype, int64_t n_rows, int64_t D, int C) {
  if (n_rows <= 0 || D <= 0) return 0;
  const int vec = 16 / elem_size(dtype);
  const int cus = cu_count();
  const bool layer_norm = C == 0;
  const RowsRoute r = route_rows(kind, layer_norm, vec, n_rows, D);
  if (r.small) return plan_small(kind, r.V, n_rows, D, C, cus).ws_bytes;
  if (r.tiles) return plan_tiles(kind != RowsKind::kFwd, vec, n_rows, D, cus).ws_bytes;
  return plan_rows(kind, r.V, n_rows, D, C, cus).ws_bytes;
}
size_t rows_fwd_ws(int dtype, bool affine, int64_t n_rows, int64_t D, int C) {
  return rows_ws(RowsKind::kFwd, dtype, n_rows, D, affine ? C : 0);
}
size_t rows_bwd_ws(int dtype, bool affine, int64_t n_rows, int64_t D, int C) {
  return rows_ws(affine ? RowsKind::kBwdAffine : RowsKind::kBwdCols, dtype, n_rows, D, affine ? C : 0);
}
static size_t cl_ws(bool bwd, int dtype, int64_t N, int64_t C, int64_t D) {
  if (N <= 0 || C <= 0 || D <= 0) return 0;
  const int vec = 16 / elem_size(dtype);
  return plan_cl(bwd, C >= vec ? vec : 1, N, C, D, cu_count()).ws_bytes;
}
size_t cl_fwd_ws(int dtype, int64_t N, int64_t C, int64_t D) { return cl_ws(false, dtype, N, C, D); }
size_t cl_bwd_ws(int dtype, int64_t N, int64_t C, int64_t D) { return cl_ws(true, dtype, N, C, D); }

}  // namespace atexn
