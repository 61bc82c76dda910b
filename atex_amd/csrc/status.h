// Error reporting shared by every translation unit of libatex_norms_hip.so.
#pragma once

#include <hip/hip_runtime.h>

#include "../../include/atex_norms.h"

namespace atexn {

// Records a printf-style message for atexn_last_error() of this thread; returns `code`.
int set_error(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
const char* last_error();

// Number of compute units of the current device (256 on MI355X); 256 if no device can be
// queried, so that the workspace queries stay usable on a host without a GPU.
int cu_count();

// A tag that no earlier call of this process has used (never 0): the single-launch
// channels-last kernels mark the partial results they exchange with it, so that whatever an
// earlier call left in the caller's workspace is never taken for data of this one.  A
// process-wide atomic counter, started from the clock.
unsigned next_call_tag();

// Whether a call on stream `st` may take the kernels whose workgroups exchange partial results
// while they run.  Not while the stream is being captured (a graph replay would repeat the call's
// tag), and not in a process started with ATEXN_NO_EXCHANGE set to anything but "0": those
// kernels need the workgroups of one instance / plane on the chip together, which a process that
// keeps other kernels resident on the same GPU (communication kernels overlapped with compute)
// may never give them; every wait then runs out and every workgroup recomputes its peers' share.
// The results are the same; the time is not.  The variable is read once, at the first call.
bool exchange_allowed(void* st);

// The current device's word for exchange_polls / exchange_gave_up (norm_common.hip.h): a static
// device variable of the library, looked up once per device.  nullptr if that fails (the kernels
// then always wait patiently).
unsigned* exchange_trouble_word();

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define ATEXN_REQUIRE(cond, ...)                                                  \
  do {                                                                            \
    if (!(cond)) return ::atexn::set_error(ATEXN_INVALID_ARGUMENT, __VA_ARGS__);  \
  } while (0)

#define ATEXN_CHECK_LAUNCH(what)                                                           \
  do {                                                                                     \
    hipError_t e_ = hipGetLastError();                                                     \
    if (e_ != hipSuccess)                                                                  \
      return ::atexn::set_error(ATEXN_LAUNCH_ERROR, "%s: %s", what, hipGetErrorString(e_)); \
  } while (0)

// Flat entry points used by the C ABI (dtype already validated).
size_t rows_fwd_ws(int dtype, bool affine, int64_t n_rows, int64_t D, int C);
size_t rows_bwd_ws(int dtype, bool affine, int64_t n_rows, int64_t D, int C);
int rows_fwd(int dtype, bool affine, const void* x, const float* gamma, const float* beta,
             int64_t n_rows, int64_t D, int C, float eps, void* y, float* mean, float* rstd,
             void* ws, size_t ws_bytes, hipStream_t st);
int rows_bwd(int dtype, bool affine, const void* dy, const void* x, const float* gamma,
             const float* mean, const float* rstd, int64_t n_rows, int64_t D, int C, void* dx,
             float* dgamma, float* dbeta, void* ws, size_t ws_bytes, hipStream_t st);

size_t cl_fwd_ws(int dtype, int64_t N, int64_t C, int64_t D);
size_t cl_bwd_ws(int dtype, int64_t N, int64_t C, int64_t D);
int cl_fwd(int dtype, const void* x, const float* gamma, const float* beta, int64_t N, int64_t C,
           int64_t D, float eps, void* y, float* mean, float* rstd, void* ws, size_t ws_bytes,
           hipStream_t st);
int cl_bwd(int dtype, const void* dy, const void* x, const float* gamma, const float* mean,
           const float* rstd, int64_t N, int64_t C, int64_t D, void* dx, float* dgamma,
           float* dbeta, void* ws, size_t ws_bytes, hipStream_t st);

// out[0..n) = 0 on the stream (a kernel, so that callers may capture it in a HIP graph).
int fill_zero(float* out, int64_t n, hipStream_t st);

// Launches the deterministic column reduction out0[j] = sum_g part[g][0][j],
// out1[j] = sum_g part[g][1][j], j < W; `batch` independent problems at the given strides
// (in floats) in one launch.
int launch_col_reduce(const float* part, float* out0, float* out1, int G, int64_t W,
                      hipStream_t st, int batch = 1, int64_t part_stride = 0,
                      int64_t out_stride = 0);

inline int elem_size(int dtype) { return dtype == ATEXN_F32 ? 4 : 2; }

}  // namespace atexn
