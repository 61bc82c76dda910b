// Host (CPU) kernels of the four ops (cpu_kernels.cc).  dtype: 0 float, 1 half, 2 bfloat16
// (the values of ATEXN_F32 / F16 / BF16); every pointer is a host pointer; the calls are
// synchronous.  Return false for an unknown dtype.  Sizes are positive (callers handle the
// empty cases).
#pragma once

#include <stdint.h>

namespace atexn {
namespace cpu {

bool layer_norm_fwd(int dtype, const void* x, const float* gamma, const float* beta, int64_t N,
                    int64_t D, float eps, void* y, float* mean, float* rstd);
bool layer_norm_bwd(int dtype, const void* dy, const void* x, const float* gamma, const float* mean,
                    const float* rstd, int64_t N, int64_t D, void* dx, float* dgamma, float* dbeta);
bool instance_norm_fwd(int dtype, bool channel_first, const void* x, const float* gamma,
                       const float* beta, int64_t N, int64_t C, int64_t D, float eps, void* y,
                       float* mean, float* rstd);
bool instance_norm_bwd(int dtype, bool channel_first, const void* dy, const void* x,
                       const float* gamma, const float* mean, const float* rstd, int64_t N,
                       int64_t C, int64_t D, void* dx, float* dgamma, float* dbeta);

}  // namespace cpu
}  // namespace atexn
