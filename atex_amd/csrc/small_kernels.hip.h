// Rows of at most kSmallMaxVec vectors (D <= 32 halves / 16 floats): one THREAD per row.
// A wave covers 64 consecutive rows, so its accesses are contiguous in memory, every
// statistic is a private sum (no cross-lane traffic at all), and the only exchange is the
// fold of the per-column dgamma / dbeta accumulators at the end of the backward kernel.
// Replaces the reference's D < 32 kernels (fused_layer_norm_op.cu:446-481, :109-141,
// fused_instance_norm_op.cu:459-556).
//
// A row is read as NV vectors at element offsets off_j = min(j * V, D - V): when D is not a
// multiple of V the last vector overlaps the one before it and owns only its last D % V
// elements for the sums; outputs are written as whole vectors (the overlap is written
// twice by the same thread with the same values).  Needs D >= V.
#pragma once

#include "norm_common.hip.h"

namespace atexn {

constexpr int kSmallThreads = 256;
constexpr int kSmallMaxVec = 4;

template <int V, int NV>
struct SmallGeom {
  int off[NV];  // element offset of vector j in the row
  int lo[NV];   // first element of vector j that vector j owns
};
template <int V, int NV>
__device__ __forceinline__ SmallGeom<V, NV> small_geom(int D) {
  SmallGeom<V, NV> g;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int nominal = j * V;
    g.off[j] = nominal + V <= D ? nominal : D - V;
    g.lo[j] = nominal - g.off[j];
  }
  return g;
}

template <typename T, int V, int NV, bool ROW_AFFINE>
__global__ void __launch_bounds__(kSmallThreads)
small_fwd(const T* x, const float* __restrict__ gamma, const float* __restrict__ beta, T* y,
          float* __restrict__ mean_out, float* __restrict__ rstd_out, int64_t n_rows, int D, int C,
          float eps) {
  const SmallGeom<V, NV> g = small_geom<V, NV>(D);
  const float inv_d = 1.0f / static_cast<float>(D);
  float gm[NV][V], bt[NV][V];
  if constexpr (!ROW_AFFINE) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      load_f32<V>(gamma + g.off[j], gm[j]);
      load_f32<V>(beta + g.off[j], bt[j]);
    }
  }
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kSmallThreads;
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kSmallThreads + threadIdx.x; row < n_rows;
       row += stride) {
    const T* xr = x + row * D;
    Pack<T, V> pk[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) pk[j] = load_pack<T, V>(xr + g.off[j]);
    float gs = 1.f, bs = 0.f;
    if constexpr (ROW_AFFINE) {
      const int c = static_cast<int>(row % C);
      gs = gamma[c];
      bs = beta[c];
    }
    float f[NV][V];
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        f[j][i] = to_f32(pk[j].v[i]);
        s += i >= g.lo[j] ? f[j][i] : 0.f;
      }
    }
    const float mean = s * inv_d;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        f[j][i] -= mean;
        q += i >= g.lo[j] ? f[j][i] * f[j][i] : 0.f;
      }
    }
    const float rstd = rsqrtf(q * inv_d + eps);
    T* yr = y + row * D;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      Pack<T, V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        if constexpr (ROW_AFFINE) {
          o.v[i] = from_f32<T>(f[j][i] * (rstd * gs) + bs);
        } else {
          o.v[i] = from_f32<T>(f[j][i] * (rstd * gm[j][i]) + bt[j][i]);
        }
      }
      store_pack<T, V>(yr + g.off[j], o);
    }
    mean_out[row] = mean;
    rstd_out[row] = rstd;
  }
}

// Backward.  LayerNorm: part[blockIdx.x][0][0..D) / [1][0..D) get the block's dgamma / dbeta
// partial sums (col_reduce finishes); channel-first InstanceNorm: part[n][0][c] = sum dy * xh,
// part[n][1][c] = sum dy of row (n, c).  dx may alias dy, not x.
template <typename T, int V, int NV, bool ROW_AFFINE>
__global__ void __launch_bounds__(kSmallThreads)
small_bwd(const T* dy, const T* __restrict__ x, const float* __restrict__ gamma,
          const float* __restrict__ mean_in, const float* __restrict__ rstd_in, T* dx,
          float* __restrict__ part, int64_t n_rows, int D, int C) {
  constexpr int NWV = kSmallThreads / kWave;
  __shared__ float fold[NWV][2][NV * V];
  const SmallGeom<V, NV> g = small_geom<V, NV>(D);
  const float inv_d = 1.0f / static_cast<float>(D);
  float gm[NV][V], ag[NV][V], ab[NV][V];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    if constexpr (!ROW_AFFINE) load_f32<V>(gamma + g.off[j], gm[j]);
#pragma unroll
    for (int i = 0; i < V; ++i) ag[j][i] = ab[j][i] = 0.f;
  }
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kSmallThreads;
  for (int64_t row = static_cast<int64_t>(blockIdx.x) * kSmallThreads + threadIdx.x; row < n_rows;
       row += stride) {
    const T* xr = x + row * D;
    const T* dr = dy + row * D;
    Pack<T, V> px[NV], pd[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      px[j] = load_pack_last<T, V>(xr + g.off[j]);
      pd[j] = load_pack_last<T, V>(dr + g.off[j]);
    }
    const float mean = mean_in[row], rstd = rstd_in[row];
    float gs = 1.f;
    if constexpr (ROW_AFFINE) gs = gamma[static_cast<int>(row % C)];
    float xh[NV][V], gv[NV][V];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const bool own = i >= g.lo[j];
        const float h = (to_f32(px[j].v[i]) - mean) * rstd;
        const float d = to_f32(pd[j].v[i]);
        xh[j][i] = h;
        if constexpr (ROW_AFFINE) {
          gv[j][i] = d;
        } else {
          gv[j][i] = d * gm[j][i];
          ag[j][i] += own ? d * h : 0.f;
          ab[j][i] += own ? d : 0.f;
        }
        s1 += own ? gv[j][i] : 0.f;
        s2 += own ? gv[j][i] * h : 0.f;
      }
    }
    const float scale = rstd * gs;
    const float ca = -scale * (s2 * inv_d), cb = -scale * (s1 * inv_d);
    T* outr = dx + row * D;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      Pack<T, V> o;
#pragma unroll
      for (int i = 0; i < V; ++i) o.v[i] = from_f32<T>(scale * gv[j][i] + (ca * xh[j][i] + cb));
      store_pack<T, V>(outr + g.off[j], o);
    }
    if constexpr (ROW_AFFINE) {
      const int64_t n = row / C;
      const int c = static_cast<int>(row % C);
      part[(n * 2 + 0) * C + c] = s2;
      part[(n * 2 + 1) * C + c] = s1;
    }
  }
  if constexpr (!ROW_AFFINE) {
    // every thread holds sums for the same D columns: fold lanes, then the waves via LDS
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float a = group_sum<kWave>(ag[j][i]);
        const float b = group_sum<kWave>(ab[j][i]);
        if (lane == 0) {
          fold[wave][0][j * V + i] = a;
          fold[wave][1][j * V + i] = b;
        }
      }
    }
    __syncthreads();
    const int t = threadIdx.x;
    if (t < 2 * NV * V) {
      const int which = t / (NV * V);
      const int e = t % (NV * V);
      const int j = e / V, i = e % V;
      float s = fold[0][which][e];
#pragma unroll
      for (int w = 1; w < NWV; ++w) s += fold[w][which][e];
      // g.off / g.lo are indexed with a runtime j here: select instead of indexing
      int off = 0, lo = 0;
#pragma unroll
      for (int jj = 0; jj < NV; ++jj) {
        if (jj == j) {
          off = g.off[jj];
          lo = g.lo[jj];
        }
      }
      if (i >= lo) part[(static_cast<int64_t>(blockIdx.x) * 2 + which) * D + off + i] = s;
    }
  }
}

}  // namespace atexn
