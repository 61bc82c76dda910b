// Kernels for channels-last InstanceNorm, x viewed as [N, D, C] (D = product of the
// spatial dims).  They replace the reference's channel-last ladder
//   forward   fused_instance_norm_op.cu:23-101 (ToTemp / TempToOut), :774-818 (update),
//             :1066-1165 (smem variant)
//   backward  fused_instance_norm_op.cu:666-730, :103-146, :732-772
// The reference maps one channel to a lane (2-byte loads for fp16, a grid of
// DivUp(C,32) x ppr x N blocks).  Here a lane owns one 128-bit vector of V adjacent
// channels, TPP lanes cover a pixel, and a block of 256 threads sweeps 256 / TPP pixels
// per step, so every wave-load is a contiguous 1 KiB.  The spatial extent of one
// instance is cut into S slabs, one block per (n, slab, channel tile):
//   stage 1 writes per-slab per-channel partials, stage 2 merges them and applies.
#pragma once

#include "norm_common.cuh"

namespace atexn {

constexpr int kClThreads = 256;

// Thread geometry.  TPP: threads per pixel (power of two, <= 256).
struct ClGeom {
  int64_t n;      // instance
  int s;          // slab
  int cvi;        // channel-vector index of this thread
  int slot;       // pixel slot inside the block
  int ppb;        // pixel slots per block
  bool ch_ok;     // channel vector inside C
  int64_t p0, p1; // pixel range of the slab
};

__device__ __forceinline__ ClGeom cl_geom(int64_t work, int S, int CT, int TPP, int CV,
                                          int64_t D, int64_t slab_len) {
  ClGeom g;
  const int ct = static_cast<int>(work % CT);
  const int64_t ns = work / CT;
  g.s = static_cast<int>(ns % S);
  g.n = ns / S;
  g.cvi = ct * TPP + static_cast<int>(threadIdx.x) % TPP;
  g.slot = static_cast<int>(threadIdx.x) / TPP;
  g.ppb = kClThreads / TPP;
  g.ch_ok = g.cvi < CV;
  g.p0 = static_cast<int64_t>(g.s) * slab_len;
  g.p1 = g.p0 + slab_len < D ? g.p0 + slab_len : D;
  return g;
}

// Sum K per-thread values over all threads of the block that own the same channels
// (same threadIdx.x % TPP).  Every such thread ends with the same total, added in a
// fixed order.  lds: K * 256 floats.  Ends with a barrier-protected state: the caller
// must __syncthreads() before reusing lds.
template <int K>
__device__ __forceinline__ void cl_block_sum(float (&v)[K], float* lds, int TPP) {
  for (int m = TPP; m < kWave; m <<= 1) {
#pragma unroll
    for (int i = 0; i < K; ++i) v[i] += lane_xor(v[i], m);
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  constexpr int NW = kClThreads / kWave;
  const int wpc = TPP > kWave ? TPP / kWave : 1;  // waves per channel sweep
  if (wpc == NW) return;                           // TPP == 256: nothing to fold
#pragma unroll
  for (int i = 0; i < K; ++i) lds[(i * NW + wave) * kWave + lane] = v[i];
  __syncthreads();
#pragma unroll
  for (int i = 0; i < K; ++i) {
    float s = lds[(i * NW + (wave % wpc)) * kWave + lane];
    for (int w = (wave % wpc) + wpc; w < NW; w += wpc) s += lds[(i * NW + w) * kWave + lane];
    v[i] = s;
  }
}

// Same for per-channel Welford triples (V channels sharing one count).  lds: (2V+1)*256.
template <int V>
__device__ __forceinline__ void cl_block_wf(float (&mean)[V], float (&m2)[V], float& cnt,
                                            float* lds, int TPP) {
  for (int m = TPP; m < kWave; m <<= 1) {
    const float ocnt = lane_xor(cnt, m);
    float ncnt = cnt;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      Wf a{mean[i], m2[i], cnt};
      Wf b{lane_xor(mean[i], m), lane_xor(m2[i], m), ocnt};
      Wf r = wf_merge(a, b);
      mean[i] = r.mean;
      m2[i] = r.m2;
      ncnt = r.n;
    }
    cnt = ncnt;
  }
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  constexpr int NW = kClThreads / kWave;
  const int wpc = TPP > kWave ? TPP / kWave : 1;
  if (wpc == NW) return;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    lds[((2 * i) * NW + wave) * kWave + lane] = mean[i];
    lds[((2 * i + 1) * NW + wave) * kWave + lane] = m2[i];
  }
  lds[((2 * V) * NW + wave) * kWave + lane] = cnt;
  __syncthreads();
  const int w0 = wave % wpc;
  float c0 = lds[((2 * V) * NW + w0) * kWave + lane];
  float cend = c0;
#pragma unroll
  for (int i = 0; i < V; ++i) {
    Wf r{lds[((2 * i) * NW + w0) * kWave + lane], lds[((2 * i + 1) * NW + w0) * kWave + lane], c0};
    for (int w = w0 + wpc; w < NW; w += wpc) {
      Wf o{lds[((2 * i) * NW + w) * kWave + lane], lds[((2 * i + 1) * NW + w) * kWave + lane],
           lds[((2 * V) * NW + w) * kWave + lane]};
      r = wf_merge(r, o);
    }
    mean[i] = r.mean;
    m2[i] = r.m2;
    cend = r.n;
  }
  cnt = cend;
}

// ---------------------------------------------------------------- forward, stage 1
// pmean / pm2: [N * S, C] partial mean and sum of squared deviations of each slab.
template <typename T, int V>
__global__ void cl_fwd_stats(const T* __restrict__ x, float* __restrict__ pmean,
                             float* __restrict__ pm2, int64_t n_work, int64_t D, int C, int S,
                             int CT, int TPP, int64_t slab_len) {
  __shared__ float lds[(2 * V + 1) * kClThreads];
  const int CV = (C + V - 1) / V;
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x) {
    const ClGeom g = cl_geom(w, S, CT, TPP, CV, D, slab_len);
    float mean[V], m2[V], cnt = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) mean[i] = m2[i] = 0.f;
    if (g.ch_ok) {
      const T* base = x + (g.n * D) * C + static_cast<int64_t>(g.cvi) * V;
      for (int64_t p = g.p0 + g.slot; p < g.p1; p += g.ppb) {
        Pack<T, V> pk = load_pack<T, V>(base + p * C);
        cnt += 1.f;
        const float inv = 1.0f / cnt;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const float f = to_f32(pk.v[i]);
          const float d = f - mean[i];
          mean[i] += d * inv;
          m2[i] += d * (f - mean[i]);
        }
      }
    }
    cl_block_wf<V>(mean, m2, cnt, lds, TPP);
    if (g.ch_ok && g.slot == 0) {
      const int64_t o = (g.n * S + g.s) * C + static_cast<int64_t>(g.cvi) * V;
      store_f32<V>(pmean + o, mean);
      store_f32<V>(pm2 + o, m2);
    }
    __syncthreads();  // lds is reused by the next work item
  }
}

// ---------------------------------------------------------------- forward, stage 2
// y may alias x: stage 1 has completed (it is an earlier launch on the same stream) and
// every thread reads a vector before it writes the same vector.
template <typename T, int V>
__global__ void cl_fwd_apply(const T* x, const float* __restrict__ pmean,
                             const float* __restrict__ pm2, const float* __restrict__ gamma,
                             const float* __restrict__ beta, T* y,
                             float* __restrict__ mean_out, float* __restrict__ rstd_out,
                             int64_t n_work, int64_t D, int C, int S, int CT, int TPP,
                             int64_t slab_len, float eps) {
  __shared__ float lds[(2 * V + 1) * kClThreads];
  const int CV = (C + V - 1) / V;
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x) {
    const ClGeom g = cl_geom(w, S, CT, TPP, CV, D, slab_len);
    float mean[V], m2[V], cnt = 0.f;
#pragma unroll
    for (int i = 0; i < V; ++i) mean[i] = m2[i] = 0.f;
    if (g.ch_ok) {
      // every pixel slot merges its share of the slab partials
      for (int s = g.slot; s < S; s += g.ppb) {
        const int64_t o = (g.n * S + s) * C + static_cast<int64_t>(g.cvi) * V;
        const int64_t b0 = static_cast<int64_t>(s) * slab_len;
        const float len = static_cast<float>((b0 + slab_len < D ? b0 + slab_len : D) - b0);
        float pm[V], pq[V];
        load_f32<V>(pmean + o, pm);
        load_f32<V>(pm2 + o, pq);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          Wf r = wf_merge(Wf{mean[i], m2[i], cnt}, Wf{pm[i], pq[i], len});
          mean[i] = r.mean;
          m2[i] = r.m2;
        }
        cnt += len;
      }
    }
    cl_block_wf<V>(mean, m2, cnt, lds, TPP);
    if (g.ch_ok) {
      float gm[V], bt[V], rs[V];
      load_f32<V>(gamma + static_cast<int64_t>(g.cvi) * V, gm);
      load_f32<V>(beta + static_cast<int64_t>(g.cvi) * V, bt);
#pragma unroll
      for (int i = 0; i < V; ++i) rs[i] = rsqrtf(m2[i] / static_cast<float>(D) + eps);
      if (g.s == 0 && g.slot == 0) {
        store_f32<V>(mean_out + g.n * C + static_cast<int64_t>(g.cvi) * V, mean);
        store_f32<V>(rstd_out + g.n * C + static_cast<int64_t>(g.cvi) * V, rs);
      }
      const int64_t boff = (g.n * D) * C + static_cast<int64_t>(g.cvi) * V;
      for (int64_t p = g.p0 + g.slot; p < g.p1; p += g.ppb) {
        Pack<T, V> pk = load_pack<T, V>(x + boff + p * C);
        Pack<T, V> o;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          // subtract the mean first: x * scale - mean * scale would cancel badly when
          // |mean| >> std
          o.v[i] = from_f32<T>((to_f32(pk.v[i]) - mean[i]) * rs[i] * gm[i] + bt[i]);
        }
        store_pack<T, V>(y + boff + p * C, o);
      }
    }
    __syncthreads();
  }
}

// --------------------------------------------------------------- backward, stage 1
// part[(n * S + s)][0][c] = sum dy * xh, part[...][1][c] = sum dy over the slab.
template <typename T, int V>
__global__ void cl_bwd_sums(const T* __restrict__ dy, const T* __restrict__ x,
                            const float* __restrict__ mean_in,
                            const float* __restrict__ rstd_in, float* __restrict__ part,
                            int64_t n_work, int64_t D, int C, int S, int CT, int TPP,
                            int64_t slab_len) {
  __shared__ float lds[2 * V * kClThreads];
  const int CV = (C + V - 1) / V;
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x) {
    const ClGeom g = cl_geom(w, S, CT, TPP, CV, D, slab_len);
    float acc[2 * V];
#pragma unroll
    for (int i = 0; i < 2 * V; ++i) acc[i] = 0.f;
    if (g.ch_ok) {
      float mu[V], rs[V];
      load_f32<V>(mean_in + g.n * C + static_cast<int64_t>(g.cvi) * V, mu);
      load_f32<V>(rstd_in + g.n * C + static_cast<int64_t>(g.cvi) * V, rs);
      const int64_t boff = (g.n * D) * C + static_cast<int64_t>(g.cvi) * V;
      for (int64_t p = g.p0 + g.slot; p < g.p1; p += g.ppb) {
        Pack<T, V> px = load_pack<T, V>(x + boff + p * C);
        Pack<T, V> pd = load_pack<T, V>(dy + boff + p * C);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const float d = to_f32(pd.v[i]);
          const float xh = (to_f32(px.v[i]) - mu[i]) * rs[i];
          acc[i] += d * xh;
          acc[V + i] += d;
        }
      }
    }
    cl_block_sum<2 * V>(acc, lds, TPP);
    if (g.ch_ok && g.slot == 0) {
      float* o = part + ((g.n * S + g.s) * 2) * C + static_cast<int64_t>(g.cvi) * V;
      float t0[V], t1[V];
#pragma unroll
      for (int i = 0; i < V; ++i) {
        t0[i] = acc[i];
        t1[i] = acc[V + i];
      }
      store_f32<V>(o, t0);
      store_f32<V>(o + C, t1);
    }
    __syncthreads();
  }
}

// --------------------------------------------------------------- backward, stage 2
// dx = r * gamma * (dy - (A + xh * B) / D) with A = sum dy, B = sum dy * xh over the
// whole (n, c) instance (norm_util.h:599-615 in s1 / s2 form).
template <typename T, int V>
__global__ void cl_bwd_apply(const T* __restrict__ dy, const T* __restrict__ x,
                             const float* __restrict__ gamma,
                             const float* __restrict__ mean_in,
                             const float* __restrict__ rstd_in,
                             const float* __restrict__ part, T* __restrict__ dx,
                             int64_t n_work, int64_t D, int C, int S, int CT, int TPP,
                             int64_t slab_len) {
  __shared__ float lds[2 * V * kClThreads];
  const int CV = (C + V - 1) / V;
  const float inv_d = 1.0f / static_cast<float>(D);
  for (int64_t w = blockIdx.x; w < n_work; w += gridDim.x) {
    const ClGeom g = cl_geom(w, S, CT, TPP, CV, D, slab_len);
    float acc[2 * V];
#pragma unroll
    for (int i = 0; i < 2 * V; ++i) acc[i] = 0.f;
    if (g.ch_ok) {
      for (int s = g.slot; s < S; s += g.ppb) {
        const float* o = part + ((g.n * S + s) * 2) * C + static_cast<int64_t>(g.cvi) * V;
        float t0[V], t1[V];
        load_f32<V>(o, t0);
        load_f32<V>(o + C, t1);
#pragma unroll
        for (int i = 0; i < V; ++i) {
          acc[i] += t0[i];
          acc[V + i] += t1[i];
        }
      }
    }
    cl_block_sum<2 * V>(acc, lds, TPP);
    if (g.ch_ok) {
      float mu[V], rs[V], gm[V];
      load_f32<V>(mean_in + g.n * C + static_cast<int64_t>(g.cvi) * V, mu);
      load_f32<V>(rstd_in + g.n * C + static_cast<int64_t>(g.cvi) * V, rs);
      load_f32<V>(gamma + static_cast<int64_t>(g.cvi) * V, gm);
      const int64_t boff = (g.n * D) * C + static_cast<int64_t>(g.cvi) * V;
      for (int64_t p = g.p0 + g.slot; p < g.p1; p += g.ppb) {
        Pack<T, V> px = load_pack<T, V>(x + boff + p * C);
        Pack<T, V> pd = load_pack<T, V>(dy + boff + p * C);
        Pack<T, V> o;
#pragma unroll
        for (int i = 0; i < V; ++i) {
          const float d = to_f32(pd.v[i]);
          const float xh = (to_f32(px.v[i]) - mu[i]) * rs[i];
          o.v[i] = from_f32<T>(rs[i] * gm[i] * (d - (acc[V + i] + xh * acc[i]) * inv_d));
        }
        store_pack<T, V>(dx + boff + p * C, o);
      }
    }
    __syncthreads();
  }
}

}  // namespace atexn
