// Device-side building blocks shared by the LayerNorm / InstanceNorm kernels
// (gfx950, wave64).  Counterpart of the reference's norm_util.h:29-180 (Pack / Load /
// Store / Copy*), norm_util.h:182-211 (Welford merge) and norm_util.h:423-464
// (warp / block reductions), redesigned for 64-lane wavefronts, 128-bit accesses and
// register-resident rows.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace atexn {

constexpr int kWave = 64;

using f16_t = _Float16;
using bf16_t = __bf16;

// Number of storage elements in one 128-bit access.
template <typename T>
struct VecOf {
  static constexpr int value = 16 / sizeof(T);
};

// V storage elements moved by one load / store instruction (V * sizeof(T) is 16 bytes
// on the vector paths and sizeof(T) on the element-wise paths).
template <typename T, int V>
struct alignas(sizeof(T) * V) Pack {
  T v[V];
};

template <typename T, int V>
__device__ __forceinline__ Pack<T, V> load_pack(const T* p) {
  return *reinterpret_cast<const Pack<T, V>*>(p);
}
template <typename T, int V>
__device__ __forceinline__ void store_pack(T* p, const Pack<T, V>& v) {
  *reinterpret_cast<Pack<T, V>*>(p) = v;
}

template <typename T>
__device__ __forceinline__ float to_f32(T v) {
  return static_cast<float>(v);
}
template <typename T>
__device__ __forceinline__ T from_f32(float v) {
  return static_cast<T>(v);  // round-to-nearest-even for f16 / bf16
}

// V consecutive fp32 values (gamma, beta, saved statistics, partial sums).
template <int V>
__device__ __forceinline__ void load_f32(const float* p, float (&out)[V]) {
  if constexpr (V % 4 == 0) {
#pragma unroll
    for (int i = 0; i < V; i += 4) {
      float4 t = *reinterpret_cast<const float4*>(p + i);
      out[i] = t.x;
      out[i + 1] = t.y;
      out[i + 2] = t.z;
      out[i + 3] = t.w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) out[i] = p[i];
  }
}
template <int V>
__device__ __forceinline__ void store_f32(float* p, const float (&in)[V]) {
  if constexpr (V % 4 == 0) {
#pragma unroll
    for (int i = 0; i < V; i += 4) {
      *reinterpret_cast<float4*>(p + i) = make_float4(in[i], in[i + 1], in[i + 2], in[i + 3]);
    }
  } else {
#pragma unroll
    for (int i = 0; i < V; ++i) p[i] = in[i];
  }
}

// ------------------------------------------------------------------ cross-lane
// Exchange with the lane whose id differs in bit `mask` (butterfly step).
__device__ __forceinline__ float lane_xor(float v, int mask) { return __shfl_xor(v, mask, kWave); }

// Butterfly all-reduce (sum) over aligned groups of `width` lanes, width a power of two
// <= 64.  Every lane of the group ends with the same bits.
template <int WIDTH>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int m = WIDTH / 2; m > 0; m >>= 1) v += lane_xor(v, m);
  return v;
}

// ------------------------------------------------------------------- Welford
// (mean, m2 = sum of squared deviations, n) of a set; merge is Chan's pairwise update
// (reference: norm_util.h:190-210).  The merge is written to be bitwise symmetric in
// its arguments so that a butterfly leaves identical values in every lane.
struct Wf {
  float mean, m2, n;
};

__device__ __forceinline__ Wf wf_merge(const Wf& a, const Wf& b) {
#pragma clang fp contract(off)
  Wf r;
  r.n = a.n + b.n;
  const float inv = r.n > 0.f ? 1.0f / r.n : 0.f;
  const float d = b.mean - a.mean;
  const float wa = a.mean * a.n;
  const float wb = b.mean * b.n;
  r.mean = (wa + wb) * inv;
  const float nn = a.n * b.n;
  r.m2 = (a.m2 + b.m2) + (d * d) * (nn * inv);
  return r;
}

template <int WIDTH>
__device__ __forceinline__ Wf group_wf(Wf w) {
#pragma unroll
  for (int m = WIDTH / 2; m > 0; m >>= 1) {
    Wf o;
    o.mean = lane_xor(w.mean, m);
    o.m2 = lane_xor(w.m2, m);
    o.n = lane_xor(w.n, m);
    w = wf_merge(w, o);
  }
  return w;
}

// Block-wide Welford all-reduce for blocks that are a whole number of waves.  `buf`
// must hold 16 Wf entries and be private to this call until the block has passed
// another barrier (callers alternate between two buffers).
__device__ __forceinline__ Wf block_wf(Wf w, Wf* buf) {
  w = group_wf<kWave>(w);
  const int nw = blockDim.x / kWave;
  if (nw == 1) return w;
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) buf[wave] = w;
  __syncthreads();
  Wf r = buf[0];
  for (int i = 1; i < nw; ++i) r = wf_merge(r, buf[i]);
  return r;
}

// Block-wide all-reduce of two sums, same contract as block_wf (`buf` holds 16 float2).
__device__ __forceinline__ float2 block_sum2(float a, float b, float2* buf) {
  a = group_sum<kWave>(a);
  b = group_sum<kWave>(b);
  const int nw = blockDim.x / kWave;
  if (nw == 1) return make_float2(a, b);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) buf[wave] = make_float2(a, b);
  __syncthreads();
  float2 r = buf[0];
  for (int i = 1; i < nw; ++i) {
    r.x += buf[i].x;
    r.y += buf[i].y;
  }
  return r;
}

// Statistics of the V*NV register-resident values of one thread (exact two-pass, the
// data is on chip), as a Welford triple.  valid[k] tells whether vector k is inside the
// row; elements of a valid vector are all valid.
template <int N>
__device__ __forceinline__ Wf local_wf(const float (&f)[N], int n_valid) {
  Wf w;
  w.n = static_cast<float>(n_valid);
  if (n_valid == 0) {
    w.mean = 0.f;
    w.m2 = 0.f;
    return w;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) s += (i < n_valid) ? f[i] : 0.f;
  w.mean = s / w.n;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    const float d = f[i] - w.mean;
    q += (i < n_valid) ? d * d : 0.f;
  }
  w.m2 = q;
  return w;
}

}  // namespace atexn
